"""Operand, result and attribute lists of the XLA-FFI custom calls, in binding order.

One table for both sides of the boundary: `_jax_op.py` builds its `ffi_call`s from these
lists, and `csrc/fa2_xla_ffi.cc` binds its handlers in the same order (a host-only test
parses the `Bind()` chains of that file and compares them with this module).  They take
the place of the positional operand lists of the reference's `triton_call`s
(_forward_triton.py:547-588, _backward_triton.py:1049-1154).

No jax import here: the module is importable without jax.
"""

# Absent optional operands are passed as 0-element buffers; a 0-element `dbias` result means
# "no bias gradient wanted".
FWD_OPERANDS = ("q", "k", "v", "bias", "seqlens", "kv_lens", "seed")
FWD_RESULTS = ("o", "lse", "scratch")
BWD_OPERANDS = ("q", "k", "v", "bias", "seqlens", "kv_lens", "seed", "o", "lse", "dout")
BWD_RESULTS = ("dq", "dk", "dv", "dbias", "scratch")

# (name, C++ type of the Attr<> binding); the same list for both handlers
ATTRS = (
	("scale", "float"),
	("dropout_p", "float"),
	("causal", "bool"),
	("bias_group", "bool"),
	("has_window", "bool"),
	("window_left", "int32_t"),
	("window_right", "int32_t"),
	("softcap", "float"),
)

MASK_OPERANDS = ("seed",)
MASK_RESULTS = ("keep",)
MASK_ATTRS = (("dropout_p", "float"),)

HANDLERS = {
	"fa2_fwd_ffi": (FWD_OPERANDS, FWD_RESULTS, ATTRS),
	"fa2_bwd_ffi": (BWD_OPERANDS, BWD_RESULTS, ATTRS),
	"fa2_dropout_mask_ffi": (MASK_OPERANDS, MASK_RESULTS, MASK_ATTRS),
}

# which field of fa2_params (include/fa2.h) each operand / attribute fills
PARAM_FIELDS = {
	"q": "q", "k": "k", "v": "v", "o": "o", "lse": "lse", "dout": "dout", "dq": "dq", "dk": "dk", "dv": "dv",
	"bias": "bias, bias_dtype (FA2_MASK_U8 for a boolean / byte buffer), bias_stride_*",
	"seqlens": "seqlens", "kv_lens": "kv_lens", "seed": "seed_dev", "scratch": "scratch, scratch_bytes",
	"dbias": "dbias, dbias_stride_*",
	"scale": "scale", "dropout_p": "p_drop", "causal": "causal", "bias_group": "bias_group",
	"has_window": "has_window", "window_left": "window_left", "window_right": "window_right", "softcap": "softcap",
}
