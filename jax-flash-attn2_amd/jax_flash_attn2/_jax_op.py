"""JAX spelling of the HIP attention operator: `jax.custom_vjp` around two XLA-FFI
custom calls into libfa2_hip.so.

Takes the place of `jax_flash_attn2/flash_attention_triton/_flash_attention.py:27-157`
of the reference (`_jax_fwd_attention_call`, `_jax_bwd_attention_call`,
`flash_attention_call`, `flash_attention`): same argument list, same static
arguments (softmax_scale, dropout_prob, causal, varlen_mode), same residuals
(q, k, v, bias, mask, out, lse, seed), gradients for q, k, v only.

The FFI handlers live in csrc/fa2_xla_ffi.cc (built into libfa2_xla_ffi.so with
`make -C csrc ffi XLA_FFI_INCLUDE=$(python -c "import jax; print(jax.ffi.include_dir())")`);
they forward to exactly the C entry points the ctypes path calls.

This module imports jax at import time and is only loaded when the caller
passes jax arrays.  The image this package is developed in has no jax, so the
module is exercised by reading only.
"""

from __future__ import annotations

import ctypes
import functools
import math
import os
import typing as tp

import jax
import jax.numpy as jnp
import numpy as np

from ._checks import check_shapes

_HERE = os.path.dirname(os.path.abspath(__file__))
FFI_LIB_PATH = os.path.join(os.path.dirname(_HERE), "libfa2_xla_ffi.so")

_ffi = getattr(jax, "ffi", None)
if _ffi is None:  # jax < 0.4.38
	import jax.extend.ffi as _ffi  # type: ignore

_registered = False


def _register():
	global _registered
	if _registered:
		return
	if not os.path.exists(FFI_LIB_PATH):
		raise ImportError(
			f"{FFI_LIB_PATH} is missing: build it with `make -C {os.path.join(os.path.dirname(_HERE), 'csrc')} ffi` "
			"(there is no non-HIP fallback for this path)"
		)
	lib = ctypes.CDLL(FFI_LIB_PATH)
	for name in ("fa2_fwd_ffi", "fa2_bwd_ffi", "fa2_dropout_mask_ffi"):
		_ffi.register_ffi_target(name, _ffi.pycapsule(getattr(lib, name)), platform="ROCM")
	_registered = True


def _absent(dtype):
	return jnp.zeros((0,), dtype)


def _prep(q, k, v, bias, attention_mask):
	"""Shape checks of `_fwd_attention_kernel_call` (_forward_triton.py:474-495); the 2-D
	right-padded mask becomes one length per batch row instead of a packed layout."""
	check_shapes(q, k, v, bias, attention_mask)
	seqlens = _absent(jnp.int32)
	if attention_mask is not None:
		if attention_mask.ndim != 2:
			raise ValueError("attention_mask must be a 2-D [batch, seq] right-padded validity mask; use bias for general masks")
		seqlens = (attention_mask != 0).sum(axis=1, dtype=jnp.int32)
	bias_group = False
	if bias is None:
		bias = _absent(q.dtype)
	else:
		if bias.dtype not in (jnp.float16, jnp.bfloat16, jnp.float32):
			bias = bias.astype(jnp.float32)
		bias_group = bias.shape[1] == k.shape[2] and k.shape[2] != q.shape[2] and bias.shape[1] != 1
	return bias, seqlens, bias_group


def _attrs(q, softmax_scale, dropout_prob, causal, bias_group):
	"""Attributes of the custom calls: compile-time constants only (the seed is an operand)."""
	scale = 1.0 / math.sqrt(q.shape[-1]) if softmax_scale is None else softmax_scale
	return dict(
		scale=np.float32(scale),
		dropout_p=np.float32(dropout_prob),
		causal=bool(causal),
		bias_group=bool(bias_group),
	)


def _seed_operand(dropout_seed):
	"""The dropout seed as the 8-byte operand of the custom calls: uint32[2], low word first.
	A Python int is split on the host; an array or tracer (the reference jits with a traced
	dropout_seed, _flash_attention.py:91-92) is split with array operations, so nothing is
	ever converted to a host scalar and one executable serves every seed."""
	if dropout_seed is None:
		return jnp.zeros((2,), jnp.uint32)
	if isinstance(dropout_seed, (int, np.integer)):
		s = int(dropout_seed) & 0xFFFFFFFFFFFFFFFF
		return jnp.array([s & 0xFFFFFFFF, s >> 32], dtype=jnp.uint32)
	x = jnp.asarray(dropout_seed).reshape(())
	if x.dtype.itemsize == 8:
		x = x.astype(jnp.uint64)
		return jnp.stack([(x & 0xFFFFFFFF).astype(jnp.uint32), (x >> 32).astype(jnp.uint32)])
	return jnp.stack([x.astype(jnp.uint32), jnp.zeros((), jnp.uint32)])


def _fwd_scratch_bytes(q, k) -> int:
	"""fa2_fwd_scratch_bytes for these shapes (host-only query; at least one aligned unit so the result is never empty)."""
	import ctypes

	from . import _lib

	p = _lib.new_params()
	p.B, p.Sq, p.Hq, p.D = (int(x) for x in q.shape)
	p.Sk, p.Hkv = int(k.shape[1]), int(k.shape[2])
	return max(int(_lib.load().fa2_fwd_scratch_bytes(ctypes.byref(p))), 256)


def _bwd_scratch_bytes(q, k, causal=False) -> int:
	"""Scratch of the backward for these shapes (host-only query): fa2_bwd_scratch_bytes, or the larger
	fa2_bwd_split_scratch_bytes where the dK/dV kernel can split a key tile's work over workgroups."""
	import ctypes

	from . import _lib

	p = _lib.new_params()
	p.B, p.Sq, p.Hq, p.D = (int(x) for x in q.shape)
	p.Sk, p.Hkv = int(k.shape[1]), int(k.shape[2])
	p.causal = 1 if causal else 0  # (causal launches split further: their key tiles differ in length)
	lib = _lib.load()
	return max(int(lib.fa2_bwd_scratch_bytes(ctypes.byref(p))), int(lib.fa2_bwd_split_scratch_bytes(ctypes.byref(p))), 256)


def _fwd_call(q, k, v, bias, seqlens, seed, attrs):
	_register()
	B, Sq, Hq, _ = q.shape
	out_types = (
		jax.ShapeDtypeStruct(q.shape, q.dtype),
		jax.ShapeDtypeStruct((B, Hq, Sq), jnp.float32),
		jax.ShapeDtypeStruct((_fwd_scratch_bytes(q, k),), jnp.uint8),
	)
	out, lse, _ = _ffi.ffi_call("fa2_fwd_ffi", out_types)(q, k, v, bias, seqlens, seed, **attrs)
	return out, lse


def _bwd_call(q, k, v, bias, seqlens, seed, out, lse, dout, attrs):
	_register()
	scratch_bytes = _bwd_scratch_bytes(q, k, attrs["causal"])
	out_types = (
		jax.ShapeDtypeStruct(q.shape, q.dtype),
		jax.ShapeDtypeStruct(k.shape, k.dtype),
		jax.ShapeDtypeStruct(v.shape, v.dtype),
		jax.ShapeDtypeStruct((scratch_bytes,), jnp.uint8),
	)
	dq, dk, dv, _ = _ffi.ffi_call("fa2_bwd_ffi", out_types)(q, k, v, bias, seqlens, seed, out, lse, dout, **attrs)
	return dq, dk, dv


# static: softmax_scale, dropout_prob, causal, varlen_mode (as in the reference, _flash_attention.py:119); dropout_seed
# (argument 8) is an ordinary operand and may be traced
@functools.partial(jax.custom_vjp, nondiff_argnums=(5, 6, 7, 9))
def flash_attention_call(q, k, v, attention_mask=None, bias=None, softmax_scale=None, dropout_prob=0.0, causal=False,
                         dropout_seed=None, varlen_mode=True):
	return _fwd_rule(q, k, v, attention_mask, bias, softmax_scale, dropout_prob, causal, dropout_seed, varlen_mode)[0]


def _fwd_rule(q, k, v, attention_mask, bias, softmax_scale, dropout_prob, causal, dropout_seed, varlen_mode):
	bias_op, seqlens, bias_group = _prep(q, k, v, bias, attention_mask)
	attrs = _attrs(q, softmax_scale, dropout_prob, causal, bias_group)
	out, lse = _fwd_call(q, k, v, bias_op, seqlens, _seed_operand(dropout_seed), attrs)
	return out, (q, k, v, bias, attention_mask, out, lse, dropout_seed)


def _bwd_rule(softmax_scale, dropout_prob, causal, varlen_mode, residual, dout):
	q, k, v, bias, attention_mask, out, lse, dropout_seed = residual
	bias_op, seqlens, bias_group = _prep(q, k, v, bias, attention_mask)
	attrs = _attrs(q, softmax_scale, dropout_prob, causal, bias_group)
	dq, dk, dv = _bwd_call(q, k, v, bias_op, seqlens, _seed_operand(dropout_seed), out, lse, dout, attrs)
	return dq, dk, dv, None, None, None  # no gradient for mask, bias, seed (_flash_attention.py:88)


flash_attention_call.defvjp(_fwd_rule, _bwd_rule)


def flash_attention(
	q,
	k,
	v,
	attention_mask=None,
	bias=None,
	softmax_scale: tp.Optional[float] = None,
	dropout_prob: float = 0.0,
	causal: bool = False,
	dropout_seed: tp.Optional[int] = None,
	varlen_mode: bool = True,
):
	"""Same signature as the reference's `triton_flash_attention` (_flash_attention.py:125-157).
	`dropout_seed` may be a Python int, an array or a tracer: it is an operand of the custom call.
	A 4-D boolean mask becomes the bias where(mask, 0, finfo(dtype).min) (README.md:188)."""
	if attention_mask is not None and attention_mask.ndim == 4:
		assert bias is None, "Attention mask is not supported along with attention bias. Just use bias instead."
		bias = jnp.where(attention_mask.astype(bool), jnp.zeros((), q.dtype), jnp.full((), jnp.finfo(q.dtype).min, q.dtype))
		attention_mask = None
	# head dims other than 64 / 128 / 256: zero-pad to the next one (the reference pads to the next power of two,
	# _forward_triton.py:525-526); pad and slice are differentiated by jax, the scale keeps the true head dim
	D0 = q.shape[-1]
	D = next((d for d in (64, 128, 256) if D0 <= d), None)
	if D is None:
		raise ValueError(f"head dim {D0} is not supported (at most 256)")
	if D != D0:
		if softmax_scale is None:
			softmax_scale = 1.0 / math.sqrt(D0)
		pad = ((0, 0), (0, 0), (0, 0), (0, D - D0))
		q, k, v = jnp.pad(q, pad), jnp.pad(k, pad), jnp.pad(v, pad)
	out = flash_attention_call(q, k, v, attention_mask, bias, softmax_scale, dropout_prob, causal, dropout_seed, varlen_mode)
	return out if D == D0 else out[..., :D0]


def dropout_mask(B, H, Sq, Sk, dropout_prob, dropout_seed):
	_register()
	out_type = jax.ShapeDtypeStruct((B, H, Sq, Sk), jnp.uint8)
	return _ffi.ffi_call("fa2_dropout_mask_ffi", out_type)(_seed_operand(dropout_seed), dropout_p=np.float32(dropout_prob))


def place_on_least_used_gpu(query, key, value, bias):
	"""`adjust_sharindgs` of the reference's GPU branch (flash_attention.py:229-238, 256-257):
	move the operands to the GPU with the least memory in use (or $GPU_IDX_FLASH_ATTN) and
	return a function that puts the result back on the query's sharding."""
	sharding = getattr(query, "sharding", None)
	gpus = [d for d in jax.local_devices() if d.platform in ("gpu", "rocm")]
	if not gpus:
		return query, key, value, bias, None

	def in_use(d):
		try:
			st = d.memory_stats()
			return st["bytes_in_use"] if st else float("inf")
		except Exception:
			return float("inf")

	idx = int(os.environ.get("GPU_IDX_FLASH_ATTN", min(range(len(gpus)), key=lambda i: in_use(gpus[i]))))
	dev = gpus[idx]
	query, key, value = (jax.device_put(x, dev) for x in (query, key, value))
	if bias is not None:
		bias = jax.device_put(bias, dev)
	restore = (lambda out: jax.device_put(out, sharding)) if sharding is not None else None
	return query, key, value, bias, restore
