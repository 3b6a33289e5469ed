"""JAX spelling of the HIP attention operator: `jax.custom_vjp` around two XLA-FFI
custom calls into libfa2_hip.so.

Takes the place of `jax_flash_attn2/flash_attention_triton/_flash_attention.py:27-157`
of the reference (`_jax_fwd_attention_call`, `_jax_bwd_attention_call`,
`flash_attention_call`, `flash_attention`): same argument list, same static
arguments (softmax_scale, dropout_prob, causal, varlen_mode), same residuals
(q, k, v, bias, mask, out, lse, seed), gradients for q, k, v (and, on request, the bias).
The operand / result / attribute lists of the custom calls are spelled once, in `_ffi_spec.py`.

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

from . import _ffi_spec as spec
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
	for name in spec.HANDLERS:
		_ffi.register_ffi_target(name, _ffi.pycapsule(getattr(lib, name)), platform="ROCM")
	_registered = True


def _ffi_call(name, out_types):
	"""`ffi_call` with a batching rule: under `jax.vmap` the custom call is applied to one slice after the other
	(always correct; the batch axis of the operator itself is the way to batch for speed)."""
	try:
		return _ffi.ffi_call(name, out_types, vmap_method="sequential")
	except TypeError:  # older jax: no vmap_method
		return _ffi.ffi_call(name, out_types)


def _absent(dtype):
	return jnp.zeros((0,), dtype)


class _Cfg(tp.NamedTuple):
	"""Compile-time constants of a call: hashable, the one non-differentiable argument of the differentiation rule."""
	scale: float
	dropout_p: float
	causal: bool
	bias_group: bool
	has_window: bool
	window_left: int
	window_right: int
	softcap: float
	bias_grad: bool


def _attr_dict(cfg: _Cfg):
	"""Attributes of the custom calls in binding order (spec.ATTRS): compile-time constants only (the seed is an operand)."""
	conv = {"float": np.float32, "bool": bool, "int32_t": np.int32}
	return {name: conv[ctype](getattr(cfg, name)) for name, ctype in spec.ATTRS}


def _operands(q, k, v, bias, attention_mask, kv_lens):
	"""Shape checks of `_fwd_attention_kernel_call` (_forward_triton.py:474-495) and the optional operands as the
	handlers take them.  The 2-D right-padded mask becomes one length per batch row instead of a packed layout; a
	4-D boolean mask is the `bias` operand itself, one byte per position - the kernels add finfo(dtype).min at
	masked positions, which is what the bias where(mask, 0, finfo(dtype).min) of README.md:188 would add, without
	that bias ever being built."""
	if attention_mask is not None and attention_mask.ndim == 4:
		assert bias is None, "Attention mask is not supported along with attention bias. Just use bias instead."
		bias, attention_mask = attention_mask.astype(jnp.bool_), None
	check_shapes(q, k, v, bias, attention_mask)
	seqlens = _absent(jnp.int32)
	if attention_mask is not None:
		if attention_mask.ndim != 2:
			raise ValueError("attention_mask must be a 2-D [batch, seq] right-padded validity mask; use bias for general masks")
		seqlens = (attention_mask != 0).sum(axis=1, dtype=jnp.int32)
	bias_group = False
	if bias is None:
		bias_op = _absent(q.dtype)
	else:
		bias_op = bias
		if bias_op.dtype not in (jnp.float16, jnp.bfloat16, jnp.float32, jnp.bool_, jnp.uint8, jnp.int8):
			bias_op = bias_op.astype(jnp.float32)
		bias_group = bias.shape[1] == k.shape[2] and k.shape[2] != q.shape[2] and bias.shape[1] != 1
	if kv_lens is None:
		kv_op = _absent(jnp.int32)
	else:
		kv_op = jnp.asarray(kv_lens).astype(jnp.int32).reshape((q.shape[0],))
	return bias_op, seqlens, kv_op, bias_group


def _seed_operand(dropout_seed):
	"""The dropout seed as the 8-byte operand of the custom calls: uint32[2], low word first.
	A Python int is split on the host (all 64 bits); an array or tracer (the reference jits with a traced
	dropout_seed, _flash_attention.py:91-92) is split with array operations, so nothing is ever converted to a
	host scalar and one executable serves every seed.  `flash_attention` / `flash_attention_call` convert the seed
	BEFORE it reaches the differentiation rule: inside `jax.grad` a Python int argument would otherwise be traced
	as a weakly typed int32 and a seed of 2^31 or more would overflow."""
	if dropout_seed is None:
		return jnp.zeros((2,), jnp.uint32)
	if isinstance(dropout_seed, (int, np.integer)):
		s = int(dropout_seed) & 0xFFFFFFFFFFFFFFFF
		return jnp.asarray(np.array([s & 0xFFFFFFFF, s >> 32], dtype=np.uint32))
	x = jnp.asarray(dropout_seed)
	if x.dtype == jnp.uint32 and x.shape == (2,):
		return x  # already the operand
	x = x.reshape(())
	if x.dtype.itemsize == 8:
		x = x.astype(jnp.uint64)
		return jnp.stack([(x & 0xFFFFFFFF).astype(jnp.uint32), (x >> 32).astype(jnp.uint32)])
	return jnp.stack([x.astype(jnp.uint32), jnp.zeros((), jnp.uint32)])


def _size_query(q, k, cfg: _Cfg, fn_names):
	"""max over the named host-only size queries of the library for these shapes (at least one aligned unit so that
	the result buffer is never empty)."""
	from . import _lib

	p = _lib.new_params()
	p.B, p.Sq, p.Hq, p.D = (int(x) for x in q.shape)
	p.Sk, p.Hkv = int(k.shape[1]), int(k.shape[2])
	p.causal = 1 if cfg.causal else 0  # (causal backward launches split further: their key tiles differ in length)
	p.has_window = 1 if cfg.has_window else 0
	p.softcap = float(cfg.softcap)
	lib = _lib.load()
	return max([int(getattr(lib, n)(ctypes.byref(p))) for n in fn_names] + [256])


def _fwd_call(ops: dict, cfg: _Cfg):
	_register()
	q, k = ops["q"], ops["k"]
	B, Sq, Hq, _ = q.shape
	out_types = dict(
		o=jax.ShapeDtypeStruct(q.shape, q.dtype),
		lse=jax.ShapeDtypeStruct((B, Hq, Sq), jnp.float32),
		scratch=jax.ShapeDtypeStruct((_size_query(q, k, cfg, ("fa2_fwd_scratch_bytes",)),), jnp.uint8),
	)
	res = _ffi_call("fa2_fwd_ffi", tuple(out_types[n] for n in spec.FWD_RESULTS))(*[ops[n] for n in spec.FWD_OPERANDS], **_attr_dict(cfg))
	res = dict(zip(spec.FWD_RESULTS, res))
	return res["o"], res["lse"]


def _bwd_call(ops: dict, cfg: _Cfg):
	_register()
	q, k, v = ops["q"], ops["k"], ops["v"]
	B, Sq, Hq, _ = q.shape
	Sk = k.shape[1]
	scratch_bytes = _size_query(q, k, cfg, ("fa2_bwd_scratch_bytes", "fa2_bwd_split_scratch_bytes"))
	out_types = dict(
		dq=jax.ShapeDtypeStruct(q.shape, q.dtype),
		dk=jax.ShapeDtypeStruct(k.shape, k.dtype),
		dv=jax.ShapeDtypeStruct(v.shape, v.dtype),
		# gradient of the additive term, fp32, IN THE SHAPE OF THE BIAS (the kernels sum over the axes it is broadcast on);
		# 0 elements = not wanted
		dbias=jax.ShapeDtypeStruct(tuple(ops["bias"].shape) if cfg.bias_grad else (0,), jnp.float32),
		scratch=jax.ShapeDtypeStruct((scratch_bytes,), jnp.uint8),
	)
	res = _ffi_call("fa2_bwd_ffi", tuple(out_types[n] for n in spec.BWD_RESULTS))(*[ops[n] for n in spec.BWD_OPERANDS], **_attr_dict(cfg))
	res = dict(zip(spec.BWD_RESULTS, res))
	return res["dq"], res["dk"], res["dv"], res["dbias"]


# differentiable: q, k, v, bias; integer operands (seqlens, kv_lens, seed) get no cotangent; cfg is static
@functools.partial(jax.custom_vjp, nondiff_argnums=(7,))
def _attention(q, k, v, bias, seqlens, kv_lens, seed, cfg):
	return _attention_fwd(q, k, v, bias, seqlens, kv_lens, seed, cfg)[0]


def _attention_fwd(q, k, v, bias, seqlens, kv_lens, seed, cfg):
	out, lse = _fwd_call(dict(q=q, k=k, v=v, bias=bias, seqlens=seqlens, kv_lens=kv_lens, seed=seed), cfg)
	# residuals as in the reference (_flash_attention.py:64-66): q, k, v, bias, mask (here: lengths), out, lse, seed
	return out, (q, k, v, bias, seqlens, kv_lens, seed, out, lse)


def _attention_bwd(cfg, residual, dout):
	q, k, v, bias, seqlens, kv_lens, seed, out, lse = residual
	dq, dk, dv, dbias32 = _bwd_call(
		dict(q=q, k=k, v=v, bias=bias, seqlens=seqlens, kv_lens=kv_lens, seed=seed, o=out, lse=lse, dout=dout), cfg)
	dbias = None  # the reference returns no gradient for the bias (_flash_attention.py:88); `bias_grad=True` asks for one
	if cfg.bias_grad:
		dbias = dbias32.astype(bias.dtype)
	return dq, dk, dv, dbias, None, None, None


_attention.defvjp(_attention_fwd, _attention_bwd)


def flash_attention_call(q, k, v, attention_mask=None, bias=None, softmax_scale=None, dropout_prob=0.0, causal=False,
                         dropout_seed=None, varlen_mode=True, *, kv_lens=None, window_size=None, softcap=0.0, bias_grad=False):
	"""Argument list of the reference's `flash_attention_call` (_flash_attention.py:27-63) plus the keyword-only
	operands the library has beyond it.  Head dim must be one the kernels are built for (`flash_attention` pads)."""
	del varlen_mode  # padded batches are handled in-kernel from per-row lengths, never by packing
	bias_op, seqlens, kv_op, bias_group = _operands(q, k, v, bias, attention_mask, kv_lens)
	if bias_grad and (bias is None or not jnp.issubdtype(bias_op.dtype, jnp.floating)):
		raise ValueError("bias_grad needs a floating-point bias")
	if bias_grad and k.shape[1] % 4:
		raise ValueError("bias_grad needs a key count that is a multiple of 4 (16-byte rows of the fp32 gradient)")
	left, right = (-1, -1) if window_size is None else (int(window_size[0]), int(window_size[1]))
	cfg = _Cfg(
		scale=float(1.0 / math.sqrt(q.shape[-1]) if softmax_scale is None else softmax_scale),
		dropout_p=float(dropout_prob),
		causal=bool(causal),
		bias_group=bool(bias_group),
		has_window=window_size is not None,
		window_left=left,
		window_right=right,
		softcap=float(softcap or 0.0),
		bias_grad=bool(bias_grad),
	)
	return _attention(q, k, v, bias_op, seqlens, kv_op, _seed_operand(dropout_seed), cfg)


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
	*,
	kv_lens=None,
	window_size=None,
	softcap: float = 0.0,
	bias_grad: bool = False,
):
	"""Same signature as the reference's `triton_flash_attention` (_flash_attention.py:125-157).
	`dropout_seed` may be a Python int (all 64 bits are used), an array or a tracer: it is an operand of the custom call.
	A 4-D boolean `attention_mask` is handed to the kernels as bytes (see `_operands`).  Keyword-only, not in the
	reference: `kv_lens` int32 [B] (valid keys per batch row; may be combined with a bias and with Sq != Sk),
	`window_size` = (left, right) (sliding window of refrence_call.py:55-75; a negative bound is none), `softcap`
	(tanh soft-capping of refrence_call.py:48-51), `bias_grad` (also return the gradient of a floating-point bias;
	costs an fp32 [B, Hq, Sq, Sk] intermediate)."""
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
	out = flash_attention_call(q, k, v, attention_mask, bias, softmax_scale, dropout_prob, causal, dropout_seed, varlen_mode,
	                           kv_lens=kv_lens, window_size=window_size, softcap=softcap, bias_grad=bias_grad)
	return out if D == D0 else out[..., :D0]


def dropout_mask(B, H, Sq, Sk, dropout_prob, dropout_seed):
	_register()
	out_type = jax.ShapeDtypeStruct((B, H, Sq, Sk), jnp.uint8)
	return _ffi_call("fa2_dropout_mask_ffi", out_type)(_seed_operand(dropout_seed), dropout_p=np.float32(dropout_prob))


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
