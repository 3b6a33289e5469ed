"""The HIP attention operator: forward / backward calls into libfa2_hip.so and
the differentiation rule that ties them together.

Takes the place of the reference's per-platform operator
`jax_flash_attn2/flash_attention_triton/_flash_attention.py:27-157`
(`_jax_fwd_attention_call`, `_jax_bwd_attention_call`, `flash_attention_call`,
`flash_attention`): same argument list, same residuals (q, k, v, bias, mask,
out, lse, seed), gradients for q, k, v only.

Arrays here are torch tensors on a ROCm device - torch is used for device
memory and the stream handle only; every number is produced by the C ABI.  The
same two entry points are what the XLA-FFI handlers in csrc/fa2_xla_ffi.cc
forward to when the caller is JAX.
"""

from __future__ import annotations

import ctypes
import math
import typing as tp

import torch

from . import _lib
from ._checks import check_shapes  # noqa: F401  (re-exported)
from ._lib import FA2_BF16, FA2_FP16, FA2_FP32, FA2_MASK_U8, Fa2Tensor

_DTYPES = {torch.float16: FA2_FP16, torch.bfloat16: FA2_BF16}
# (a uint8 / bool `bias` is a boolean mask, one byte per position: see fa2_params.bias_dtype)
_BIAS_DTYPES = {torch.float16: FA2_FP16, torch.bfloat16: FA2_BF16, torch.float32: FA2_FP32, torch.uint8: FA2_MASK_U8}


def _stream_ptr(device) -> int:
	return torch.cuda.current_stream(device).cuda_stream


def _t4(x: torch.Tensor) -> Fa2Tensor:
	"""[B, S, H, D] tensor -> pointer + element strides (D stride must be 1)."""
	t = Fa2Tensor()
	t.ptr = x.data_ptr()
	t.stride_b, t.stride_s, t.stride_h = x.stride(0), x.stride(1), x.stride(2)
	return t


# Head dims the kernels are built for.  Any other head dim up to 256 is zero-padded to the next
# one, as the reference pads to the next power of two (_forward_triton.py:525-526): zero
# columns of q / k leave the scores unchanged, zero columns of v and dO give zero columns of
# O, dV and dQ / dK, which are cut off again.  The softmax scale keeps using the true head dim.
HEAD_DIMS = (64, 128, 256)


def _kernel_head_dim(D: int) -> int:
	for d in HEAD_DIMS:
		if D <= d:
			return d
	raise ValueError(f"head dim {D} is not supported (at most {HEAD_DIMS[-1]})")


def _pad_d(x: torch.Tensor, Dp: int) -> torch.Tensor:
	return x if x.shape[-1] == Dp else torch.nn.functional.pad(x, (0, Dp - x.shape[-1]))


def _usable(x: torch.Tensor) -> torch.Tensor:
	"""Kernels read 16 bytes at a time along D: unit D stride, 16-byte aligned rows."""
	if x.stride(3) != 1 or any(s % 8 for s in x.stride()[:3]) or x.data_ptr() % 16:
		return x.contiguous()
	return x


def _fill_common(p, q, k, v, bias, seqlens, scale, p_drop, causal, seed, kv_lens=None, window=None, softcap=0.0):
	B, Sq, Hq, D = q.shape
	Sk, Hkv = k.shape[1], k.shape[2]
	p.dtype = _DTYPES[q.dtype]
	p.B, p.Sq, p.Sk, p.Hq, p.Hkv, p.D = B, Sq, Sk, Hq, Hkv, D
	p.causal = 1 if causal else 0
	p.scale = float(scale)
	p.p_drop = float(p_drop)
	_fill_seed(p, seed, q.device)
	p.q, p.k, p.v = _t4(q), _t4(k), _t4(v)
	if bias is not None:
		p.bias = bias.data_ptr()
		p.bias_dtype = _BIAS_DTYPES[bias.dtype]
		# broadcast rules of calc_bias_strides (_utils.py:169-190): size-1 axes get stride 0.
		p.bias_stride_b = 0 if bias.shape[0] == 1 else bias.stride(0)
		p.bias_stride_h = 0 if bias.shape[1] == 1 else bias.stride(1)
		p.bias_stride_m = bias.stride(2)
		# a bias with Hkv heads is read per KV group instead of being repeated to Hq heads
		# (the facade materialises that repeat, flash_attention.py:161-164)
		p.bias_group = 1 if (bias.shape[1] == Hkv and Hkv != Hq and bias.shape[1] != 1) else 0
	if seqlens is not None:
		p.seqlens = seqlens.data_ptr()
	if window is not None:
		left, right = window
		p.has_window, p.window_left, p.window_right = 1, int(left), int(right)
	p.softcap = float(softcap or 0.0)
	if kv_lens is not None:
		if kv_lens.dtype != torch.int32 or kv_lens.numel() != B or not kv_lens.is_contiguous():
			raise ValueError("kv_lens must be a contiguous int32 tensor with one entry per batch row")
		p.kv_lens = kv_lens.data_ptr()


def _fill_seed(p, seed, device):
	"""The dropout seed is a Python int (copied into the parameter block) or a one-element int64 tensor on the device,
	which the kernels read there: a seed that is itself the result of device work - as a traced `dropout_seed` is in
	the reference, an operand of the custom call (_forward_triton.py:553) - needs no host round trip."""
	if isinstance(seed, torch.Tensor):
		if seed.dtype != torch.int64 or seed.numel() != 1 or seed.device != device:
			raise ValueError("a tensor dropout_seed must be a one-element int64 tensor on the device of q")
		p.seed = 0
		p.seed_dev = seed.data_ptr()
	else:
		p.seed = int(seed or 0) & 0xFFFFFFFFFFFFFFFF
		p.seed_dev = None


def _prep_bias(bias):
	if bias is None:
		return None
	if bias.dtype == torch.bool:
		bias = bias.view(torch.uint8)  # same bytes: 0 = masked
	if bias.dtype not in _BIAS_DTYPES:
		bias = bias.to(torch.float32)
	if bias.stride(3) != 1:
		bias = bias.contiguous()
	return bias


def _mask_operand(mask, q):
	"""A 4-D boolean mask [B|1, H|1, Sq, Sk] is handed to the kernels as it is, one byte per position.  They add the
	lowest finite value of q's dtype at masked positions, i.e. they compute what the reference's documentation
	spells as the bias where(mask, 0, finfo(dtype).min) (README.md:188) without that bias ever being built.
	(The reference's GPU path itself only takes the 2-D mask.)"""
	m = mask.to(device=q.device)
	m = m if m.dtype == torch.bool else m.ne(0)
	return m.contiguous() if m.stride(3) != 1 else m


def _seqlens_from_mask(attention_mask, q):
	"""The reference's GPU path takes a right-padded 2-D validity mask [B, S] and
	packs the valid tokens (_forward_triton.py:499-510).  Here the mask is reduced
	to one length per batch row which the kernels consume directly."""
	if attention_mask is None:
		return None
	if attention_mask.dim() != 2:
		raise ValueError("attention_mask must be a 2-D [batch, seq] right-padded validity mask; use bias for general masks")
	return attention_mask.to(device=q.device).ne(0).sum(dim=1, dtype=torch.int32).contiguous()


def fwd(q, k, v, bias=None, seqlens=None, softmax_scale=None, dropout_prob=0.0, causal=False, dropout_seed=None, kv_lens=None,
        window=None, softcap=0.0):
	"""Returns (out [B,Sq,Hq,D] in q.dtype, lse [B,Hq,Sq] fp32 natural log)."""
	lib = _lib.load()
	D0 = q.shape[-1]
	D = _kernel_head_dim(D0)
	q, k, v = _usable(_pad_d(q, D)), _usable(_pad_d(k, D)), _usable(_pad_d(v, D))
	bias = _prep_bias(bias)
	B, Sq, Hq, _ = q.shape
	scale = 1.0 / math.sqrt(D0) if softmax_scale is None else softmax_scale
	out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
	lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
	p = _lib.new_params()
	_fill_common(p, q, k, v, bias, seqlens, scale, dropout_prob, causal, dropout_seed, kv_lens, window, softcap)
	p.o = _t4(out)
	p.lse = lse.data_ptr()
	# short query over many keys: scratch lets the library split the keys over workgroups
	need = lib.fa2_fwd_scratch_bytes(ctypes.byref(p))
	if need:
		scratch = torch.empty((need,), dtype=torch.uint8, device=q.device)
		p.scratch = scratch.data_ptr()
		p.scratch_bytes = need
	_lib.check(lib.fa2_fwd(ctypes.byref(p), _stream_ptr(q.device)))
	return (out if D == D0 else out[..., :D0]), lse


def bwd(q, k, v, out, lse, dout, bias=None, seqlens=None, softmax_scale=None, dropout_prob=0.0, causal=False,
        dropout_seed=None, kv_lens=None, window=None, softcap=0.0, need_dbias=False):
	"""Returns (dq, dk, dv) in the dtypes of q, k, v; dk/dv summed over each KV group.  With `need_dbias` a fourth
	result: the gradient of the additive bias, fp32, in the shape of `bias` (summed over the axes it is broadcast on;
	those sums are atomic adds in the dQ kernel - see fa2_params.dbias - so the buffer is as small as the bias)."""
	lib = _lib.load()
	D0 = q.shape[-1]
	D = _kernel_head_dim(D0)
	q, k, v, out, dout = (_usable(_pad_d(x, D)) for x in (q, k, v, out, dout))
	bias = _prep_bias(bias)
	B, Sq, Hq, _ = q.shape
	scale = 1.0 / math.sqrt(D0) if softmax_scale is None else softmax_scale
	dq = torch.empty_like(q, memory_format=torch.contiguous_format)
	dk = torch.empty_like(k, memory_format=torch.contiguous_format)
	dv = torch.empty_like(v, memory_format=torch.contiguous_format)
	p = _lib.new_params()
	_fill_common(p, q, k, v, bias, seqlens, scale, dropout_prob, causal, dropout_seed, kv_lens, window, softcap)
	p.o = _t4(out)
	p.lse = lse.data_ptr()
	p.dout, p.dq, p.dk, p.dv = _t4(dout), _t4(dq), _t4(dk), _t4(dv)
	# (the larger size, where it applies, lets the dK/dV kernel of a small grid split the q-heads of a group over workgroups)
	need = max(lib.fa2_bwd_scratch_bytes(ctypes.byref(p)), lib.fa2_bwd_split_scratch_bytes(ctypes.byref(p)))
	scratch = torch.empty((max(need, 256),), dtype=torch.uint8, device=q.device)
	p.scratch = scratch.data_ptr()
	p.scratch_bytes = scratch.numel()
	dbias = None
	if need_dbias:
		if bias is None or bias.dtype == torch.uint8:
			raise ValueError("the bias gradient needs a floating-point bias")
		# fp32, zero-filled (the kernel leaves skipped key tiles alone), in the SHAPE OF THE BIAS: on the axes the bias is
		# broadcast on (size-1 batch / head axis, Hkv heads) the dQ kernel accumulates with atomic adds, so the memory is
		# that of the bias itself and not B * Hq * Sq * Sk * 4 bytes.  Rows start on 16 bytes.
		Skp = (k.shape[1] + 3) // 4 * 4
		dbias = torch.zeros((bias.shape[0], bias.shape[1], Sq, Skp), dtype=torch.float32, device=q.device)[..., : k.shape[1]]
		p.dbias = dbias.data_ptr()
		p.dbias_stride_b = 0 if bias.shape[0] == 1 else dbias.stride(0)
		p.dbias_stride_h = 0 if bias.shape[1] == 1 else dbias.stride(1)
		p.dbias_stride_m = dbias.stride(2)
	_lib.check(lib.fa2_bwd(ctypes.byref(p), _stream_ptr(q.device)))
	if D != D0:
		dq, dk, dv = dq[..., :D0], dk[..., :D0], dv[..., :D0]
	if need_dbias:
		return dq, dk, dv, dbias
	return dq, dk, dv


def dropout_mask(B, H, Sq, Sk, dropout_prob, dropout_seed, device) -> torch.Tensor:
	"""keep[b,h,i,j] (uint8) exactly as the kernels regenerate it."""
	lib = _lib.load()
	keep = torch.empty((B, H, Sq, Sk), dtype=torch.uint8, device=device)
	p = _lib.new_params()
	p.B, p.Hq, p.Hkv, p.Sq, p.Sk, p.D = B, H, H, Sq, Sk, 64
	p.p_drop = float(dropout_prob)
	_fill_seed(p, dropout_seed, torch.device(device))
	_lib.check(lib.fa2_dropout_mask(ctypes.byref(p), keep.data_ptr(), _stream_ptr(device)))
	return keep


class Plan:
	"""A filled parameter block with its output buffers, for callers that repeat
	the same call (benchmarks, graph capture): `forward()` / `backward()` only
	enqueue kernels, nothing is allocated per call."""

	def __init__(self, q, k, v, dout=None, bias=None, seqlens=None, softmax_scale=None, dropout_prob=0.0, causal=False,
	             dropout_seed=None, kv_lens=None, window=None, softcap=0.0):
		self.lib = _lib.load()
		self.q, self.k, self.v = _usable(q), _usable(k), _usable(v)
		self.bias = _prep_bias(bias)
		self.seqlens = seqlens
		B, Sq, Hq, D = q.shape
		scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
		self.out = torch.empty((B, Sq, Hq, D), dtype=q.dtype, device=q.device)
		self.lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
		p = self.params = _lib.new_params()
		self.kv_lens = kv_lens
		_fill_common(p, self.q, self.k, self.v, self.bias, seqlens, scale, dropout_prob, causal, dropout_seed, kv_lens, window, softcap)
		self.seed = dropout_seed  # (a device-resident seed must outlive the plan's calls)
		p.o = _t4(self.out)
		p.lse = self.lse.data_ptr()
		self.device = q.device
		if dout is not None:
			self.dout = _usable(dout)
			self.dq = torch.empty_like(self.q, memory_format=torch.contiguous_format)
			self.dk = torch.empty_like(self.k, memory_format=torch.contiguous_format)
			self.dv = torch.empty_like(self.v, memory_format=torch.contiguous_format)
			p.dout, p.dq, p.dk, p.dv = _t4(self.dout), _t4(self.dq), _t4(self.dk), _t4(self.dv)
			need = max(self.lib.fa2_bwd_scratch_bytes(ctypes.byref(p)), self.lib.fa2_bwd_split_scratch_bytes(ctypes.byref(p)))
		else:
			need = 0
		# one buffer serves both calls: the backward needs its scratch, the forward uses scratch when it splits a
		# short query over key ranges (the partial results do not outlive the forward call)
		need = max(need, self.lib.fa2_fwd_scratch_bytes(ctypes.byref(p)))
		if need:
			self.scratch = torch.empty((max(need, 256),), dtype=torch.uint8, device=q.device)
			p.scratch = self.scratch.data_ptr()
			p.scratch_bytes = self.scratch.numel()

	def forward(self):
		_lib.check(self.lib.fa2_fwd(ctypes.byref(self.params), _stream_ptr(self.device)))
		return self.out, self.lse

	def backward(self, stages: int = 7):
		_lib.check(self.lib.fa2_bwd_stages(ctypes.byref(self.params), _stream_ptr(self.device), stages))
		return self.dq, self.dk, self.dv


class _FlashAttentionFn(torch.autograd.Function):
	"""Differentiation rule; the torch spelling of the reference's
	`flash_attention_call.defvjp(_jax_fwd_attention_call, _jax_bwd_attention_call)`
	(_flash_attention.py:119-122).  Returns (dq, dk, dv) and None for everything else, as the reference does
	(_flash_attention.py:88) - unless the caller asked for the gradient of the bias (`bias_grad=True`)."""

	@staticmethod
	def forward(ctx, q, k, v, bias, seqlens, softmax_scale, dropout_prob, causal, dropout_seed, kv_lens=None, window=None, softcap=0.0,
	            bias_grad=False):
		out, lse = fwd(q, k, v, bias, seqlens, softmax_scale, dropout_prob, causal, dropout_seed, kv_lens, window, softcap)
		ctx.save_for_backward(q, k, v, bias, seqlens, out, lse, kv_lens)
		ctx.cfg = (softmax_scale, dropout_prob, causal, dropout_seed, window, softcap, bias_grad)
		return out

	@staticmethod
	def backward(ctx, dout):
		q, k, v, bias, seqlens, out, lse, kv_lens = ctx.saved_tensors
		softmax_scale, dropout_prob, causal, dropout_seed, window, softcap, bias_grad = ctx.cfg
		need_dbias = bool(bias_grad) and bias is not None and ctx.needs_input_grad[3]
		res = bwd(q, k, v, out, lse, dout, bias, seqlens, softmax_scale, dropout_prob, causal, dropout_seed, kv_lens, window, softcap,
		          need_dbias=need_dbias)
		dbias = res[3].to(bias.dtype) if need_dbias else None
		return res[0], res[1], res[2], dbias, None, None, None, None, None, None, None, None, None


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
	"""Same signature as the reference's `triton_flash_attention`
	(_flash_attention.py:125-157).  `varlen_mode` is accepted for source
	compatibility; padded batches are always handled in-kernel from per-row
	lengths, never by packing.  `kv_lens` (keyword only, not in the reference):
	int32 [B] number of valid keys per batch row - key padding that may be combined
	with a bias and with Sq != Sk, which the 2-D attention_mask may not.  `window_size` =
	(left, right) (keyword only): the sliding window of the reference's naive attention
	(refrence_call.py:32,55-75); a negative bound is none, causal sets right = 0.  `softcap` > 0
	(keyword only): scores become softcap * tanh(score / softcap) before bias and masks
	(refrence_call.py:33,48-51).  `bias_grad` (keyword only): also differentiate with respect to a floating-point
	`bias` that requires a gradient - off by default, as the reference returns no gradient for its bias
	(_flash_attention.py:88); costs a zero-filled fp32 buffer in the shape of the bias and, where the bias is
	broadcast over batch or heads, atomic adds in the dQ kernel (summation order not fixed)."""
	del varlen_mode
	if bias_grad and attention_mask is not None and attention_mask.dim() == 4:
		raise ValueError("bias_grad needs a floating-point bias, not a boolean mask")
	if attention_mask is not None and attention_mask.dim() == 4:
		assert bias is None, "Attention mask is not supported along with attention bias. Just use bias instead."
		bias, attention_mask = _mask_operand(attention_mask, q), None
	check_shapes(q, k, v, bias, attention_mask)
	seqlens = _seqlens_from_mask(attention_mask, q)
	return _FlashAttentionFn.apply(q, k, v, bias, seqlens, softmax_scale, dropout_prob, causal, dropout_seed, kv_lens, window_size, softcap,
	                               bias_grad)
