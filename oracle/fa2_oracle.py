"""CPU oracle for the flash-attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product (the package, the C-ABI library) may import this file;
only the test-suite, the smoke check and the benchmark's CPU-baseline leg do,
and only as the checker.

The reference package is pure Python on top of jax/chex/eformer/triton, none
of which exists in this image, so it cannot be executed.  This file restates
its algorithm in NumPy; each function cites the reference lines it follows
(paths are relative to the reference checkout).

What pins each function (see tests/test_oracle.py):
  * philox4x32_10          Random123 known-answer vectors.
  * dropout_keep_mask      by construction from philox4x32_10 + the counter
                           layout documented below; keep-rate statistics.
                           Stream equality with the reference's `tl.rand`
                           is NOT claimed: "parity unpinned" for dropout
                           (the reference's backward ignores dropout, so it
                           has no self-consistent definition to match).
  * attention_fwd          closed form softmax(scale QK^T + bias) V, checked
                           by invariants (V=1, Q=0, key permutation, row
                           shift of bias, GQA == repeated-KV MHA) and against
                           scipy.special.softmax / logsumexp.
  * attention_bwd          central finite differences of attention_fwd (fp64).
  * blockwise_fwd/_bwd     restatement of the reference's JAX-platform
                           blockwise algorithm; pinned by equality with
                           attention_fwd/attention_bwd in fp64.
  * jax_platform_call      restates the facade's JAX branch (it ignores
                           causal / attention_mask / dropout); pinned by
                           equality with attention_fwd(causal=False).
"""

from __future__ import annotations

import math

import numpy as np

# --------------------------------------------------------------------------
# Philox-4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3").
# The reference draws its forward keep-mask from triton's `tl.rand`, which is
# word 0 of this same generator (jax_flash_attn2/flash_attention_triton/
# _forward_triton.py:140-143).  This build keys it on (seed; b, h, i, j).
# --------------------------------------------------------------------------
PHILOX_M0 = np.uint64(0xD2511F53)
PHILOX_M1 = np.uint64(0xCD9E8D57)
PHILOX_W0 = np.uint32(0x9E3779B9)
PHILOX_W1 = np.uint32(0xBB67AE85)
_MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(c0, c1, c2, c3, k0, k1):
	"""Vectorised Philox-4x32 with 10 rounds.  All arguments broadcast; returns 4 uint32 arrays."""
	c0, c1, c2, c3 = (np.asarray(x, dtype=np.uint32) for x in (c0, c1, c2, c3))
	c0, c1, c2, c3 = np.broadcast_arrays(c0, c1, c2, c3)
	k0 = np.uint32(k0)
	k1 = np.uint32(k1)
	with np.errstate(over="ignore"):
		for _ in range(10):
			p0 = PHILOX_M0 * c0.astype(np.uint64)
			p1 = PHILOX_M1 * c2.astype(np.uint64)
			hi0 = (p0 >> np.uint64(32)).astype(np.uint32)
			lo0 = (p0 & _MASK32).astype(np.uint32)
			hi1 = (p1 >> np.uint64(32)).astype(np.uint32)
			lo1 = (p1 & _MASK32).astype(np.uint32)
			c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
			k0 = np.uint32((int(k0) + int(PHILOX_W0)) & 0xFFFFFFFF)
			k1 = np.uint32((int(k1) + int(PHILOX_W1)) & 0xFFFFFFFF)
	return c0, c1, c2, c3


def dropout_threshold(p_drop: float) -> int:
	"""Integer threshold: an element is kept iff its 16-bit Philox value >= threshold."""
	if not (0.0 <= p_drop < 1.0):
		raise ValueError(f"invalid dropout {p_drop}")
	return min(int(math.floor(float(np.float32(p_drop)) * 65536.0)), 0xFFFF)


def dropout_keep_scale(p_drop: float) -> float:
	"""Factor applied to kept values: the reciprocal of the keep probability the 16-bit threshold really gives,
	65536 / (65536 - threshold) - the reference's 1 / (1 - p) (_forward_triton.py:435-438) for the p that the
	threshold realises, so that E[O] equals the output without dropout exactly."""
	return 65536.0 / (65536.0 - dropout_threshold(p_drop))


def dropout_keep_mask(seed: int, p_drop: float, B: int, H: int, Sq: int, Sk: int, pos_offset=(0, 0, 0)) -> np.ndarray:
	"""keep[b,h,i,j] (bool).  `pos_offset` = (b0, h0, i0) shifts the batch / head /
	row indices, for checking a slice of a larger problem (i0 must be even).

	One generator call serves two adjacent rows x four adjacent keys: counter = (j >> 2, i >> 1, h, b),
	key = (seed & 0xffffffff, seed >> 32).  Its four 32-bit words are eight 16-bit values (word w holds
	value 2w in its low half and value 2w + 1 in its high half); element (i, j) owns value
	(i & 1) * 4 + (j & 3) and is kept iff value >= floor(p * 65536).
	Position-only: independent of tiling, so forward and both backward kernels
	regenerate the same mask.  Plays the role of the reference's
	`tl.rand(seed, offs) > p` (_forward_triton.py:140-143, 325-331).
	"""
	thr = np.uint32(dropout_threshold(p_drop))
	k0 = seed & 0xFFFFFFFF
	k1 = (seed >> 32) & 0xFFFFFFFF
	b0, h0, i0 = pos_offset
	if i0 & 1:
		raise ValueError("row offset must be even (a call serves rows 2m and 2m + 1)")
	nj4 = (Sk + 3) // 4
	ni2 = (Sq + 1) // 2
	j4 = np.arange(nj4, dtype=np.uint32)[None, None, None, :]
	i2 = (np.arange(ni2, dtype=np.uint32) + np.uint32(i0 // 2))[None, None, :, None]
	h = (np.arange(H, dtype=np.uint32) + np.uint32(h0))[None, :, None, None]
	b = (np.arange(B, dtype=np.uint32) + np.uint32(b0))[:, None, None, None]
	w = np.stack(philox4x32_10(j4, i2, h, b, k0, k1), axis=-1)  # [B, H, ni2, nj4, 4]
	vals = np.stack([w & np.uint32(0xFFFF), w >> np.uint32(16)], axis=-1).reshape(B, H, ni2, nj4, 8)  # value index 2w + half
	vals = vals.reshape(B, H, ni2, nj4, 2, 4)  # [.., row parity, key & 3]
	vals = vals.transpose(0, 1, 2, 4, 3, 5).reshape(B, H, ni2 * 2, nj4 * 4)[:, :, :Sq, :Sk]
	return vals >= thr


# --------------------------------------------------------------------------
# Exact attention (the closed form every path of the reference evaluates).
# --------------------------------------------------------------------------
def _expand_bias(bias, B, Hq, Hkv, Sq, Sk, dtype):
	"""Bias broadcast rules: batch in {B,1}; heads in {Hq,1,Hkv (repeated per group)}.

	jax_flash_attn2/flash_attention.py:151-169 and flash_attention_triton/_utils.py:151-193.
	"""
	if bias is None:
		return None
	bias = np.asarray(bias, dtype=dtype)
	if bias.ndim != 4:
		raise ValueError("bias must be 4-D [B|1, H|1, Sq, Sk]")
	if bias.shape[2] != Sq or bias.shape[3] != Sk:
		raise ValueError("Bias tensor has incompatible sequence dimensions.")
	if bias.shape[0] not in (1, B):
		raise ValueError("Batch dimension mismatch in bias tensor.")
	hb = bias.shape[1]
	if hb == Hq or hb == 1:
		pass
	elif hb == Hkv:
		bias = np.repeat(bias, Hq // Hkv, axis=1)  # "b h q k -> b (h r) q k"
	else:
		raise ValueError(f"Incompatible bias shape. Got {hb} heads, expected {Hq}, {Hkv}, or 1")
	return np.broadcast_to(bias, (B, Hq, Sq, Sk))


def allowed_mask(B, Sq, Sk, causal, seqlens=None, kv_lens=None, window=None):
	"""allowed[b,i,j]: causal is bottom-right aligned (j <= i + Sk - Sq),
	_forward_triton.py:127-132, refrence_call.py:66-67.  `seqlens[b]` is the
	right-padded 2-D validity mask of the reference's GPU path reduced to a
	length: keys j >= len are masked and query rows i >= len produce zeros
	(_forward_triton.py:474-481,499-510,590-591).  With seqlens the causal
	offset is 0 (it requires Sq == Sk).  `kv_lens[b]` (not in the reference:
	plain key padding) masks keys j >= len only; rows and the causal offset
	are untouched.  `window` = (left, right) is the sliding window of the
	naive reference (refrence_call.py:36-37,55-75): row i sees keys
	i + Sk - Sq - left .. i + Sk - Sq + right, a negative bound meaning none, and
	causal sets right = 0; unlike that code, right < 0 with left >= 0 is "no right
	bound" here (there it would also hide the diagonal)."""
	i = np.arange(Sq)[:, None]
	j = np.arange(Sk)[None, :]
	ok = np.ones((B, Sq, Sk), dtype=bool)
	left, right = (-1, -1) if window is None else window
	if causal:
		right = 0
	if right >= 0:
		ok &= (j <= i + (Sk - Sq) + right)[None]
	if left >= 0:
		ok &= (j >= i + (Sk - Sq) - left)[None]
	if seqlens is not None:
		L = np.asarray(seqlens).reshape(B, 1, 1)
		ok &= (j[None] < L) & (i[None] < L)
	if kv_lens is not None:
		ok &= j[None] < np.asarray(kv_lens).reshape(B, 1, 1)
	return ok


def _bh(x):
	"""[B,S,H,D] -> contiguous [B,H,S,D] (BLAS-friendly)."""
	return np.ascontiguousarray(np.swapaxes(x, 1, 2))


def _qk(a, b):
	"""einsum('bihd,bjhd->bhij') through batched matmul."""
	return np.matmul(_bh(a), np.swapaxes(_bh(b), 2, 3))


def _pv(p, v):
	"""einsum('bhij,bjhd->bihd')."""
	return np.swapaxes(np.matmul(p, _bh(v)), 1, 2)


def _ptx(p, x):
	"""einsum('bhij,bihd->bjhd')."""
	return np.swapaxes(np.matmul(np.swapaxes(p, 2, 3), _bh(x)), 1, 2)


def _scores(q, k, bias, scale, causal, seqlens, dtype, kv_lens=None, window=None, softcap=0.0, return_tanh=False):
	B, Sq, Hq, D = q.shape
	_, Sk, Hkv, _ = k.shape
	if Hq % Hkv:
		raise ValueError(f"Query heads ({Hq}) must be divisible by key/value heads ({Hkv})")
	r = Hq // Hkv
	qf = np.asarray(q, dtype=dtype)
	kf = np.repeat(np.asarray(k, dtype=dtype), r, axis=2)  # q-head h uses kv-head h // r
	s = _qk(qf, kf) * dtype(scale)
	th = None
	if softcap and softcap > 0:
		# tanh soft-capping of the scaled scores, before masks and bias (refrence_call.py:48-51)
		th = np.tanh(s / dtype(softcap))
		s = th * dtype(softcap)
	bb = _expand_bias(bias, B, Hq, Hkv, Sq, Sk, dtype)
	if bb is not None:
		s = s + bb
	ok = allowed_mask(B, Sq, Sk, causal, seqlens, kv_lens, window)[:, None]
	s = np.where(ok, s, -np.inf)
	if return_tanh:
		return s, ok, r, th
	return s, ok, r


def attention_fwd(q, k, v, bias=None, causal=False, scale=None, seqlens=None,
                  p_drop=0.0, seed=0, dtype=np.float64, return_probs=False, pos_offset=(0, 0, 0), kv_lens=None, window=None, softcap=0.0):
	"""O [B,Sq,Hq,D] and LSE [B,Hq,Sq] (natural log) of exact attention.

	q [B,Sq,Hq,D], k/v [B,Sk,Hkv,D].  Rows with no allowed key give O = 0 and
	LSE = -inf (_forward_triton.py:287-289,440-441).  Dropout keeps P/(1-p) where
	keep is set; the normaliser excludes dropout (_forward_triton.py:138-143,435-439).
	"""
	B, Sq, Hq, D = q.shape
	Sk, Hkv = k.shape[1], k.shape[2]
	scale = (1.0 / math.sqrt(D)) if scale is None else scale
	s, ok, r = _scores(q, k, bias, scale, causal, seqlens, dtype, kv_lens, window, softcap)
	m = np.max(s, axis=-1, keepdims=True)
	m_safe = np.where(np.isfinite(m), m, 0.0)
	e = np.exp(s - m_safe)
	l = np.sum(e, axis=-1, keepdims=True)
	with np.errstate(divide="ignore", invalid="ignore"):
		p = np.where(l > 0, e / np.where(l > 0, l, 1.0), 0.0)
		lse = np.where(l[..., 0] > 0, np.log(np.where(l > 0, l, 1.0))[..., 0] + m_safe[..., 0], -np.inf)
	pd = p
	if p_drop > 0.0:
		keep = dropout_keep_mask(seed, p_drop, B, Hq, Sq, Sk, pos_offset)
		pd = np.where(keep, p, 0.0) * dtype(dropout_keep_scale(p_drop))
	vf = np.repeat(np.asarray(v, dtype=dtype), r, axis=2)
	o = _pv(pd, vf)
	if return_probs:
		return o, lse, p, pd
	return o, lse


def attention_bwd(q, k, v, dO, bias=None, causal=False, scale=None, seqlens=None,
                  p_drop=0.0, seed=0, dtype=np.float64, pos_offset=(0, 0, 0), kv_lens=None, window=None, softcap=0.0,
                  return_dbias=False, o_stored=None):
	"""Analytic gradients (dQ, dK, dV) of sum(O * dO); FlashAttention-2 Algorithm 2,
	the same five products as flash_attention_jax/_backward_jax.py:111-127, with
	dK/dV summed over the q-heads of each KV group (_backward_triton.py:1156-1161).
	No gradient for mask / seed (_flash_attention.py:88, _backward_jax.py:164).  The reference returns none for the
	bias either; `return_dbias` adds it as a fourth result: dS = P (dP - delta) before the scale, summed over the
	axes the bias is broadcast on (a size-1 batch or head axis, the q-heads of a KV group for a bias with Hkv heads).
	`o_stored`: the forward output as the backward pass receives it from the residuals (_flash_attention.py:68-75:
	the stored O, rounded to its element type), used for delta = rowsum(O * dO); default: the exact O."""
	B, Sq, Hq, D = q.shape
	Sk, Hkv = k.shape[1], k.shape[2]
	scale = (1.0 / math.sqrt(D)) if scale is None else scale
	o, lse, p, pd = attention_fwd(q, k, v, bias, causal, scale, seqlens, p_drop, seed, dtype, True, pos_offset, kv_lens, window, softcap)
	r = Hq // Hkv
	dOf = np.asarray(dO, dtype=dtype)
	qf = np.asarray(q, dtype=dtype)
	kf = np.repeat(np.asarray(k, dtype=dtype), r, axis=2)
	vf = np.repeat(np.asarray(v, dtype=dtype), r, axis=2)
	dv_full = _ptx(pd, dOf)
	dpd = _qk(dOf, vf)
	if p_drop > 0.0:
		keep = dropout_keep_mask(seed, p_drop, B, Hq, Sq, Sk, pos_offset)
		dp = np.where(keep, dpd, 0.0) * dtype(dropout_keep_scale(p_drop))
	else:
		dp = dpd
	if o_stored is not None:
		o = np.asarray(o_stored, dtype=dtype)
	delta = np.einsum("bihd,bihd->bhi", o, dOf)[..., None]  # = rowsum(P * dP)
	ds = p * (dp - delta)
	dbias = None
	if return_dbias:
		dbias = ds  # [B, Hq, Sq, Sk]
		bshape = np.shape(bias)
		if bshape[1] == 1:
			dbias = dbias.sum(axis=1, keepdims=True)
		elif bshape[1] != Hq:
			dbias = dbias.reshape(B, Hkv, r, Sq, Sk).sum(axis=2)
		if bshape[0] == 1 and B != 1:
			dbias = dbias.sum(axis=0, keepdims=True)
	if softcap and softcap > 0:
		# d/dx [c tanh(x / c)] = 1 - tanh^2(x / c)
		th = _scores(q, k, None, scale, False, None, dtype, softcap=softcap, return_tanh=True)[3]
		ds = ds * (1.0 - th * th)
	dq = _pv(ds, kf) * dtype(scale)
	dk_full = _ptx(ds, qf) * dtype(scale)
	dk = dk_full.reshape(B, Sk, Hkv, r, D).sum(axis=3)
	dv = dv_full.reshape(B, Sk, Hkv, r, D).sum(axis=3)
	if return_dbias:
		return dq, dk, dv, dbias
	return dq, dk, dv


# --------------------------------------------------------------------------
# Blockwise restatement of the reference's JAX platform (CPU baseline).
# --------------------------------------------------------------------------
def blockwise_fwd(q, k, v, bias=None, mask=None, blocksize_q=128, blocksize_k=128, dtype=np.float32):
	"""flash_attention_jax/_forward_jax.py:41-170 on [B,H,S,D] operands; q is
	already scaled.  `mask` is a boolean [B|1,H|1,Sq,Sk]; as in the reference,
	passing any mask also turns on the causal block skip j_end = min(i+1, Tc)
	(:141).  Returns (o, lse) with o in `dtype`, lse fp32 (:55,137)."""
	B, H, Sq, D = q.shape
	Sk = k.shape[2]
	assert Sq % blocksize_q == 0, "Query sequence length is not visible by queryblock size"
	assert Sk % blocksize_k == 0, "Key sequence length is not visible by keyblock size"
	Tr, Tc = Sq // blocksize_q, Sk // blocksize_k
	o = np.zeros((B, H, Sq, v.shape[3]), dtype=dtype)
	lse = np.full((B, H, Sq), -np.inf, dtype=np.float32)
	kT = np.ascontiguousarray(np.swapaxes(k, 2, 3))
	for i in range(Tr):
		qs = slice(i * blocksize_q, (i + 1) * blocksize_q)
		q_i = q[:, :, qs]
		o_i = o[:, :, qs]
		lse_i = lse[:, :, qs]
		m_i = np.full((B, H, blocksize_q), -np.inf, dtype=dtype)
		j_end = min(i + 1, Tc) if mask is not None else Tc
		for j in range(j_end):
			ks = slice(j * blocksize_k, (j + 1) * blocksize_k)
			s_ij = np.matmul(q_i, kT[:, :, :, ks])
			if bias is not None:
				s_ij = s_ij + bias[:, :, qs, ks]
			if mask is not None:
				s_ij = np.where(mask[:, :, qs, ks], s_ij, -1e10)
			m_ij = np.maximum(m_i, s_ij.max(axis=-1))
			p = np.exp(s_ij - m_ij[..., None])
			l_ij = p.sum(-1)
			with np.errstate(invalid="ignore"):
				o_scale = np.exp(m_i - m_ij)
			o_i = (o_i * o_scale[..., None] + np.matmul(p, v[:, :, ks])).astype(dtype)
			with np.errstate(divide="ignore"):
				lse_i = (np.log(np.exp(lse_i - m_ij) + l_ij) + m_ij).astype(np.float32)
			m_i = m_ij.astype(dtype)
		o_i = o_i * np.exp(m_i - lse_i)[..., None]
		o[:, :, qs] = o_i.astype(dtype)
		lse[:, :, qs] = lse_i
	return o, lse


def blockwise_bwd(q, k, v, o, lse, dO, bias=None, mask=None, blocksize_q=128, blocksize_k=128):
	"""flash_attention_jax/_backward_jax.py:54-164 on [B,H,S,D] operands (q pre-scaled).
	The reference writes dK_j/dV_j back at j*blocksize_q (:149-154); that is only
	right when both block sizes agree, so this restatement writes at j*blocksize_k."""
	B, H, Sq, D = q.shape
	Sk = k.shape[2]
	Tr, Tc = Sq // blocksize_q, Sk // blocksize_k
	Dl = np.sum(dO * o, axis=-1)
	dQ = np.zeros_like(q)
	dK = np.zeros_like(k)
	dV = np.zeros_like(v)
	is_causal = mask is not None
	for j in range(Tc):
		ks = slice(j * blocksize_k, (j + 1) * blocksize_k)
		k_j, v_j = k[:, :, ks], v[:, :, ks]
		dK_j, dV_j = dK[:, :, ks], dV[:, :, ks]
		for i in range(j if is_causal else 0, Tr):
			qs = slice(i * blocksize_q, (i + 1) * blocksize_q)
			q_i, dO_i = q[:, :, qs], dO[:, :, qs]
			s_ij = np.matmul(q_i, np.swapaxes(k_j, 2, 3))
			if bias is not None:
				s_ij = s_ij + bias[:, :, qs, ks]
			if mask is not None:
				s_ij = np.where(mask[:, :, qs, ks], s_ij, -1e10)
			p_ij = np.exp(s_ij - lse[:, :, qs, None])
			dV_j = dV_j + np.matmul(np.swapaxes(p_ij, 2, 3), dO_i)
			dP_ij = np.matmul(dO_i, np.swapaxes(v_j, 2, 3))
			dS_ij = p_ij * (dP_ij - Dl[:, :, qs, None])
			dQ[:, :, qs] = dQ[:, :, qs] + np.matmul(dS_ij, k_j)
			dK_j = dK_j + np.matmul(np.swapaxes(dS_ij, 2, 3), q_i)
		dK[:, :, ks] = dK_j
		dV[:, :, ks] = dV_j
	return dQ, dK, dV


def jax_platform_call(q, k, v, bias=None, softmax_scale=None, blocksize_q=128, blocksize_k=128,
                      dtype=np.float32, with_grads_for=None, mask=None):
	"""FlashAttention._compute_jax (flash_attention.py:324-349) followed by
	flash_attention_jax/_flash_attention.py:98-133: repeat KV heads to Hq,
	transpose to [B,H,S,D], clamp the block sizes to S, pre-scale q, run the
	blockwise forward with mask=None.  causal / attention_mask / dropout never
	reach the kernel on this branch of the reference.  q,k,v are [B,S,H,D].
	`mask` (boolean [B|1,H|1,Sq,Sk], not what the facade passes) runs the same
	functions the way their own `mask` argument does, causal block skip included
	(flash_attention_jax/_flash_attention.py:98-133 with a mask).
	With `with_grads_for=dO` also returns (dq, dk, dv) the way jax.grad would
	(chain rule through the repeat and the pre-scale)."""
	B, Sq, Hq, D = q.shape
	Hkv = k.shape[2]
	r = Hq // Hkv
	kk = np.repeat(k, r, axis=2)
	vv = np.repeat(v, r, axis=2)
	qt, kt, vt = (np.ascontiguousarray(np.swapaxes(x, 1, 2)).astype(dtype) for x in (q, kk, vv))
	bq = min(qt.shape[2], blocksize_q or 128)
	bk = min(kt.shape[2], blocksize_k or 128)
	sc = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(float(D))
	qt = qt * dtype(sc)
	bb = None
	if bias is not None:
		bb = _expand_bias(bias, B, Hq, Hkv, Sq, kt.shape[2], dtype)
	o, lse = blockwise_fwd(qt, kt, vt, bb, mask, bq, bk, dtype)
	out = np.swapaxes(o, 1, 2)
	if with_grads_for is None:
		return out
	dOt = np.ascontiguousarray(np.swapaxes(with_grads_for, 1, 2)).astype(dtype)
	dq, dk, dv = blockwise_bwd(qt, kt, vt, o, lse, dOt, bb, mask, bq, bk)
	dq = np.swapaxes(dq, 1, 2) * dtype(sc)
	dk = np.swapaxes(dk, 1, 2).reshape(B, -1, Hkv, r, D).sum(3)
	dv = np.swapaxes(dv, 1, 2).reshape(B, -1, Hkv, r, D).sum(3)
	return out, (dq, dk, dv)


# --------------------------------------------------------------------------
# Low-precision helpers shared by tests and the benchmark.
# --------------------------------------------------------------------------
def round_bf16(x):
	"""Round-to-nearest-even fp32 -> bf16 -> fp32 (NumPy has no bf16)."""
	x = np.ascontiguousarray(x, dtype=np.float32)
	u = x.view(np.uint32)
	rounded = ((u.astype(np.uint64) + np.uint64(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint64(0xFFFF0000)).astype(np.uint32)
	out = rounded.view(np.float32).copy()
	nan = np.isnan(x)
	out[nan] = np.nan
	return out


def to_bf16_bits(x):
	"""fp32 array that is already bf16-representable -> uint16 bit patterns."""
	return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def from_bf16_bits(u):
	return (np.asarray(u, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def rel_l2(a, b):
	a = np.asarray(a, dtype=np.float64)
	b = np.asarray(b, dtype=np.float64)
	return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
