"""The five benchmark configurations at FULL size on the GPU.

The NumPy oracle cannot evaluate S x S score matrices for every (batch, head)
of these shapes in seconds, so each config is checked (a) against the oracle
on slices that are self-contained - whole KV groups of one batch row, or the
last rows / last keys of a causal problem - and (b) through size-independent
properties (probabilities sum to one through LSE, V = 1 gives O = 1,
delta identity, GQA reduction).
"""

import numpy as np
import pytest
import torch

import fa2_oracle as O
from _cases import TOL_GRAD_REL_L2, TOL_O, check_forward, check_grads
from jax_flash_attn2 import _hip_op as op

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _gen(shape, seed, mul, dtype):
	g = torch.Generator(device=DEV).manual_seed(seed)
	return (torch.randn(shape, generator=g, device=DEV, dtype=torch.float32) * mul).to(dtype)


def _np(t):
	return t.float().cpu().numpy().astype(np.float32)


def _check_group(q, k, v, do, o, lse, grads, b, g, r, dtype, **kw):
	"""Oracle on batch row b, KV head g with its r query heads: self-contained for O, LSE, dQ, dK, dV."""
	hs = slice(g * r, (g + 1) * r)
	args = [_np(q[b:b + 1, :, hs]), _np(k[b:b + 1, :, g:g + 1]), _np(v[b:b + 1, :, g:g + 1])]
	kw = dict(kw, dtype=np.float32, pos_offset=(b, g * r, 0))
	o_ref, lse_ref = O.attention_fwd(*args, **kw)
	check_forward(o[b:b + 1, :, hs], lse[b:b + 1, hs], o_ref, lse_ref, dtype, f"group b{b} g{g}")
	if grads is not None:
		g_ref = O.attention_bwd(*args, _np(do[b:b + 1, :, hs]), **kw)
		got = (grads[0][b:b + 1, :, hs], grads[1][b:b + 1, :, g:g + 1], grads[2][b:b + 1, :, g:g + 1])
		check_grads(got, g_ref, f"group b{b} g{g}")


def test_c1_readme_shape_fp16_causal_forward():
	# B2 Hq16 Hkv4 S512 D64 fp16 causal, forward only, N(0,1) inputs
	dtype = torch.float16
	q, k, v = _gen((2, 512, 16, 64), 0, 1.0, dtype), _gen((2, 512, 4, 64), 1, 1.0, dtype), _gen((2, 512, 4, 64), 2, 1.0, dtype)
	o, lse = op.fwd(q, k, v, causal=True)
	o_ref, lse_ref = O.attention_fwd(_np(q), _np(k), _np(v), causal=True)
	check_forward(o, lse, o_ref, lse_ref, dtype, "c1")


def test_c1_readme_call_taken_literally():
	"""The README's call (README.md:28-45) passes q (2, 16, 512, 64) and k, v (2, 4, 512, 64) - generated as
	[batch, heads, seq, dim] - straight to an API that reads [batch, seq, heads, dim] (flash_attention.py:186-187):
	to the code this is B2, Sq16, Sk4, 512 heads without grouping, D64.  Causal is bottom-right aligned, so the first
	Sq - Sk = 12 rows see no key and come back as zeros, and with Sq != Sk a 2-D mask is dropped
	(flash_attention.py:239-242).  Through FlashAttention.__call__, against the oracle, with gradients."""
	from jax_flash_attn2 import AttentionConfig, Backend, FlashAttention, Platform

	dtype = torch.float16
	q, k, v = _gen((2, 16, 512, 64), 0, 1.0, dtype), _gen((2, 4, 512, 64), 1, 1.0, dtype), _gen((2, 4, 512, 64), 2, 1.0, dtype)
	do = _gen((2, 16, 512, 64), 3, 1.0, dtype)
	attn = FlashAttention(AttentionConfig(platform=Platform.HIP, backend=Backend.GPU))
	qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
	out = attn(query=qd, key=kd, value=vd, causal=True)
	out.backward(do)
	assert out.shape == q.shape and out.dtype == dtype
	o_ref, lse_ref = O.attention_fwd(_np(q), _np(k), _np(v), causal=True)
	g_ref = O.attention_bwd(_np(q), _np(k), _np(v), _np(do), causal=True)
	_, lse = op.fwd(q, k, v, causal=True)
	check_forward(out.detach(), lse, o_ref, lse_ref, dtype, "README call as the code reads it")
	check_grads((qd.grad, kd.grad, vd.grad), g_ref, "README call as the code reads it")
	assert out[:, :12].abs().max().item() == 0 and qd.grad[:, :12].abs().max().item() == 0  # rows without a key
	assert torch.isneginf(lse[:, :, :12]).all()
	# a 2-D mask is dropped when Sq != Sk: same result
	out_m = attn(query=q, key=k, value=v, causal=True, attention_mask=torch.ones(2, 16, dtype=torch.int32, device=DEV))
	assert torch.equal(out_m, out.detach())


def test_c2_llama_prefill_bf16_causal_fwd_bwd():
	# B4 S4096 Hq32 Hkv8 D128 bf16 causal
	dtype = torch.bfloat16
	B, S, Hq, Hkv, D = 4, 4096, 32, 8, 128
	q, k, v = _gen((B, S, Hq, D), 0, 0.5, dtype), _gen((B, S, Hkv, D), 1, 0.5, dtype), _gen((B, S, Hkv, D), 2, 0.5, dtype)
	do = _gen((B, S, Hq, D), 3, 1.0, dtype)
	o, lse = op.fwd(q, k, v, causal=True)
	grads = op.bwd(q, k, v, o, lse, do, causal=True)
	for b, g in ((0, 0), (3, 7)):
		_check_group(q, k, v, do, o, lse, grads, b, g, 4, dtype, causal=True)
	# V = 1 -> O = 1 for every (b, h, i)
	o1, _ = op.fwd(q, k, torch.ones_like(v), causal=True)
	assert (o1.float() - 1).abs().max().item() <= 1e-2
	for t in grads:
		assert torch.isfinite(t.float()).all()


def test_c3_padded_mha_bias_bf16_fwd_bwd():
	# B8 S2048 H16 D64 bf16 non-causal, bias [B,1,S,S] = 1/(1+|i-j|) + finfo.min on padded keys
	dtype = torch.bfloat16
	B, S, H, D = 8, 2048, 16, 64
	q, k, v = _gen((B, S, H, D), 0, 0.5, dtype), _gen((B, S, H, D), 1, 0.5, dtype), _gen((B, S, H, D), 2, 0.5, dtype)
	do = _gen((B, S, H, D), 3, 1.0, dtype)
	i = torch.arange(S, device=DEV)
	base = 1.0 / (1.0 + (i[:, None] - i[None, :]).abs().float())
	lens = torch.randint(S // 2, S + 1, (B,), generator=torch.Generator().manual_seed(4))
	valid = i[None, :] < lens.to(DEV)[:, None]
	bias = torch.where(valid[:, None, None, :], base[None, None], torch.tensor(torch.finfo(dtype).min, device=DEV)).to(dtype)
	o, lse = op.fwd(q, k, v, bias)
	grads = op.bwd(q, k, v, o, lse, do, bias)
	for b, h in ((0, 0), (7, 15), (3, 5)):
		_check_group(q, k, v, do, o, lse, grads, b, h, 1, dtype, bias=_np(bias[b:b + 1]))
	# masked keys receive exactly zero gradient
	for b in range(B):
		L = int(lens[b])
		if L < S:
			assert grads[1][b, L:].abs().max().item() == 0 and grads[2][b, L:].abs().max().item() == 0


def test_c4_long_context_bf16_causal_fwd_bwd():
	# B1 S32768 Hq64 Hkv8 D128 bf16 causal.  Oracle on the last 256 rows (all keys) of one KV group:
	# exact for O, LSE, dQ of those rows, and for dK, dV of the last 256 keys (only those rows see them).
	dtype = torch.bfloat16
	B, S, Hq, Hkv, D = 1, 32768, 64, 8, 128
	q, k, v = _gen((B, S, Hq, D), 0, 0.5, dtype), _gen((B, S, Hkv, D), 1, 0.5, dtype), _gen((B, S, Hkv, D), 2, 0.5, dtype)
	do = _gen((B, S, Hq, D), 3, 1.0, dtype)
	o, lse = op.fwd(q, k, v, causal=True)
	dq, dk, dv = op.bwd(q, k, v, o, lse, do, causal=True)
	R = 256
	for g in (0, 7):
		hs = slice(g * 8, (g + 1) * 8)
		args = [_np(q[:, S - R:, hs]), _np(k[:, :, g:g + 1]), _np(v[:, :, g:g + 1])]
		o_ref, lse_ref = O.attention_fwd(*args, causal=True, dtype=np.float32)
		check_forward(o[:, S - R:, hs], lse[:, hs, S - R:], o_ref, lse_ref, dtype, f"c4 g{g}")
		dq_ref, dk_ref, dv_ref = O.attention_bwd(*args, _np(do[:, S - R:, hs]), causal=True, dtype=np.float32)
		check_grads((dq[:, S - R:, hs], dk[:, S - R:, g:g + 1], dv[:, S - R:, g:g + 1]),
		            (dq_ref, dk_ref[:, S - R:], dv_ref[:, S - R:]), f"c4 g{g}")
	# The FIRST 256 keys of a KV group - the longest key tiles of the dK/dV kernel: every one of the 32768 rows of all 8
	# q-heads sees them - against an fp32 evaluation in torch on the GPU, row chunk by row chunk: the row normaliser is a
	# logsumexp over all keys of the chunk's fp32 scores and delta comes from the fp32 O of the same evaluation, nothing
	# is taken from the kernels' own lse or O.
	K0, CH, g = 256, 2048, 5
	scale = D ** -0.5
	kg, vg = k[0, :, g].float(), v[0, :, g].float()
	dk_ref = torch.zeros(K0, D, device=DEV)
	dv_ref = torch.zeros(K0, D, device=DEV)
	cols = torch.arange(S, device=DEV)
	for h in range(g * 8, (g + 1) * 8):
		for r0 in range(0, S, CH):
			qc, doc = q[0, r0:r0 + CH, h].float(), do[0, r0:r0 + CH, h].float()
			ne = r0 + CH  # keys beyond the chunk's last row are masked for all of its rows
			sc = (qc @ kg[:ne].T) * scale
			sc.masked_fill_(cols[None, :ne] > (r0 + torch.arange(CH, device=DEV))[:, None], float("-inf"))
			pr = torch.exp(sc - torch.logsumexp(sc, dim=-1, keepdim=True))
			delta = ((pr @ vg[:ne]) * doc).sum(-1, keepdim=True)
			p0 = pr[:, :K0]
			dv_ref += p0.T @ doc
			dk_ref += (p0 * (doc @ vg[:K0].T - delta)).T @ qc * scale
			del sc, pr
	for name, got, ref in (("dk", dk[0, :K0, g], dk_ref), ("dv", dv[0, :K0, g], dv_ref)):
		e = float((got.float() - ref).norm() / ref.norm())
		assert e <= TOL_GRAD_REL_L2, f"c4 first {K0} keys of group {g}: {name} rel-L2 {e:.3e}"
	# first rows: row 0 attends to key 0 only -> O[0] = V[0], LSE = scale q0.k0
	assert torch.equal(o[0, 0].reshape(8, 8, D), v[0, 0][:, None, :].expand(8, 8, D))
	# V = 1 -> O = 1 everywhere (every row tile, every causal tile boundary)
	o1, _ = op.fwd(q, k, torch.ones_like(v), causal=True)
	assert (o1.float() - 1).abs().max().item() <= 1e-2
	assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all() and torch.isfinite(dv.float()).all()


def test_c5_dropout_wide_heads_bf16_causal_fwd_bwd():
	# B8 S2048 H16 D256 bf16 causal, dropout 0.1, seed 42
	dtype = torch.bfloat16
	B, S, H, D = 8, 2048, 16, 256
	q, k, v = _gen((B, S, H, D), 0, 0.5, dtype), _gen((B, S, H, D), 1, 0.5, dtype), _gen((B, S, H, D), 2, 0.5, dtype)
	do = _gen((B, S, H, D), 3, 1.0, dtype)
	o, lse = op.fwd(q, k, v, None, None, None, 0.1, True, 42)
	grads = op.bwd(q, k, v, o, lse, do, None, None, None, 0.1, True, 42)
	for b, h in ((0, 0), (7, 15)):
		_check_group(q, k, v, do, o, lse, grads, b, h, 1, dtype, causal=True, p_drop=0.1, seed=42)
	# LSE does not depend on dropout (up to fp32 rounding: the two variants of the kernel hold different running references)
	_, lse0 = op.fwd(q, k, v, causal=True)
	assert torch.allclose(lse, lse0, rtol=0, atol=1e-5)


@pytest.mark.parametrize("B,S,Hq,Hkv,D,dtype,p", [
	(8, 800, 16, 8, 128, torch.bfloat16, 0.0),    # 7 key tiles (odd: the middle one has no partner), ragged last tile
	(4, 2048, 16, 8, 64, torch.float16, 0.0),     # 16 key tiles -> 8 pairs x 32 groups
	(8, 1024, 8, 8, 128, torch.bfloat16, 0.15),   # dropout, no grouping
	(2, 2000, 32, 16, 64, torch.bfloat16, 0.0),   # 16 tiles, ragged, 2 q-heads per kv-head
])
def test_paired_key_tiles_of_causal_self_attention(B, S, Hq, Hkv, D, dtype, p):
	"""Causal self-attention on grids that fill the chip in whole rounds: a workgroup of the dK/dV kernel takes the key
	tiles t and ntiles - 1 - t one after the other, walking the query tiles down for the first and up for the second with
	the q-heads innermost.  dK / dV (and everything else) of whole KV groups against the oracle, and run-to-run identical."""
	r = Hq // Hkv
	assert ((-(-S // 128) + 1) // 2 * B * Hkv) % 256 == 0  # the launcher pairs on such grids
	q, k, v = _gen((B, S, Hq, D), 0, 0.5, dtype), _gen((B, S, Hkv, D), 1, 0.5, dtype), _gen((B, S, Hkv, D), 2, 0.5, dtype)
	do = _gen((B, S, Hq, D), 3, 1.0, dtype)
	o, lse = op.fwd(q, k, v, None, None, None, p, True, 77)
	grads = op.bwd(q, k, v, o, lse, do, None, None, None, p, True, 77)
	for b, g in ((0, 0), (B - 1, Hkv - 1), (B // 2, 1)):
		_check_group(q, k, v, do, o, lse, grads, b, g, r, dtype, causal=True, p_drop=p, seed=77)
	again = op.bwd(q, k, v, o, lse, do, None, None, None, p, True, 77)
	for a, b_ in zip(grads, again):
		assert torch.equal(a, b_)


@pytest.mark.parametrize("D,S,P,Hq,Hkv", [(64, 16640, 8192, 4, 2), (128, 8448, 4096, 8, 2), (128, 4096, 2048, 32, 8)])
def test_long_causal_rows_reproduce_their_prefix(D, S, P, Hq, Hkv):
	"""The forward and dQ kernels run as 128-row workgroups, two per CU, while the K and V of a head fit an XCD's L2, and
	as 256-row workgroups beyond (the first two shapes; the third stays within).  Out of the oracle's reach at these
	lengths, but under a causal mask the first P rows of O, LSE and dQ depend on the first P rows and keys only: they
	must agree with the problem cut to P, which takes the other tiling."""
	dtype = torch.bfloat16
	q, k, v = _gen((1, S, Hq, D), 0, 0.5, dtype), _gen((1, S, Hkv, D), 1, 0.5, dtype), _gen((1, S, Hkv, D), 2, 0.5, dtype)
	do = _gen((1, S, Hq, D), 3, 1.0, dtype)
	o, lse = op.fwd(q, k, v, causal=True)
	dq, dk, dv = op.bwd(q, k, v, o, lse, do, causal=True)
	qp, kp, vp, dop = (t[:, :P].contiguous() for t in (q, k, v, do))
	o_p, lse_p = op.fwd(qp, kp, vp, causal=True)
	dq_p, _, _ = op.bwd(qp, kp, vp, o_p, lse_p, dop, causal=True)
	assert (o[:, :P].float() - o_p.float()).abs().max().item() <= TOL_O[dtype]
	assert (lse[:, :, :P] - lse_p).abs().max().item() <= 2e-3
	rel = float((dq[:, :P].float() - dq_p.float()).norm() / dq_p.float().norm())
	assert rel <= TOL_GRAD_REL_L2, rel
	o1, _ = op.fwd(q, k, torch.ones_like(v), causal=True)
	assert (o1.float() - 1).abs().max().item() <= 1e-2
	for t in (dq, dk, dv):
		assert torch.isfinite(t.float()).all()


def test_bias_gradient_at_c3_size_stays_within_the_size_of_the_bias():
	"""A bias [B, 1, S, S] at the c3 shape (B8 H16 S2048 D64) that asks for its gradient: the gradient buffer has the
	shape of the bias (fp32, 128 MiB) - not one entry per (batch, head), 2 GiB - because the dQ kernel sums over the
	heads itself.  Peak allocation of the backward call is checked as well as the values (fp32 evaluation in torch
	on the GPU, one batch row at a time); without `bias_grad` no gradient is formed, as in the reference
	(_flash_attention.py:88)."""
	dtype = torch.bfloat16
	B, S, H, D = 8, 2048, 16, 64
	q, k, v = _gen((B, S, H, D), 0, 0.5, dtype), _gen((B, S, H, D), 1, 0.5, dtype), _gen((B, S, H, D), 2, 0.5, dtype)
	do = _gen((B, S, H, D), 3, 1.0, dtype)
	bias = _gen((B, 1, S, S), 4, 1.0, dtype).requires_grad_()
	qd = q.clone().requires_grad_()
	out = op.flash_attention(qd, k, v, bias=bias, bias_grad=True)
	torch.cuda.synchronize()
	torch.cuda.reset_peak_memory_stats()
	base = torch.cuda.memory_allocated()
	out.backward(do)
	torch.cuda.synchronize()
	peak = torch.cuda.max_memory_allocated() - base
	# dq, dk, dv (3 x 32 MiB), delta scratch, the fp32 gradient buffer (128 MiB) and its copy in the bias's dtype (64 MiB)
	assert peak <= 384 << 20, f"backward allocated {peak >> 20} MiB"
	assert bias.grad is not None and bias.grad.shape == bias.shape and bias.grad.dtype == dtype
	scale = D ** -0.5
	for b in (0, 5):
		qf, kf, vf, dof = (t[b].float().transpose(0, 1) for t in (q, k, v, do))  # [H, S, D]
		sc = qf @ kf.transpose(1, 2) * scale + bias.detach()[b].float()
		pr = torch.softmax(sc, dim=-1)
		dp = dof @ vf.transpose(1, 2)
		ds = pr * (dp - (dp * pr).sum(-1, keepdim=True))
		ref = ds.sum(0)
		e = float((bias.grad[b, 0].float() - ref).norm() / ref.norm())
		assert e <= TOL_GRAD_REL_L2, f"dbias of batch row {b}: rel-L2 {e:.3e}"
		dq_ref = (ds @ kf * scale).transpose(0, 1)
		e = float((qd.grad[b].float() - dq_ref).norm() / dq_ref.norm())
		assert e <= TOL_GRAD_REL_L2, f"dq of batch row {b}: rel-L2 {e:.3e}"
	# off by default
	b2 = bias.detach().clone().requires_grad_()
	q2 = q.clone().requires_grad_()
	op.flash_attention(q2, k, v, bias=b2).backward(do)
	assert b2.grad is None and torch.equal(q2.grad, qd.grad)
