"""Pins the CPU oracle: known-answer vectors, closed forms, invariants, finite
differences and the committed golden fixtures.  No GPU."""

import math
import os

import numpy as np
import pytest
import scipy.special

import fa2_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))


def _hex(words):
	return " ".join("%08x" % int(x) for x in words)


# Random123 kat_vectors, philox4x32 with 10 rounds
@pytest.mark.parametrize(
	"ctr,key,expect",
	[
		((0, 0, 0, 0), (0, 0), "6627e8d5 e169c58d bc57ac4c 9b00dbd8"),
		((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, "408f276d 41c83b0e a20bc7c6 6d5451fd"),
		((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0), "d16cfe09 94fdcceb 5001e420 24126ea1"),
	],
)
def test_philox_known_answers(ctr, key, expect):
	assert _hex(O.philox4x32_10(*[np.uint32(c) for c in ctr], *key)) == expect


def test_dropout_mask_definition_and_rate():
	B, H, Sq, Sk, p, seed = 2, 3, 37, 50, 0.25, (7 << 32) | 12345
	keep = O.dropout_keep_mask(seed, p, B, H, Sq, Sk)
	thr = O.dropout_threshold(p)
	assert thr == 1 << 14
	# every element against a scalar evaluation of the definition: one call per (two rows, four keys), eight 16-bit
	# values, element (i, j) owns value (i & 1) * 4 + (j & 3) = half (v & 1) of word v >> 1
	for (b, h, i, j) in [(0, 0, 0, 0), (1, 2, 36, 49), (0, 1, 5, 6), (1, 0, 20, 3), (0, 2, 21, 3), (1, 1, 1, 47), (0, 0, 36, 0)]:
		w = O.philox4x32_10(np.uint32(j >> 2), np.uint32(i >> 1), np.uint32(h), np.uint32(b), seed & 0xFFFFFFFF, seed >> 32)
		v = (i & 1) * 4 + (j & 3)
		val = (int(w[v >> 1]) >> 16) if (v & 1) else (int(w[v >> 1]) & 0xFFFF)
		assert bool(keep[b, h, i, j]) == (val >= thr)
	# the eight values of one call are used once each: rows (2m, 2m + 1) x keys (4n .. 4n + 3)
	w = [int(x) for x in O.philox4x32_10(np.uint32(3), np.uint32(4), np.uint32(1), np.uint32(0), seed & 0xFFFFFFFF, seed >> 32)]
	vals = [(w[v >> 1] >> 16) if (v & 1) else (w[v >> 1] & 0xFFFF) for v in range(8)]
	assert np.array_equal(keep[0, 1, 8:10, 12:16], (np.array(vals).reshape(2, 4) >= thr))
	big = O.dropout_keep_mask(42, 0.1, 1, 2, 512, 512)
	n = big.size
	assert abs(big.mean() - 0.9) < 4 * np.sqrt(0.09 / n)
	# slices of a larger problem reproduce through pos_offset
	sl = O.dropout_keep_mask(seed, p, 1, 1, 7, Sk, pos_offset=(1, 2, 30))
	assert np.array_equal(sl[0, 0], keep[1, 2, 30:37])
	assert O.dropout_keep_mask(1, 0.0, 1, 1, 8, 8).all()


@pytest.mark.parametrize("p", [0.0, 1e-6, 0.1, 0.25, 0.3, 0.5, 0.999, 0.99999])
def test_dropout_keep_scale_makes_the_expectation_exact(p):
	"""Kept values are scaled by the reciprocal of the keep probability the 16-bit threshold really gives: over the
	65536 equally likely values of an element, sum(keep) * scale is exactly the number of values - so E[O] is the
	output without dropout for every p, also where p is not a multiple of 2^-16 and below 2^-16 (nothing dropped,
	nothing rescaled).  The reference's factor 1 / (1 - p) (_forward_triton.py:435-438) is the same number for the
	probability that is realised."""
	thr = O.dropout_threshold(p)
	kept = int((np.arange(65536) >= thr).sum())
	assert kept >= 1
	assert kept * O.dropout_keep_scale(p) == pytest.approx(65536.0, rel=1e-15)
	assert abs(O.dropout_keep_scale(p) - 1.0 / (1.0 - float(np.float32(p)))) <= 2.0 ** -16 * O.dropout_keep_scale(p) ** 2 * 1.0001 or thr == 0xFFFF


def _rand(rng, B, Sq, Sk, Hq, Hkv, D):
	return (rng.normal(size=(B, Sq, Hq, D)), rng.normal(size=(B, Sk, Hkv, D)), rng.normal(size=(B, Sk, Hkv, D)),
	        rng.normal(size=(B, Sq, Hq, D)))


def test_forward_matches_scipy_softmax():
	rng = np.random.default_rng(1)
	q, k, v, _ = _rand(rng, 2, 9, 11, 4, 4, 8)
	bias = rng.normal(size=(2, 4, 9, 11))
	o, lse = O.attention_fwd(q, k, v, bias=bias, scale=0.3)
	s = np.einsum("bihd,bjhd->bhij", q, k) * 0.3 + bias
	p = scipy.special.softmax(s, axis=-1)
	assert np.allclose(o, np.einsum("bhij,bjhd->bihd", p, v), atol=1e-12)
	assert np.allclose(lse, scipy.special.logsumexp(s, axis=-1), atol=1e-12)


def test_forward_invariants():
	rng = np.random.default_rng(2)
	q, k, v, _ = _rand(rng, 2, 16, 16, 4, 2, 8)
	# V = 1 -> O = 1
	o, _ = O.attention_fwd(q, k, np.ones_like(v), causal=True)
	assert np.allclose(o, 1.0)
	# Q = 0, causal -> prefix mean of V (per kv group)
	o, _ = O.attention_fwd(np.zeros_like(q), k, v, causal=True)
	pm = np.cumsum(v, axis=1) / np.arange(1, 17)[None, :, None, None]
	assert np.allclose(o, np.repeat(pm, 2, axis=2))
	# key permutation leaves O unchanged without a causal mask
	perm = rng.permutation(16)
	o1, l1 = O.attention_fwd(q, k, v)
	o2, l2 = O.attention_fwd(q, k[:, perm], v[:, perm])
	assert np.allclose(o1, o2) and np.allclose(l1, l2)
	# a per-row constant in the bias does not change O and shifts LSE
	c = rng.normal(size=(2, 4, 16, 1))
	o3, l3 = O.attention_fwd(q, k, v, bias=np.broadcast_to(c, (2, 4, 16, 16)))
	assert np.allclose(o1, o3) and np.allclose(l3, l1 + c[..., 0])
	# GQA == MHA over repeated K/V, q-head h -> kv-head h // r
	o4, _ = O.attention_fwd(q, np.repeat(k, 2, axis=2), np.repeat(v, 2, axis=2))
	assert np.allclose(o1, o4)


def test_causal_alignment_and_fully_masked_rows():
	rng = np.random.default_rng(3)
	# Sq > Sk: rows i < Sq - Sk see no key -> zeros and LSE = -inf (bottom-right aligned)
	q, k, v, _ = _rand(rng, 1, 6, 4, 2, 2, 4)
	o, lse = O.attention_fwd(q, k, v, causal=True)
	assert np.all(o[:, :2] == 0) and np.all(np.isneginf(lse[:, :, :2]))
	ok = O.allowed_mask(1, 6, 4, True)[0]
	assert np.array_equal(ok, np.arange(4)[None, :] <= np.arange(6)[:, None] - 2)
	# Sq < Sk: row i sees keys <= i + (Sk - Sq)
	assert np.array_equal(O.allowed_mask(1, 2, 5, True)[0], np.array([[1, 1, 1, 1, 0], [1, 1, 1, 1, 1]], bool))
	# seqlens: keys beyond len masked, padded rows zero
	q, k, v, _ = _rand(rng, 2, 8, 8, 2, 2, 4)
	o, lse = O.attention_fwd(q, k, v, seqlens=[5, 8])
	o5, _ = O.attention_fwd(q[:1, :5], k[:1, :5], v[:1, :5])
	assert np.allclose(o[0, :5], o5[0]) and np.all(o[0, 5:] == 0)


def test_bias_broadcast_rules():
	rng = np.random.default_rng(4)
	B, S, Hq, Hkv, D = 2, 8, 4, 2, 4
	q, k, v, _ = _rand(rng, B, S, S, Hq, Hkv, D)
	full = rng.normal(size=(B, Hq, S, S))
	for shape in [(1, 1), (B, 1), (1, Hq), (B, Hq)]:
		b = full[: shape[0], : shape[1]]
		o1, _ = O.attention_fwd(q, k, v, bias=b)
		o2, _ = O.attention_fwd(q, k, v, bias=np.broadcast_to(b, (B, Hq, S, S)))
		assert np.allclose(o1, o2)
	bg = full[:, :Hkv]
	o1, _ = O.attention_fwd(q, k, v, bias=bg)
	o2, _ = O.attention_fwd(q, k, v, bias=np.repeat(bg, 2, axis=1))
	assert np.allclose(o1, o2)
	with pytest.raises(ValueError):
		O.attention_fwd(q, k, v, bias=full[:, :3])
	with pytest.raises(ValueError):
		O.attention_fwd(q, k, v, bias=full[..., :7])
	# mask -> finfo.min bias equals boolean masking when each row keeps a key
	valid = np.arange(S)[None, :] < np.array([5, 8])[:, None]
	mb = np.broadcast_to(np.where(valid[:, None, None, :], 0.0, np.finfo(np.float32).min), (2, 1, S, S))
	o3, _ = O.attention_fwd(q, k, v, bias=mb)
	o4, _ = O.attention_fwd(q[:1], k[:1, :5], v[:1, :5])
	assert np.allclose(o3[0], o4[0])


@pytest.mark.parametrize(
	"kw",
	[dict(), dict(causal=True), dict(bias=True), dict(causal=True, p_drop=0.3, seed=7), dict(seqlens=[5, 6]),
	 dict(causal=True, scale=0.7), dict(softcap=0.8), dict(causal=True, bias=True, softcap=1.5, p_drop=0.2, seed=3),
	 dict(window=(2, 1), kv_lens=[6, 4])],
)
def test_backward_matches_finite_differences(kw):
	rng = np.random.default_rng(5)
	B, Sq, Sk, Hq, Hkv, D = 2, 6, 6, 4, 2, 4
	q, k, v, dO = _rand(rng, B, Sq, Sk, Hq, Hkv, D)
	kw = dict(kw)
	if kw.get("bias") is True:
		kw["bias"] = rng.normal(size=(B, Hkv, Sq, Sk))
	grads = O.attention_bwd(q, k, v, dO, **kw)
	f = lambda *a: np.sum(O.attention_fwd(*a, **kw)[0] * dO)
	eps = 1e-6
	for idx, g in enumerate(grads):
		xs = [q, k, v]
		num = np.zeros_like(xs[idx])
		it = np.nditer(xs[idx], flags=["multi_index"])
		for _ in it:
			mi = it.multi_index
			a = [t.copy() for t in xs]
			b = [t.copy() for t in xs]
			a[idx][mi] += eps
			b[idx][mi] -= eps
			num[mi] = (f(*a) - f(*b)) / (2 * eps)
		assert np.abs(num - g).max() < 1e-7


@pytest.mark.parametrize("bshape", [(2, 4), (2, 2), (2, 1), (1, 4), (1, 1)], ids=["bBhH", "bBhKV", "bBh1", "b1hH", "b1h1"])
@pytest.mark.parametrize("kw", [dict(), dict(causal=True, p_drop=0.3, seed=7), dict(softcap=0.8, window=(3, 1))])
def test_bias_gradient_matches_finite_differences(bshape, kw):
	"""dbias of attention_bwd(return_dbias=True) against central differences in the entries of the bias, for every
	broadcast shape of the bias (the gradient of a broadcast entry is the sum over the positions it feeds)."""
	rng = np.random.default_rng(11)
	B, Sq, Sk, Hq, Hkv, D = 2, 5, 6, 4, 2, 4
	q, k, v, dO = _rand(rng, B, Sq, Sk, Hq, Hkv, D)
	bias = rng.normal(size=(*bshape, Sq, Sk))
	dbias = O.attention_bwd(q, k, v, dO, bias=bias, return_dbias=True, **kw)[3]
	assert dbias.shape == bias.shape
	f = lambda bb: np.sum(O.attention_fwd(q, k, v, bias=bb, **kw)[0] * dO)
	eps = 1e-6
	num = np.zeros_like(bias)
	it = np.nditer(bias, flags=["multi_index"])
	for _ in it:
		mi = it.multi_index
		a, b = bias.copy(), bias.copy()
		a[mi] += eps
		b[mi] -= eps
		num[mi] = (f(a) - f(b)) / (2 * eps)
	assert np.abs(num - dbias).max() < 1e-7
	# the first three results do not depend on the flag
	for x, y in zip(O.attention_bwd(q, k, v, dO, bias=bias, **kw), O.attention_bwd(q, k, v, dO, bias=bias, return_dbias=True, **kw)):
		assert np.array_equal(x, y)


def test_backward_identities():
	rng = np.random.default_rng(6)
	q, k, v, dO = _rand(rng, 1, 12, 12, 4, 2, 8)
	o, lse, p, _ = O.attention_fwd(q, k, v, causal=True, return_probs=True)
	assert np.allclose(p.sum(-1), 1.0)
	# delta = rowsum(dO * O) = rowsum(P * dP)
	vf = np.repeat(v, 2, axis=2)
	dp = np.einsum("bihd,bjhd->bhij", dO, vf)
	assert np.allclose(np.einsum("bihd,bihd->bhi", o, dO), (p * dp).sum(-1))
	# dK/dV of a group = sum of the MHA gradients over its q-heads
	dq, dk, dv = O.attention_bwd(q, k, v, dO, causal=True)
	dq2, dk2, dv2 = O.attention_bwd(q, np.repeat(k, 2, axis=2), vf, dO, causal=True)
	assert np.allclose(dq, dq2)
	assert np.allclose(dk, dk2.reshape(1, 12, 2, 2, 8).sum(3)) and np.allclose(dv, dv2.reshape(1, 12, 2, 2, 8).sum(3))


def test_key_lengths_equal_an_explicit_key_mask():
	"""kv_lens (key padding only) = -inf bias on the padded keys; rows and the causal offset stay as they are."""
	rng = np.random.default_rng(11)
	B, Sq, Sk, Hq, Hkv, D = 2, 10, 14, 4, 2, 8
	q, k, v, dO = _rand(rng, B, Sq, Sk, Hq, Hkv, D)
	lens = [9, 14]
	big = np.zeros((B, 1, Sq, Sk))
	big[0, :, :, 9:] = -1e30
	for causal in (False, True):
		o, lse = O.attention_fwd(q, k, v, causal=causal, kv_lens=lens)
		o2, lse2 = O.attention_fwd(q, k, v, bias=big, causal=causal)
		assert np.allclose(o, o2) and np.allclose(lse, lse2)
		for a, b in zip(O.attention_bwd(q, k, v, dO, causal=causal, kv_lens=lens), O.attention_bwd(q, k, v, dO, bias=big, causal=causal)):
			assert np.allclose(a, b)
	# a length of zero: no key at all
	o, lse = O.attention_fwd(q, k, v, kv_lens=[0, 14])
	assert np.all(o[0] == 0) and np.all(np.isneginf(lse[0])) and np.all(np.isfinite(lse[1]))


def test_key_lengths_keep_the_window_aligned_to_the_full_key_count():
	"""Chosen semantics, on purpose different from the reference's naive attention: there a key_padding_mask moves the
	window (row i is aligned with key i + valid_keys - Sq, refrence_call.py:58-66); `kv_lens` is padding at the end of
	a key axis whose positions keep their meaning, so row i stays aligned with key i + Sk - Sq and the length only
	removes keys.  Written out for Sq 3, Sk 8, window (1, 1), kv_len 6."""
	got = O.allowed_mask(1, 3, 8, False, kv_lens=[6], window=(1, 1))[0].astype(int)
	expect = np.array([
		# keys 0 1 2 3 4 5 | 6 7 (padding)
		[0, 0, 0, 0, 1, 1, 0, 0],  # row 0 <-> key 5: keys 4..6, key 6 is padding
		[0, 0, 0, 0, 0, 1, 0, 0],  # row 1 <-> key 6: keys 5..7, only 5 is valid
		[0, 0, 0, 0, 0, 0, 0, 0],  # row 2 <-> key 7: keys 6..7, none valid -> O = 0, lse = -inf
	])
	assert np.array_equal(got, expect)
	# the reference's alignment (to the valid length: row i <-> key i + 6 - 3) would have given another set of keys
	ref_style = O.allowed_mask(1, 3, 6, False, window=(1, 1))[0].astype(int)
	assert not np.array_equal(got[:, :6], ref_style)
	# same with the causal flag: row i sees keys <= i + Sk - Sq that are valid
	got = O.allowed_mask(1, 3, 8, True, kv_lens=[6])[0]
	assert np.array_equal(got, (np.arange(8)[None, :] <= np.arange(3)[:, None] + 5) & (np.arange(8)[None, :] < 6))
	rng = np.random.default_rng(3)
	q, k, v = rng.normal(size=(1, 3, 2, 4)), rng.normal(size=(1, 8, 2, 4)), rng.normal(size=(1, 8, 2, 4))
	o, lse = O.attention_fwd(q, k, v, kv_lens=[6], window=(1, 1))
	assert np.all(o[0, 2] == 0) and np.all(np.isneginf(lse[0, :, 2]))
	assert np.allclose(o[0, 1], v[0, 5])  # a single key: its value


def test_sliding_window_is_the_local_mask_of_the_naive_reference():
	"""refrence_call.py:55-75 with no padding masks: a key is hidden iff col > min(row + sk - sq + right, sk) or
	col < row + sk - sq - left (left >= 0), or col > row + sk - sq + right (left < 0); causal sets right = 0 (:36-37).
	The oracle's window must be that mask wherever both bounds are given or only the right one; rows hidden
	entirely give zeros (:80-82)."""
	rng = np.random.default_rng(3)
	for (Sq, Sk) in ((12, 12), (7, 15), (15, 7)):
		row = np.arange(Sq)[:, None]
		col = np.arange(Sk)[None, :]
		for (left, right) in ((3, 0), (2, 2), (0, 0), (-1, 2), (-1, 0), (5, 1), (100, 100)):
			if left < 0:
				hidden = col > row + Sk - Sq + right
			else:
				hidden = (col > np.minimum(row + Sk - Sq + right, Sk)) | (col < row + Sk - Sq - left)
			ok = O.allowed_mask(1, Sq, Sk, False, window=(left, right))[0]
			assert np.array_equal(ok, ~hidden), (Sq, Sk, left, right)
		assert np.array_equal(O.allowed_mask(1, Sq, Sk, True, window=(4, 9))[0], O.allowed_mask(1, Sq, Sk, False, window=(4, 0))[0])
		assert np.array_equal(O.allowed_mask(1, Sq, Sk, True)[0], O.allowed_mask(1, Sq, Sk, False, window=(-1, 0))[0])
	# equals an explicit -inf bias; fully hidden rows give O = 0
	B, Sq, Sk, Hq, Hkv, D = 1, 9, 14, 2, 1, 4
	q, k, v, dO = _rand(rng, B, Sq, Sk, Hq, Hkv, D)
	ok = O.allowed_mask(B, Sq, Sk, False, window=(2, 1))
	big = np.where(ok[:, None], 0.0, -1e30)
	o, lse = O.attention_fwd(q, k, v, window=(2, 1))
	o2, lse2 = O.attention_fwd(q, k, v, bias=big)
	assert np.allclose(o, o2) and np.allclose(lse, lse2)
	for a, b in zip(O.attention_bwd(q, k, v, dO, window=(2, 1)), O.attention_bwd(q, k, v, dO, bias=big)):
		assert np.allclose(a, b)
	o, lse = O.attention_fwd(q[:, :, :, :], k[:, :3], v[:, :3], window=(1, 0))  # Sq 9 > Sk 3: the first rows see nothing
	assert np.all(o[:, :5] == 0) and np.all(np.isneginf(lse[..., :5]))


def test_softcap_is_the_tanh_capping_of_the_naive_reference():
	"""refrence_call.py:48-51: scores / softcap -> tanh -> * softcap, on the scaled scores, before masks and bias.
	Against scipy's softmax of the formula written out; a large cap changes nothing; scores stay within +-cap."""
	rng = np.random.default_rng(11)
	B, Sq, Sk, Hq, Hkv, D = 2, 7, 9, 4, 2, 8
	q, k, v, _ = _rand(rng, B, Sq, Sk, Hq, Hkv, D)
	q = q * 3.0
	bias = rng.normal(size=(B, Hq, Sq, Sk))
	cap = 1.3
	kr = np.repeat(k, 2, axis=2)
	vr = np.repeat(v, 2, axis=2)
	sc = np.einsum("bthd,bshd->bhts", q / math.sqrt(D), kr)
	assert np.abs(sc).max() > 2 * cap  # the cap bites
	x = np.tanh(sc / cap) * cap + bias
	want = np.einsum("bhts,bshd->bthd", scipy.special.softmax(x, axis=-1), vr)
	o, lse = O.attention_fwd(q, k, v, bias=bias, softcap=cap)
	assert np.allclose(o, want)
	assert np.allclose(lse, scipy.special.logsumexp(x, axis=-1))
	o_big, _ = O.attention_fwd(q, k, v, bias=bias, softcap=1e9)
	o_off, _ = O.attention_fwd(q, k, v, bias=bias)
	assert np.allclose(o_big, o_off, atol=1e-9)


def test_blockwise_restatement_equals_closed_form():
	rng = np.random.default_rng(7)
	B, S, Hq, Hkv, D = 1, 256, 4, 2, 16
	q, k, v, dO = _rand(rng, B, S, S, Hq, Hkv, D)
	bias = rng.normal(size=(B, 1, S, S))
	o, (dq, dk, dv) = O.jax_platform_call(q, k, v, bias=bias, dtype=np.float64, with_grads_for=dO, blocksize_q=64, blocksize_k=128)
	o2, _ = O.attention_fwd(q, k, v, bias=bias)
	g2 = O.attention_bwd(q, k, v, dO, bias=bias)
	assert np.abs(o - o2).max() < 1e-6
	for a, b in zip((dq, dk, dv), g2):
		assert np.abs(a - b).max() < 1e-5
	# with a mask the reference also skips blocks above the diagonal
	qt, kt, vt = (np.ascontiguousarray(np.swapaxes(x, 1, 2)) for x in (q, np.repeat(k, 2, 2), np.repeat(v, 2, 2)))
	tri = np.tril(np.ones((S, S), bool))[None, None]
	ob, lse = O.blockwise_fwd(qt / 4.0, kt, vt, mask=tri, dtype=np.float64, blocksize_q=64, blocksize_k=64)
	oc, _ = O.attention_fwd(q, k, v, causal=True)
	assert np.abs(np.swapaxes(ob, 1, 2) - oc).max() < 1e-6
	# ... and so does the backward (the causal leg of the CPU baseline runs exactly this)
	oc2, gc = O.jax_platform_call(q, k, v, dtype=np.float64, with_grads_for=dO, mask=tri, blocksize_q=64, blocksize_k=64)
	assert np.abs(oc2 - oc).max() < 1e-6
	for a, b in zip(gc, O.attention_bwd(q, k, v, dO, causal=True)):
		assert np.abs(a - b).max() < 1e-5


def test_bf16_helpers_round_trip():
	x = np.array([1.0, 1.00390625, 1.005859375, -3.3895314e38, 65504.0, 1e-40], np.float32)
	r = O.round_bf16(x)
	assert r[0] == 1.0 and r[1] == 1.0 and r[2] == 1.0078125  # ties-to-even, then up
	assert np.array_equal(O.from_bf16_bits(O.to_bf16_bits(r)), r)


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(os.path.join(HERE, "golden")) if f.endswith(".npz")))
def test_golden_fixtures(name):
	"""The committed fixtures (made by tests/golden/make_golden.py from this oracle) still reproduce."""
	z = np.load(os.path.join(HERE, "golden", name))
	kw = dict(causal=bool(z["causal"]), p_drop=float(z["p_drop"]), seed=int(z["seed"]))
	if "bias" in z:
		kw["bias"] = z["bias"]
	if "seqlens" in z:
		kw["seqlens"] = z["seqlens"]
	o, lse = O.attention_fwd(z["q"], z["k"], z["v"], **kw)
	dq, dk, dv = O.attention_bwd(z["q"], z["k"], z["v"], z["dout"], **kw)
	fin = np.isfinite(z["lse"])
	assert np.allclose(o, z["o"], atol=1e-6) and np.allclose(lse[fin], z["lse"][fin], atol=1e-6)
	assert np.array_equal(np.isfinite(lse), fin)
	for a, b in ((dq, z["dq"]), (dk, z["dk"]), (dv, z["dv"])):
		assert np.allclose(a, b, atol=1e-6)
	if float(z["p_drop"]) > 0:
		B, Sq, Hq, _ = z["q"].shape
		keep = O.dropout_keep_mask(int(z["seed"]), float(z["p_drop"]), B, Hq, Sq, z["k"].shape[1])
		assert np.array_equal(np.unpackbits(z["keep_bits"])[: keep.size].astype(bool).reshape(keep.shape), keep)


def test_backward_with_the_stored_output():
	"""`o_stored` only replaces O in delta = rowsum(O * dO): the exact O reproduces the default result, and with a single
	key (P = 1) the exact gradients of q and k cancel to zero while a rounded O leaves its rounding error, summed over the rows."""
	rng = np.random.default_rng(5)
	q, k, v, do = (rng.standard_normal(s) for s in ((2, 9, 2, 8), (2, 5, 1, 8), (2, 5, 1, 8), (2, 9, 2, 8)))
	o, _ = O.attention_fwd(q, k, v, causal=True)
	ref = O.attention_bwd(q, k, v, do, causal=True)
	same = O.attention_bwd(q, k, v, do, causal=True, o_stored=o)
	for a, b in zip(ref, same):
		assert np.array_equal(a, b)
	k1, v1 = k[:, :1], v[:, :1]
	o1, _ = O.attention_fwd(q, k1, v1)
	exact = O.attention_bwd(q, k1, v1, do)
	assert np.abs(exact[0]).max() <= 1e-12 and np.abs(exact[1]).max() <= 1e-12
	noisy = O.attention_bwd(q, k1, v1, do, o_stored=o1 + 1e-3)
	delta_err = 1e-3 * do.sum(-1)  # [B, Sq, H]: the error of delta; dS = -P * that, P = 1
	want_dq = -delta_err[..., None] * np.repeat(k1, 2, axis=2) / np.sqrt(8)
	assert np.allclose(noisy[0], want_dq, atol=1e-12)
	assert np.allclose(noisy[2], exact[2])  # dV does not involve delta
