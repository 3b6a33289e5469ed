"""GPU parity: the HIP path, called through the C ABI of libfa2_hip.so,
against the NumPy oracle on the same seeded inputs.

Tolerances (BASELINE north star): max-abs error on O <= 2e-2 (bf16) / 5e-3
(fp16) and relative L2 error on dQ/dK/dV <= 1e-2, against an fp64/fp32
evaluation; the dropout keep-mask is bit-exact.
"""

import os

import numpy as np
import pytest
import torch

import fa2_oracle as O
from _cases import TOL_O, check_forward, check_grads, f64, make_inputs
from jax_flash_attn2 import _hip_op as op

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HERE = os.path.dirname(os.path.abspath(__file__))


def _dev(t):
	return None if t is None else t.to(DEV)


def _run_case(B, Sq, Sk, Hq, Hkv, D, dtype, causal=False, bias_shape=None, p=0.0, seed=0, seqlens=None, scale=None,
              bias_dtype=None, data_seed=0, qk_scale=None):
	q, k, v, do, bias = make_inputs(B, Sq, Sk, Hq, Hkv, D, dtype, data_seed, bias_shape, bias_dtype=bias_dtype, qk_scale=qk_scale)
	sl = None if seqlens is None else torch.tensor(seqlens, dtype=torch.int32)
	kw = dict(causal=causal, p_drop=p, seed=seed, seqlens=seqlens, scale=scale)
	o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), **kw)
	o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), _dev(sl), scale, p, causal, seed)
	g = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), _dev(sl), scale, p, causal, seed)
	torch.cuda.synchronize()
	what = f"B{B} Sq{Sq} Sk{Sk} Hq{Hq} Hkv{Hkv} D{D} {dtype} causal={causal} bias={bias_shape} p={p} seqlens={seqlens}"
	check_forward(o, lse, o_ref, lse_ref, dtype, what)
	stored = None
	if min(np.abs(x).max() for x in g_ref) <= 1e-10:
		# a gradient that cancels exactly (a single key ...): what the rounding of the stored O leaves of it
		o_st = torch.from_numpy(np.nan_to_num(o_ref)).to(dtype).to(torch.float64).numpy()
		stored = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), o_stored=o_st, **kw)
	check_grads(g, g_ref, what, stored)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_basic_shapes(dtype, D, causal):
	_run_case(2, 320, 320, 4, 2, D, dtype, causal=causal)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("qk_scale,score_range", [(2.1, 20), (4.2, 80)])
def test_large_logits(dtype, qk_scale, score_range):
	"""Scores of realistic and of extreme magnitude (within about +-20 and +-80; the other cases stay within +-5):
	the softmax scale is applied to the fp32 result of q.k as the reference does (_forward_triton.py:281), so the
	tolerances hold at any magnitude.  v keeps its usual size, so that O stays of order 1."""
	q, k, *_ = make_inputs(2, 384, 384, 4, 2, 128, dtype, qk_scale=qk_scale)
	sc = torch.einsum("bihd,bjhd->bhij", q.float(), k.float().repeat_interleave(2, dim=2)) / 128**0.5
	assert 0.7 * score_range <= sc.abs().max().item() <= 1.3 * score_range
	_run_case(2, 384, 384, 4, 2, 128, dtype, causal=True, qk_scale=qk_scale)
	_run_case(1, 200, 333, 4, 4, 64, dtype, causal=False, qk_scale=qk_scale, data_seed=1)
	_run_case(1, 160, 160, 2, 1, 256, dtype, causal=True, qk_scale=qk_scale, data_seed=2)
	_run_case(1, 160, 160, 2, 2, 128, dtype, causal=True, qk_scale=qk_scale, p=0.1, seed=5, data_seed=3)
	# head dim 256, many tiles without masking: the row reference has to be raised in later tiles too (with and without dropout)
	_run_case(1, 96, 448, 2, 1, 256, dtype, causal=False, qk_scale=qk_scale, p=0.1, seed=7, data_seed=4)
	_run_case(1, 72, 520, 2, 2, 256, dtype, causal=False, qk_scale=qk_scale, data_seed=5)
	# the same at head dim 128, whose four-wave workgroups take the pipelined path for tiles without masking
	_run_case(1, 96, 448, 2, 1, 128, dtype, causal=False, qk_scale=qk_scale, data_seed=6)
	_run_case(1, 200, 520, 4, 2, 128, dtype, causal=True, qk_scale=qk_scale, data_seed=7)


@pytest.mark.parametrize(
	"Sq,Sk",
	[(1, 1), (1, 77), (7, 5), (33, 33), (63, 65), (128, 128), (129, 257), (257, 129), (200, 333), (500, 64), (64, 500)],
)
@pytest.mark.parametrize("causal", [False, True])
def test_ragged_and_cross_lengths(Sq, Sk, causal):
	"""Ragged tiles, Sq != Sk with the bottom-right aligned causal mask, rows without any allowed key."""
	_run_case(2, Sq, Sk, 4, 2, 128, torch.bfloat16, causal=causal)
	_run_case(1, Sq, Sk, 2, 1, 64, torch.float16, causal=causal, data_seed=1)


def test_single_key_with_dropout_gradients_cancel():
	"""One key: P = 1, so dS = P (dP - delta) cancels exactly and dQ = dK = 0 - up to what the rounding of the
	stored O (from which delta is formed, as in the reference's backward) leaves, summed over the rows: with
	dropout and a few hundred rows that is above 1e-2, and the check measures it with the oracle instead of
	assuming a bound."""
	_run_case(3, 227, 1, 1, 1, 64, torch.bfloat16, causal=False, p=0.3, seed=1913384172, data_seed=193)
	_run_case(2, 300, 1, 4, 2, 128, torch.float16, causal=False, p=0.2, seed=11, data_seed=7)
	_run_case(1, 64, 1, 2, 2, 256, torch.bfloat16, causal=False, data_seed=3)


@pytest.mark.parametrize("r", [1, 2, 4, 8])
def test_gqa_group_sizes(r):
	_run_case(2, 192, 192, 8, 8 // r, 128, torch.bfloat16, causal=True)
	_run_case(1, 130, 130, 8, 8 // r, 64, torch.bfloat16, causal=False, data_seed=2)


@pytest.mark.parametrize(
	"bshape", [(1, 1), (2, 1), (1, 4), (2, 4), (2, 2)], ids=["b1h1", "bBh1", "b1hH", "bBhH", "bBhKV"]
)
@pytest.mark.parametrize("D", [64, 128])
def test_bias_broadcast(bshape, D):
	B, Sq, Sk, Hq, Hkv = 2, 160, 224, 4, 2
	_run_case(B, Sq, Sk, Hq, Hkv, D, torch.bfloat16, causal=False, bias_shape=(*bshape, Sq, Sk))
	_run_case(B, Sq, Sk, Hq, Hkv, D, torch.bfloat16, causal=True, bias_shape=(*bshape, Sq, Sk), data_seed=3)


@pytest.mark.parametrize(
	"shape",
	[
		# B, Sq, Sk, Hq, Hkv, D, dtype, causal, bias heads, p
		(1, 1, 4096, 8, 2, 128, torch.bfloat16, False, None, 0.0),
		(2, 17, 1500, 4, 4, 64, torch.float16, True, None, 0.0),
		(1, 64, 2048, 2, 1, 256, torch.bfloat16, True, 2, 0.1),
		(2, 5, 1024, 4, 2, 128, torch.bfloat16, False, 1, 0.0),
		(1, 33, 777, 2, 2, 64, torch.bfloat16, True, None, 0.25),
		# the rows of all q-heads of a kv-head share one workgroup when they fit one tile of 64 rows
		(2, 7, 900, 8, 2, 128, torch.bfloat16, True, 8, 0.2),
		(1, 16, 1024, 8, 2, 64, torch.float16, True, 2, 0.0),
		(2, 3, 640, 12, 4, 256, torch.bfloat16, False, None, 0.0),
	],
	ids=["decode_gqa", "short_causal_fp16", "d256_bias_dropout", "bias_lds", "ragged_dropout", "packed_bias_dropout",
	     "packed_kvhead_bias", "packed_d256"],
)
def test_short_query_split_over_keys(shape):
	"""Sq <= 64 over many keys: the forward runs split over key ranges (partial results merged by
	a second kernel) when the caller provides scratch, as the host layer does.  `Sq == 1` is the
	decoding case of flash_attention.py:239-242."""
	import ctypes

	from jax_flash_attn2 import _lib

	B, Sq, Sk, Hq, Hkv, D, dtype, causal, bh, p = shape
	pr = _lib.new_params()
	pr.B, pr.Sq, pr.Sk, pr.Hq, pr.Hkv, pr.D = B, Sq, Sk, Hq, Hkv, D
	assert _lib.load().fa2_fwd_scratch_bytes(ctypes.byref(pr)) > 0, "this shape is meant to take the split path"
	_run_case(B, Sq, Sk, Hq, Hkv, D, dtype, causal=causal, bias_shape=None if bh is None else (B, bh, Sq, Sk), p=p, seed=3)


def _random_case(rng):
	"""One configuration drawn from everything the operator accepts (sizes the fp64 oracle handles in well under a second)."""
	r = int(rng.choice([1, 1, 2, 4]))
	Hkv = int(rng.choice([1, 2, 3]))
	Hq = Hkv * r
	B = int(rng.choice([1, 2, 3]))
	D = int(rng.choice([64, 64, 128, 128, 256, 40, 96]))
	kind = rng.choice(["square", "square", "cross", "short_query", "one_tile"])
	if kind == "square":
		Sq = Sk = int(rng.integers(1, 400))
	elif kind == "cross":
		Sq, Sk = int(rng.integers(1, 300)), int(rng.integers(1, 600))
	elif kind == "short_query":
		Sq, Sk = int(rng.integers(1, 65)), int(rng.integers(512, 1400))
	else:
		Sq, Sk = int(rng.choice([64, 128, 256])), int(rng.choice([128, 256, 384]))
	dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
	causal = bool(rng.random() < 0.5)
	p = float(rng.choice([0.0, 0.0, 0.1, 0.3]))
	bias_shape = bias_dtype = seqlens = None
	extra = rng.choice(["none", "none", "bias", "bias", "seqlens"])
	if extra == "bias":
		bb = int(rng.choice([1, B]))
		bh = int(rng.choice([1, Hq, Hkv]))
		bias_shape = (bb, bh, Sq, Sk)
		bias_dtype = torch.float32 if rng.random() < 0.25 else None
	elif extra == "seqlens" and Sq == Sk:
		seqlens = [int(rng.integers(0, Sk + 1)) for _ in range(B)]
	return dict(B=B, Sq=Sq, Sk=Sk, Hq=Hq, Hkv=Hkv, D=D, dtype=dtype, causal=causal, bias_shape=bias_shape, p=p,
	            seed=int(rng.integers(0, 2**31)), seqlens=seqlens, bias_dtype=bias_dtype, data_seed=int(rng.integers(0, 1000)))


@pytest.mark.parametrize("chunk", range(6))
def test_random_configurations(chunk):
	"""Seeded sweep over shapes, head groupings, head dims, dtypes, causal, bias kinds, lengths and dropout."""
	rng = np.random.default_rng(1000 + chunk)
	for _ in range(8):
		_run_case(**_random_case(rng))


def _run_extra_case(rng):
	"""One configuration drawn from the operands that `_random_case` leaves out: key lengths, sliding window,
	soft-capping (with and without a bias) and the bias gradient, in any combination with causal, dropout, GQA."""
	r = int(rng.choice([1, 2, 4]))
	Hkv = int(rng.choice([1, 2]))
	Hq = Hkv * r
	B = int(rng.choice([1, 2, 3]))
	D = int(rng.choice([64, 128, 256]))
	dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
	Sq = int(rng.integers(1, 330))
	Sk = Sq if rng.random() < 0.5 else int(rng.integers(1, 700))
	causal = bool(rng.random() < 0.4)
	p = float(rng.choice([0.0, 0.0, 0.15]))
	window = None
	if rng.random() < 0.5:
		window = (int(rng.choice([-1, 0, 7, 64, 150, 400])), int(rng.choice([-1, 0, 3, 64, 200])))
	softcap = float(rng.choice([0.0, 0.0, 2.0, 20.0]))
	with_bias = (softcap > 0 and rng.random() < 0.5) or rng.random() < 0.3
	bias_shape = (int(rng.choice([1, B])), int(rng.choice([1, Hq])), Sq, Sk) if with_bias else None
	kv_lens = [int(rng.integers(0, Sk + 1)) for _ in range(B)] if rng.random() < 0.4 else None
	need_dbias = bias_shape is not None and rng.random() < 0.5
	seed = int(rng.integers(0, 2**31))
	q, k, v, do, bias = make_inputs(B, Sq, Sk, Hq, Hkv, D, dtype, int(rng.integers(0, 1000)), bias_shape)
	kw = dict(causal=causal, p_drop=p, seed=seed, kv_lens=kv_lens, window=window, softcap=softcap)
	what = (f"B{B} Sq{Sq} Sk{Sk} Hq{Hq} Hkv{Hkv} D{D} {dtype} causal={causal} p={p} window={window} softcap={softcap} "
	        f"bias={bias_shape} kv_lens={kv_lens} dbias={need_dbias}")
	o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), return_dbias=need_dbias, **kw)
	kl = None if kv_lens is None else torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
	o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), None, None, p, causal, seed, kl, window, softcap)
	g = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), None, None, p, causal, seed, kl, window, softcap, need_dbias)
	torch.cuda.synchronize()
	check_forward(o, lse, o_ref, lse_ref, dtype, what)
	stored = None
	if min(np.abs(x).max() for x in g_ref[:3]) <= 1e-10:
		o_st = torch.from_numpy(np.nan_to_num(o_ref)).to(dtype).to(torch.float64).numpy()
		stored = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), o_stored=o_st, **kw)
	check_grads(g[:3], g_ref[:3], what, stored)
	if need_dbias and np.abs(g_ref[3]).max() > 1e-10:
		e = O.rel_l2(g[3].float().cpu().numpy(), g_ref[3])
		assert e <= 1e-2, f"{what}: dbias rel-L2 {e:.3e}"


@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (128, torch.bfloat16), (128, torch.float16), (64, torch.float16)])
def test_grids_that_fill_the_chip(D, dtype):
	"""The forward and dQ kernels tile the rows in 128 when that still gives at most one workgroup per CU, which is what
	the small shapes of the other tests get; these shapes (B x Hq x ceil(Sq / 128) > 256) take the 256-row workgroups
	with every kind of operand: causal, dropout, bias through LDS and loaded directly (fp32), key lengths, lengths,
	sliding window, soft-capping with the bias gradient.  Causal grids of 257 to 512 such units run two 128-row
	workgroups per CU with the second half of the launch order reversed (B4 Hq16, B3 Hq32, B3 Hq24 below: groups placed
	by XCD and in plain order), larger ones 256 rows (B4 Hq32)."""
	B, Hq, Hkv, S = 4, 16, 4, 520
	assert 256 < B * Hq * ((S + 127) // 128) <= 512
	assert 2 * B * Hq * ((S + 127) // 128) > 512
	_run_case(B, S, S, 2 * Hq, 2 * Hkv, D, dtype, causal=True, data_seed=5)
	_run_case(B, S, S, 2 * Hq, 2 * Hkv, D, dtype, causal=True, p=0.2, seed=3, data_seed=6)
	_run_case(3, S, S, 2 * Hq, Hkv, D, dtype, causal=True, seqlens=[520, 1, 300], data_seed=7)
	_run_case(3, 700, 700, 8, 1, D, dtype, causal=True, data_seed=8)     # 144 units: at most one workgroup per CU, not folded
	_run_case(3, 700, 700, 24, 3, D, dtype, causal=True, data_seed=9)  # 432 units, groups not a multiple of 8: folded over the plain order
	_run_case(B, S, S, Hq, Hkv, D, dtype, causal=True)
	_run_case(B, S, S, Hq, Hkv, D, dtype, causal=True, p=0.2, seed=3, data_seed=1)
	_run_case(B, S, 456, Hq, Hkv, D, dtype, causal=False, bias_shape=(B, 1, S, 456), data_seed=2)
	_run_case(B, S, 457, Hq, Hkv, D, dtype, causal=False, bias_shape=(1, Hq, S, 457), bias_dtype=torch.float32, p=0.1, seed=4, data_seed=3)
	_run_case(B, S, S, Hq, Hkv, D, dtype, causal=True, seqlens=[520, 1, 300, 77], data_seed=4)
	rng = np.random.default_rng(7)
	for window, softcap, with_bias, kv_lens, need_dbias in (((150, 0), 0.0, False, None, False), ((-1, 64), 0.0, False, [520, 0, 333, 64], False),
	                                                        (None, 5.0, True, None, True), ((64, 64), 20.0, False, [100, 520, 519, 3], False)):
		bias_shape = (B, Hq, S, S) if with_bias else None
		q, k, v, do, bias = make_inputs(B, S, S, Hq, Hkv, D, dtype, int(rng.integers(0, 1000)), bias_shape)
		kw = dict(causal=False, p_drop=0.0, seed=0, kv_lens=kv_lens, window=window, softcap=softcap)
		what = f"D{D} {dtype} window={window} softcap={softcap} bias={bias_shape} kv_lens={kv_lens} dbias={need_dbias}"
		o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
		g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), return_dbias=need_dbias, **kw)
		kl = None if kv_lens is None else torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
		o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), None, None, 0.0, False, 0, kl, window, softcap)
		g = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), None, None, 0.0, False, 0, kl, window, softcap, need_dbias)
		check_forward(o, lse, o_ref, lse_ref, dtype, what)
		check_grads(g[:3], g_ref[:3], what)
		if need_dbias:
			assert O.rel_l2(g[3].float().cpu().numpy(), g_ref[3]) <= 1e-2, f"{what}: dbias"


@pytest.mark.parametrize("chunk", range(5))
def test_random_configurations_of_the_further_operands(chunk):
	"""Seeded sweep over key lengths, sliding windows, soft-capping and the bias gradient, combined at random."""
	rng = np.random.default_rng(4000 + chunk)
	for _ in range(8):
		_run_extra_case(rng)


@pytest.mark.parametrize("D", [32, 80, 96, 160, 192])
def test_other_head_dims(D):
	"""Head dims between the built ones are zero-padded by the host layer (the reference pads
	to the next power of two, _forward_triton.py:525-526); scale stays 1/sqrt(D)."""
	_run_case(2, 150, 150, 4, 2, D, torch.bfloat16, causal=True)
	_run_case(1, 96, 130, 2, 2, D, torch.float16, causal=False, bias_shape=(1, 2, 96, 130), data_seed=4)


@pytest.mark.parametrize("bshape", [(1, 1), (2, 1), (2, 4), (2, 2)], ids=["b1h1", "bBh1", "bBhH", "bBhKV"])
@pytest.mark.parametrize("D", [64, 128])
def test_bias_whole_key_tiles(bshape, D):
	"""Sk a multiple of 128 with a bias in the element type of q: the kernels copy bias tiles to
	LDS instead of loading single values (ragged query rows, causal and not, dropout on top)."""
	B, Sq, Sk, Hq, Hkv = 2, 200, 256, 4, 2
	_run_case(B, Sq, Sk, Hq, Hkv, D, torch.bfloat16, causal=False, bias_shape=(*bshape, Sq, Sk))
	_run_case(B, Sq, Sk, Hq, Hkv, D, torch.float16, causal=True, bias_shape=(*bshape, Sq, Sk), data_seed=5)
	_run_case(B, 256, 256, Hq, Hkv, D, torch.bfloat16, causal=True, bias_shape=(*bshape, 256, 256), p=0.2, seed=11, data_seed=6)


def test_bias_dtypes_and_unaligned_rows():
	# fp32 bias with a 16-bit q; odd Sk makes bias rows unaligned for vector loads
	_run_case(1, 70, 75, 2, 2, 64, torch.float16, bias_shape=(1, 2, 70, 75), bias_dtype=torch.float32)
	_run_case(1, 70, 75, 2, 2, 128, torch.bfloat16, bias_shape=(1, 1, 70, 75), bias_dtype=torch.float16, causal=True)
	_run_case(1, 96, 96, 2, 2, 256, torch.bfloat16, bias_shape=(1, 2, 96, 96))


def test_rows_masked_entirely_by_finfo_min_bias_stay_finite():
	"""A query row whose keys are all masked through the finfo.min bias (a padded query under the README mask
	recipe) gives the plain average of V - every score is the same huge negative number - and finite gradients;
	the valid rows are unaffected."""
	dtype = torch.bfloat16
	B, S, H, D = 2, 192, 2, 64
	q, k, v, do, _ = make_inputs(B, S, S, H, H, D, dtype, 17)
	fill = float(torch.finfo(dtype).min)
	bias = torch.zeros(B, 1, S, S)
	bias[:, :, 150:, :] = fill          # rows 150.. see nothing
	bias[:, :, :, 170:] = fill          # keys 170.. are padding
	bias = bias.to(dtype)
	o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias))
	g = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias))
	torch.cuda.synchronize()
	assert torch.isfinite(o).all() and all(torch.isfinite(x).all() for x in g)
	want = v.float().mean(dim=1, keepdim=True).expand(B, S - 150, H, D)
	assert float((o[:, 150:].float().cpu() - want).abs().max()) <= TOL_O[dtype]
	o_ref, lse_ref = O.attention_fwd(f64(q[:, :150]), f64(k), f64(v), f64(bias[:, :, :150]))
	assert float(np.abs(o[:, :150].float().cpu().numpy() - o_ref).max()) <= TOL_O[dtype]


def test_boolean_4d_mask_through_the_facade():
	"""A 4-D boolean mask acts as the finfo.min bias of README.md:188 (the kernels read the mask itself); also for Sq != Sk, where
	the facade drops the reference's 2-D mask (flash_attention.py:239-242)."""
	from jax_flash_attn2 import AttentionConfig, FlashAttention, Platform

	attn = FlashAttention(AttentionConfig(platform=Platform.HIP))
	for (Sq, Sk) in ((96, 96), (40, 200)):
		q, k, v, do, _ = make_inputs(2, Sq, Sk, 4, 2, 64, torch.bfloat16, 12)
		g = torch.Generator().manual_seed(5)
		mask = torch.rand(2, 1, Sq, Sk, generator=g) < 0.7
		mask[..., 0] = True  # every row keeps a key
		bias = torch.where(mask, 0.0, float(torch.finfo(torch.bfloat16).min)).to(torch.bfloat16)
		o_ref, _ = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias))
		out = attn(_dev(q), _dev(k), _dev(v), attention_mask=_dev(mask))
		err = float(np.abs(out.float().cpu().numpy() - o_ref).max())
		assert err <= TOL_O[torch.bfloat16], f"4-D mask Sq{Sq} Sk{Sk}: O max-abs {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mshape", [(2, 1), (1, 1), (2, 4), (1, 4)], ids=["bBh1", "b1h1", "bBhH", "b1hH"])
def test_boolean_mask_operand_equals_the_finfo_min_bias(dtype, mshape):
	"""A boolean mask handed over as one byte per position (fa2_params.bias_dtype = FA2_MASK_U8) against the oracle
	given the bias where(mask, 0, finfo(dtype).min) of README.md:188 - forward and backward, broadcast over batch
	and heads, ragged key counts, causal or not, including rows whose every key is masked (which that bias turns
	into a plain average over all keys for bf16, and into the unmasked softmax for fp16, whose finfo.min does not
	absorb the score)."""
	B, Hq, Hkv = 2, 4, 2
	for (Sq, Sk, D, causal) in ((160, 160, 128, False), (96, 203, 64, False), (130, 130, 64, True), (64, 96, 256, False)):
		q, k, v, do, _ = make_inputs(B, Sq, Sk, Hq, Hkv, D, dtype, 31)
		g = torch.Generator().manual_seed(9)
		mask = torch.rand(*mshape, Sq, Sk, generator=g) < 0.6
		if causal:
			mask[..., 0] = True    # (or the first rows, which see few keys, would often have none left)
		mask[..., 5, :] = False    # a row without any allowed key
		mask[..., 0, 1:] = False   # rows with a single key
		mask[..., 0, 0] = True
		# (bf16: the logsumexp of a fully masked row is finfo.min + log(sum), which fp32 rounds to finfo.min - the
		# backward of such a row is then off by the factor `sum`, with a finfo.min bias just the same; the row gets
		# no incoming gradient here, as rows that attend to nothing do not in practice)
		do[:, 5] = 0
		bias = torch.where(mask, 0.0, float(torch.finfo(dtype).min)).to(dtype)
		kw = dict(causal=causal)
		o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
		g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), **kw)
		o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(mask), None, None, 0.0, causal, 0)
		gr = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(mask), None, None, 0.0, causal, 0)
		what = f"mask {mshape} Sq{Sq} Sk{Sk} D{D} {dtype} causal={causal}"
		# lse of a fully masked row sits near finfo.min: compare it relatively there
		fin = lse_ref > -1e4
		check_forward(o, torch.where(_dev(torch.from_numpy(fin)), lse, torch.zeros_like(lse)), o_ref, np.where(fin, lse_ref, 0.0), dtype, what)
		lg = lse.cpu().numpy()
		assert np.allclose(lg[~fin], lse_ref[~fin], rtol=1e-3), what
		check_grads(gr, g_ref, what)
		# the same numbers as the bias the mask stands for
		o_b, lse_b = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), None, None, 0.0, causal, 0)
		assert float((o.float() - o_b.float()).abs().max()) <= 2.0 ** -7


@pytest.mark.parametrize("causal", [False, True])
def test_key_lengths_with_bias_and_cross_lengths(causal):
	"""fa2_params.kv_lens: per-batch key padding that, unlike the reference's 2-D mask, goes together with a bias and
	with Sq != Sk.  Checked against explicit masking in the oracle; keys beyond the length get exactly zero gradient,
	a length of zero leaves rows without keys (O = 0, lse = -inf)."""
	for (B, Sq, Sk, Hq, Hkv, D, lens, bshape) in (
		(3, 160, 160, 4, 2, 128, [160, 77, 1], (3, 1)),
		(2, 100, 300, 4, 4, 64, [300, 130], None),
		(4, 64, 200, 2, 1, 64, [0, 200, 64, 199], (1, 2)),
		(2, 130, 130, 2, 2, 256, [129, 40], None),
	):
		bias_shape = None if bshape is None else (*bshape, Sq, Sk)
		q, k, v, do, bias = make_inputs(B, Sq, Sk, Hq, Hkv, D, torch.bfloat16, 41, bias_shape)
		kw = dict(causal=causal, kv_lens=lens)
		o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
		g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), **kw)
		kl = torch.tensor(lens, dtype=torch.int32, device=DEV)
		o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), None, None, 0.0, causal, 0, kl)
		gr = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), None, None, 0.0, causal, 0, kl)
		what = f"kv_lens {lens} Sq{Sq} Sk{Sk} D{D} causal={causal} bias={bshape}"
		check_forward(o, lse, o_ref, lse_ref, torch.bfloat16, what)
		check_grads(gr, g_ref, what)
		for b, n in enumerate(lens):
			assert gr[1][b, n:].abs().max().item() == 0 and gr[2][b, n:].abs().max().item() == 0 if n < Sk else True
	# through the differentiation rule
	q, k, v, do, bias = make_inputs(2, 96, 96, 2, 2, 64, torch.bfloat16, 42, (2, 1, 96, 96))
	kl = torch.tensor([50, 96], dtype=torch.int32, device=DEV)
	qq = _dev(q).requires_grad_()
	out = op.flash_attention(qq, _dev(k), _dev(v), bias=_dev(bias), causal=causal, kv_lens=kl)
	out.backward(_dev(do))
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), causal=causal, kv_lens=[50, 96])
	assert O.rel_l2(qq.grad.float().cpu().numpy(), g_ref[0]) <= 1e-2


@pytest.mark.parametrize("window", [(64, 0), (17, 5), (0, 0), (-1, 40), (200, -1), (130, 130), (1000, 1000)])
def test_sliding_window(window):
	"""The sliding window of the reference's naive attention (refrence_call.py:32,55-75), fused: forward and
	backward against the oracle, self and cross lengths, with and without the causal flag (which caps the
	right bound at 0), GQA, every head dim, with bias, dropout and key lengths; rows that the window leaves
	without a key give zeros."""
	cases = (
		# B, Sq, Sk, Hq, Hkv, D, dtype, causal, bias heads, p
		(2, 320, 320, 4, 2, 128, torch.bfloat16, False, None, 0.0),
		(1, 200, 333, 4, 4, 64, torch.float16, False, None, 0.0),
		(1, 333, 200, 2, 1, 64, torch.bfloat16, False, None, 0.0),
		(2, 260, 260, 4, 2, 128, torch.bfloat16, True, None, 0.0),
		(1, 192, 192, 2, 2, 256, torch.bfloat16, False, None, 0.0),
		(2, 160, 224, 4, 2, 64, torch.bfloat16, False, (2, 1), 0.0),
		(1, 192, 192, 4, 2, 128, torch.bfloat16, False, None, 0.2),
		(1, 320, 448, 2, 1, 256, torch.bfloat16, False, None, 0.1),
	)
	for (B, Sq, Sk, Hq, Hkv, D, dtype, causal, bh, p) in cases:
		bias_shape = None if bh is None else (*bh, Sq, Sk)
		q, k, v, do, bias = make_inputs(B, Sq, Sk, Hq, Hkv, D, dtype, 51, bias_shape)
		kw = dict(causal=causal, window=window, p_drop=p, seed=9)
		o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
		g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), **kw)
		o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), None, None, p, causal, 9, None, window)
		gr = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), None, None, p, causal, 9, None, window)
		what = f"window {window} Sq{Sq} Sk{Sk} D{D} {dtype} causal={causal} bias={bh} p={p}"
		check_forward(o, lse, o_ref, lse_ref, dtype, what)
		check_grads(gr, g_ref, what)
	# with key lengths, and through the differentiation rule
	q, k, v, do, _ = make_inputs(2, 150, 150, 2, 2, 64, torch.bfloat16, 52)
	kl = torch.tensor([150, 90], dtype=torch.int32, device=DEV)
	qq = _dev(q).requires_grad_()
	out = op.flash_attention(qq, _dev(k), _dev(v), kv_lens=kl, window_size=window)
	out.backward(_dev(do))
	o_ref, _ = O.attention_fwd(f64(q), f64(k), f64(v), kv_lens=[150, 90], window=window)
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), kv_lens=[150, 90], window=window)
	assert np.abs(out.detach().float().cpu().numpy() - o_ref).max() <= TOL_O[torch.bfloat16]
	check_grads((qq.grad,), (g_ref[0],), f"window {window} with key lengths")
	# cross lengths with key lengths: the window (and the causal flag) stay aligned to the FULL key count, row i <-> key
	# i + Sk - Sq, the length only removes keys (the oracle's test_key_lengths_keep_the_window_aligned_... spells it out)
	for causal in (False, True):
		q, k, v, do, _ = make_inputs(2, 130, 300, 4, 2, 128, torch.bfloat16, 53)
		kw = dict(causal=causal, kv_lens=[300, 201], window=window)
		o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), **kw)
		g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), **kw)
		kl = torch.tensor([300, 201], dtype=torch.int32, device=DEV)
		o, lse = op.fwd(_dev(q), _dev(k), _dev(v), None, None, None, 0.0, causal, 0, kl, window)
		gr = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), None, None, None, 0.0, causal, 0, kl, window)
		check_forward(o, lse, o_ref, lse_ref, torch.bfloat16, f"window {window} Sq130 Sk300 kv_lens causal={causal}")
		check_grads(gr, g_ref, f"window {window} Sq130 Sk300 kv_lens causal={causal}")


@pytest.mark.parametrize("cap", [1.0, 5.0, 30.0])
def test_softcap(cap):
	"""tanh soft-capping of the scores (refrence_call.py:33,48-51), fused: forward and backward against the oracle with
	scores that reach several times the cap (so that tanh saturates) and scores well inside it; with and without
	bias (all element types, the mask bytes too), causal, GQA, every head dim, dropout, key lengths, a window and a
	short query (which otherwise takes the split forward)."""
	cases = (
		# B, Sq, Sk, Hq, Hkv, D, dtype, causal, bias shape, bias dtype, p, qk_scale
		(2, 320, 320, 4, 2, 128, torch.bfloat16, True, None, None, 0.0, 2.1),
		(1, 200, 333, 4, 4, 64, torch.float16, False, None, None, 0.0, 2.1),
		(1, 160, 160, 2, 1, 256, torch.bfloat16, True, None, None, 0.0, 1.0),
		(2, 160, 224, 4, 2, 64, torch.bfloat16, False, (2, 1, 160, 224), None, 0.0, 2.1),
		(2, 160, 224, 4, 2, 128, torch.bfloat16, True, (1, 4, 160, 224), torch.float32, 0.0, 1.0),
		(1, 192, 192, 4, 2, 128, torch.bfloat16, True, None, None, 0.2, 2.1),
		(1, 130, 130, 2, 2, 256, torch.float16, False, (1, 2, 130, 130), None, 0.1, 1.0),
		(2, 16, 1024, 4, 2, 128, torch.bfloat16, False, None, None, 0.0, 2.1),
	)
	for (B, Sq, Sk, Hq, Hkv, D, dtype, causal, bshape, bdt, p, qs) in cases:
		q, k, v, do, bias = make_inputs(B, Sq, Sk, Hq, Hkv, D, dtype, 61, bshape, bias_dtype=bdt, qk_scale=qs)
		kw = dict(causal=causal, p_drop=p, seed=4, softcap=cap)
		o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
		g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), **kw)
		o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), None, None, p, causal, 4, softcap=cap)
		gr = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), None, None, p, causal, 4, softcap=cap)
		what = f"softcap {cap} B{B} Sq{Sq} Sk{Sk} Hq{Hq} Hkv{Hkv} D{D} {dtype} causal={causal} bias={bshape} {bdt} p={p}"
		check_forward(o, lse, o_ref, lse_ref, dtype, what)
		check_grads(gr, g_ref, what)
	# with a boolean mask operand, key lengths and a window, through the differentiation rule
	q, k, v, do, _ = make_inputs(2, 150, 150, 2, 2, 64, torch.bfloat16, 62, qk_scale=2.1)
	kl = torch.tensor([150, 90], dtype=torch.int32, device=DEV)
	qq, kk, vv = (_dev(x).requires_grad_() for x in (q, k, v))
	out = op.flash_attention(qq, kk, vv, kv_lens=kl, window_size=(40, 3), softcap=cap)
	out.backward(_dev(do))
	kw = dict(kv_lens=[150, 90], window=(40, 3), softcap=cap)
	o_ref, _ = O.attention_fwd(f64(q), f64(k), f64(v), **kw)
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), **kw)
	assert np.abs(out.detach().float().cpu().numpy() - o_ref).max() <= TOL_O[torch.bfloat16]
	check_grads((qq.grad, kk.grad, vv.grad), g_ref, f"softcap {cap} with key lengths and a window")
	# cap off (0) is the plain operator
	o0, lse0 = op.fwd(_dev(q), _dev(k), _dev(v), softcap=0.0)
	o1, lse1 = op.fwd(_dev(q), _dev(k), _dev(v))
	assert torch.equal(o0, o1) and torch.equal(lse0, lse1)


def test_mask_as_finfo_min_bias():
	"""Boolean mask -> where(mask, 0, finfo.min) bias (the README recipe) must equal key-length masking."""
	B, S, H, D = 2, 192, 4, 64
	dtype = torch.bfloat16
	q, k, v, do, _ = make_inputs(B, S, S, H, H, D, dtype, 5)
	lens = [100, 192]
	valid = torch.arange(S)[None, :] < torch.tensor(lens)[:, None]
	i = torch.arange(S)
	base = 1.0 / (1.0 + (i[:, None] - i[None, :]).abs().float())
	bias = torch.where(valid[:, None, None, :], base[None, None], torch.tensor(torch.finfo(dtype).min)).to(dtype)
	o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias))
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias))
	o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias))
	g = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias))
	check_forward(o, lse, o_ref, lse_ref, dtype, "finfo.min bias")
	check_grads(g, g_ref, "finfo.min bias")
	# masked keys get exactly zero gradient
	assert g[1][0, 100:].abs().max().item() == 0 and g[2][0, 100:].abs().max().item() == 0


@pytest.mark.parametrize(
	"bshape", [(1, 1), (2, 1), (1, 4), (2, 4), (2, 2)], ids=["b1h1", "bBh1", "b1hH", "bBhH", "bBhKV"]
)
@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (128, torch.float16), (256, torch.bfloat16)])
def test_bias_gradient(bshape, D, dtype):
	"""fa2_params.dbias in the shape of the bias (the dQ kernel adds the per-head gradient of the additive term into it,
	with atomic adds on the axes the bias is broadcast on) against the oracle; ragged tiles, causal, dropout, key lengths;
	dq / dk / dv unchanged."""
	B, Sq, Sk, Hq, Hkv = 2, 160, 203, 4, 2
	for causal, p, kv_lens in ((False, 0.0, None), (True, 0.2, None), (False, 0.0, [150, 64])):
		q, k, v, do, bias = make_inputs(B, Sq, Sk, Hq, Hkv, D, dtype, 5, (*bshape, Sq, Sk))
		kw = dict(causal=causal, p_drop=p, seed=9, kv_lens=kv_lens)
		ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), return_dbias=True, **kw)
		kl = None if kv_lens is None else torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
		o, lse = op.fwd(_dev(q), _dev(k), _dev(v), _dev(bias), None, None, p, causal, 9, kv_lens=kl)
		g = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), None, None, p, causal, 9, kv_lens=kl, need_dbias=True)
		g0 = op.bwd(_dev(q), _dev(k), _dev(v), o, lse, _dev(do), _dev(bias), None, None, p, causal, 9, kv_lens=kl)
		torch.cuda.synchronize()
		what = f"bias {bshape} D{D} causal={causal} p={p} kv_lens={kv_lens}"
		check_grads(g[:3], ref[:3], what)
		for a, b in zip(g[:3], g0):
			assert torch.equal(a, b), what
		db = g[3].cpu().numpy()
		assert db.shape == ref[3].shape and np.isfinite(db).all(), what
		e = O.rel_l2(db, ref[3])
		assert e <= 1e-2, f"{what}: dbias rel-L2 {e:.3e}"


def test_bias_gradient_through_autograd_and_softcap():
	"""A bias that requires a gradient gets one from the operator's differentiation rule when the caller asks for it with
	`bias_grad=True` (the reference returns None for it, _flash_attention.py:88, and so does this operator by default); with
	soft-capping the bias gradient does not carry the 1 - tanh^2 factor."""
	B, Sq, Sk, Hq, Hkv, D = 1, 96, 130, 4, 4, 64
	q, k, v, do, bias = make_inputs(B, Sq, Sk, Hq, Hkv, D, torch.bfloat16, 2, (1, 1, Sq, Sk), bias_dtype=torch.float32)
	ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), causal=True, softcap=2.0, return_dbias=True)
	qd, kd, vd, bd = (_dev(t).requires_grad_(True) for t in (q, k, v, bias))
	out = op.flash_attention(qd, kd, vd, bias=bd, causal=True, softcap=2.0, bias_grad=True)
	out.backward(_dev(do))
	torch.cuda.synchronize()
	check_grads((qd.grad, kd.grad, vd.grad), ref[:3], "autograd with bias gradient")
	assert bd.grad.shape == bias.shape and bd.grad.dtype == torch.float32
	assert O.rel_l2(bd.grad.cpu().numpy(), ref[3]) <= 1e-2
	# no gradient asked for the bias: none computed
	qd2 = _dev(q).requires_grad_(True)
	b2 = _dev(bias)
	op.flash_attention(qd2, _dev(k), _dev(v), bias=b2, causal=True, softcap=2.0).backward(_dev(do))
	assert b2.grad is None and torch.equal(qd2.grad, qd.grad)
	# ... nor for a bias that requires one but was not asked for (as in the reference)
	qd3, b3 = _dev(q).requires_grad_(True), _dev(bias).requires_grad_(True)
	op.flash_attention(qd3, _dev(k), _dev(v), bias=b3, causal=True, softcap=2.0).backward(_dev(do))
	assert b3.grad is None and torch.equal(qd3.grad, qd.grad)


@pytest.mark.parametrize("causal", [False, True])
def test_seqlens(causal):
	_run_case(4, 256, 256, 4, 2, 128, torch.bfloat16, causal=causal, seqlens=[256, 100, 1, 0])
	_run_case(3, 200, 200, 2, 2, 64, torch.float16, causal=causal, seqlens=[17, 200, 129])


def test_2d_mask_is_applied_for_a_single_batch_row_too():
	"""Intended difference from the reference: its GPU path only honours a 2-D attention_mask when the batch has more
	than one row (`varlen_mode = attention_mask.shape[0] > 1`, _forward_triton.py:474-475, 498) and silently ignores
	it for B == 1.  Here the mask always applies: keys beyond the valid length are masked, padded query rows give 0."""
	B, S, H, D, n = 1, 96, 2, 64, 40
	q, k, v, do, _ = make_inputs(B, S, S, H, H, D, torch.bfloat16, 21)
	mask = torch.zeros(B, S, dtype=torch.int32)
	mask[:, :n] = 1
	qq, kk, vv = (_dev(t).requires_grad_() for t in (q, k, v))
	out = op.flash_attention(qq, kk, vv, attention_mask=_dev(mask), causal=True)
	out.backward(_dev(do))
	o_ref, _ = O.attention_fwd(f64(q), f64(k), f64(v), causal=True, seqlens=[n])
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), causal=True, seqlens=[n])
	got = out.detach().float().cpu().numpy()
	assert np.abs(got - o_ref).max() <= TOL_O[torch.bfloat16]
	assert np.abs(got[:, n:]).max() == 0.0 and np.abs(o_ref[:, n:]).max() == 0.0
	check_grads((qq.grad, kk.grad, vv.grad), g_ref, "B == 1 with a 2-D mask")
	# what the reference computes for this call (mask ignored) is something else
	o_unmasked, _ = O.attention_fwd(f64(q), f64(k), f64(v), causal=True)
	assert np.abs(o_unmasked[:, n:]).max() > 0.1


@pytest.mark.parametrize("D", [64, 128, 256])
def test_dropout(D):
	_run_case(2, 192, 192, 4, 2, D, torch.bfloat16, causal=True, p=0.1, seed=42)
	_run_case(1, 100, 150, 2, 2, D, torch.float16, causal=False, p=0.5, seed=(9 << 32) | 5, data_seed=4)


def test_custom_softmax_scale():
	_run_case(1, 128, 128, 2, 2, 128, torch.bfloat16, causal=True, scale=0.2)


@pytest.mark.parametrize(
	"name", sorted(f[:-4] for f in os.listdir(os.path.join(HERE, "golden")) if f.endswith(".npz"))
)
def test_golden_fixtures(name):
	z = np.load(os.path.join(HERE, "golden", name + ".npz"))
	dtype = torch.bfloat16  # fixture inputs are bf16-representable
	t = lambda a: torch.from_numpy(np.asarray(a)).to(dtype).to(DEV)
	causal, p, seed = bool(z["causal"]), float(z["p_drop"]), int(z["seed"])
	bias = t(z["bias"]) if "bias" in z else None
	sl = torch.from_numpy(z["seqlens"]).to(DEV) if "seqlens" in z else None
	o, lse = op.fwd(t(z["q"]), t(z["k"]), t(z["v"]), bias, sl, None, p, causal, seed)
	g = op.bwd(t(z["q"]), t(z["k"]), t(z["v"]), o, lse, t(z["dout"]), bias, sl, None, p, causal, seed)
	check_forward(o, lse, z["o"], z["lse"], dtype, name)
	check_grads(g, (z["dq"], z["dk"], z["dv"]), name)
	if p > 0:
		B, Sq, Hq, _ = z["q"].shape
		Sk = z["k"].shape[1]
		keep = op.dropout_mask(B, Hq, Sq, Sk, p, seed, DEV).cpu().numpy().astype(bool)
		want = np.unpackbits(z["keep_bits"])[: keep.size].astype(bool).reshape(keep.shape)
		assert np.array_equal(keep, want)


@pytest.mark.parametrize(
	"B,H,Sq,Sk,p,seed",
	[(2, 3, 37, 50, 0.25, 12345), (1, 2, 128, 129, 0.1, 42), (1, 1, 5, 3, 0.9, (1 << 63) | 7), (3, 1, 64, 256, 0.5, 0),
	 (1, 2, 16, 16, 0.0, 99)],
)
def test_dropout_mask_is_bit_exact(B, H, Sq, Sk, p, seed):
	keep = op.dropout_mask(B, H, Sq, Sk, p, seed, DEV).cpu().numpy().astype(bool)
	assert np.array_equal(keep, O.dropout_keep_mask(seed, p, B, H, Sq, Sk))


def test_seed_in_device_memory_gives_the_masks_of_the_host_seed():
	"""The dropout seed as a run-time operand: a 64-bit value in device memory that the kernels read
	(fa2_params.seed_dev) - as the reference hands dropout_seed to its custom call as an operand
	(_forward_triton.py:553).  Forward, backward and the exported mask are bit-identical to the host-seed path."""
	B, S, Hq, Hkv, D, p = 2, 200, 4, 2, 128, 0.2
	q, k, v, do, _ = make_inputs(B, S, S, Hq, Hkv, D, torch.bfloat16, 5)
	q, k, v, do = (_dev(t) for t in (q, k, v, do))
	for seed in (42, (1 << 63) | 12345, 0):
		signed = seed - (1 << 64) if seed >= (1 << 63) else seed
		seed_t = torch.tensor([signed], dtype=torch.int64, device=DEV)
		o0, lse0 = op.fwd(q, k, v, None, None, None, p, True, seed)
		o1, lse1 = op.fwd(q, k, v, None, None, None, p, True, seed_t)
		assert torch.equal(o0, o1) and torch.equal(lse0, lse1)
		g0 = op.bwd(q, k, v, o0, lse0, do, None, None, None, p, True, seed)
		g1 = op.bwd(q, k, v, o0, lse0, do, None, None, None, p, True, seed_t)
		for a, b in zip(g0, g1):
			assert torch.equal(a, b)
		m0 = op.dropout_mask(B, Hq, S, S, p, seed, DEV)
		m1 = op.dropout_mask(B, Hq, S, S, p, seed_t, DEV)
		assert torch.equal(m0, m1)
		assert np.array_equal(m1.cpu().numpy().astype(bool), O.dropout_keep_mask(seed, p, B, Hq, S, S))
	# the seed is read at run time: a new value in the same buffer changes the mask of the next call
	seed_t = torch.tensor([1], dtype=torch.int64, device=DEV)
	m1 = op.dropout_mask(1, 1, 64, 64, 0.5, seed_t, DEV)
	seed_t.fill_(2)
	m2 = op.dropout_mask(1, 1, 64, 64, 0.5, seed_t, DEV)
	assert np.array_equal(m2.cpu().numpy().astype(bool), O.dropout_keep_mask(2, 0.5, 1, 1, 64, 64)) and not torch.equal(m1, m2)
	# the differentiation rule passes a device seed through as well
	qq, kk, vv = (t.clone().requires_grad_() for t in (q, k, v))
	out = op.flash_attention(qq, kk, vv, dropout_prob=p, causal=True, dropout_seed=torch.tensor([42], dtype=torch.int64, device=DEV))
	out.backward(do)
	o0, lse0 = op.fwd(q, k, v, None, None, None, p, True, 42)
	g0 = op.bwd(q, k, v, o0, lse0, do, None, None, None, p, True, 42)
	assert torch.equal(out.detach(), o0) and torch.equal(qq.grad, g0[0]) and torch.equal(kk.grad, g0[1])


def test_kernels_apply_exactly_the_exported_mask():
	"""Read the mask back out of each kernel: with q = 0 the probabilities are uniform,
	and one-hot V / dO / K rows turn O, dV and dQ into scaled copies of the keep-mask."""
	B, H, S, D, p, seed = 2, 2, 64, 64, 0.3, 4242
	dtype = torch.float16
	eye = torch.eye(S, D, dtype=dtype, device=DEV)[None, :, None, :].expand(B, S, H, D).contiguous()
	zero = torch.zeros(B, S, H, D, dtype=dtype, device=DEV)
	ones = torch.ones(B, S, H, D, dtype=dtype, device=DEV)
	keep = O.dropout_keep_mask(seed, p, B, H, S, S)  # [B,H,i,j]
	inv = O.dropout_keep_scale(p)
	# forward: O[b,i,h,j] = keep[b,h,i,j] / (S (1-p))
	o, lse = op.fwd(zero, eye, eye, None, None, None, p, False, seed)
	got = (o.float().permute(0, 2, 1, 3).cpu().numpy() * S / inv) > 0.5
	assert np.array_equal(got, keep)
	# dK/dV kernel: dO one-hot -> dV[b,j,h,i] = keep[b,h,i,j] / (S (1-p))
	dq, dk, dv = op.bwd(zero, eye, eye, o, lse, eye, None, None, None, p, False, seed)
	got = (dv.float().permute(0, 2, 3, 1).cpu().numpy() * S / inv) > 0.5
	assert np.array_equal(got, keep)
	# dQ kernel: K, V one-hot, dO = 1 -> dQ[b,i,h,j] = scale/S (keep/(1-p) - delta_i)
	dq, dk, dv = op.bwd(zero, eye, eye, o, lse, ones, None, None, None, p, False, seed)
	delta = (o.float() * 1.0).sum(-1, keepdim=True)
	rec = dq.float() * S * (D ** 0.5) + delta
	got = (rec.permute(0, 2, 1, 3).cpu().numpy() / inv) > 0.5
	assert np.array_equal(got, keep)


def test_backward_is_deterministic_and_outputs_fully_written():
	q, k, v, do, _ = make_inputs(2, 300, 300, 8, 2, 128, torch.bfloat16, 7)
	q, k, v, do = (_dev(t) for t in (q, k, v, do))
	o, lse = op.fwd(q, k, v, causal=True)
	a = op.bwd(q, k, v, o, lse, do, causal=True)
	b = op.bwd(q, k, v, o, lse, do, causal=True)
	for x, y in zip(a, b):
		assert torch.equal(x, y)
	# poison-filled outputs: every element must be overwritten
	plan = op.Plan(q, k, v, dout=do, causal=True)
	for t in (plan.out, plan.dq, plan.dk, plan.dv):
		t.fill_(float("nan"))
	plan.lse.fill_(float("nan"))
	plan.forward()
	plan.backward()
	torch.cuda.synchronize()
	for t in (plan.out, plan.lse, plan.dq, plan.dk, plan.dv):
		assert torch.isfinite(t.float()).all()
	assert torch.equal(plan.dq, a[0]) and torch.equal(plan.dk, a[1]) and torch.equal(plan.dv, a[2])


@pytest.mark.parametrize("D,dtype,p_drop", [(128, torch.bfloat16, 0.0), (64, torch.float16, 0.1), (256, torch.bfloat16, 0.0)])
def test_backward_with_and_without_the_step_split(D, dtype, p_drop):
	"""On a small grid the dK/dV kernel splits the steps of a key tile (q-heads of the group x query tiles) over
	workgroups when the caller's scratch has room for the partial sums (fa2_bwd_split_scratch_bytes), and runs unsplit
	with the minimum scratch: both give the oracle's gradients, each bit-identical from call to call."""
	import ctypes
	from jax_flash_attn2 import _lib
	lib = _lib.load()
	B, S, Hq, Hkv = 2, 333, 8, 2
	q, k, v, do, _ = make_inputs(B, S, S, Hq, Hkv, D, dtype, 21)
	kw = dict(causal=True, p_drop=p_drop, seed=6)
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), None, **kw)
	plan = op.Plan(_dev(q), _dev(k), _dev(v), dout=_dev(do), causal=True, dropout_prob=p_drop, dropout_seed=6 if p_drop else None)
	P = ctypes.byref(plan.params)
	need_min, need_split = lib.fa2_bwd_scratch_bytes(P), lib.fa2_bwd_split_scratch_bytes(P)
	assert need_split > need_min and plan.params.scratch_bytes >= need_split
	plan.forward()
	results = {}
	for name, nbytes in (("split", plan.params.scratch_bytes), ("unsplit", need_min)):
		plan.params.scratch_bytes = nbytes
		runs = []
		for _ in range(2):
			for t in (plan.dq, plan.dk, plan.dv):
				t.fill_(float("nan"))
			plan.backward()
			torch.cuda.synchronize()
			runs.append([t.clone() for t in (plan.dq, plan.dk, plan.dv)])
		for x, y in zip(*runs):
			assert torch.equal(x, y), name
		check_grads(runs[0], g_ref, f"{name} D{D} {dtype} p={p_drop}")
		results[name] = runs[0]
	assert torch.equal(results["split"][0], results["unsplit"][0])  # dQ does not depend on the split


@pytest.mark.parametrize("B,Hq,Hkv,S,D,parts", [(1, 32, 8, 4096, 128, 2), (2, 16, 1, 4096, 64, 8), (3, 16, 4, 4096, 256, 2)])
def test_step_split_of_a_causal_grid_near_the_cu_count(B, Hq, Hkv, S, D, parts):
	"""Causal grids of fewer than 512 key-tile workgroups are split further than filling the chip needs (their key tiles
	differ in length).  At these sizes the oracle is out of reach: the split launch must reproduce the unsplit one, which
	sums the same fp32 products in another order - dQ bit for bit, dK / dV to rounding of the 16-bit results."""
	import ctypes
	from jax_flash_attn2 import _lib
	lib = _lib.load()
	dev = torch.device("cuda:0")
	g = torch.Generator(device=dev)
	g.manual_seed(5)
	rnd = lambda *shape: (torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * 0.5).to(torch.bfloat16)
	q, k, v, do = rnd(B, S, Hq, D), rnd(B, S, Hkv, D), rnd(B, S, Hkv, D), rnd(B, S, Hq, D)
	plan = op.Plan(q, k, v, dout=do, causal=True)
	P = ctypes.byref(plan.params)
	need_min, need_split = lib.fa2_bwd_scratch_bytes(P), lib.fa2_bwd_split_scratch_bytes(P)
	if parts:
		assert need_split == need_min + parts * B * Hkv * S * 2 * D * 4
	assert need_split > need_min and plan.params.scratch_bytes >= need_split
	plan.forward()
	results = {}
	for name, nbytes in (("split", plan.params.scratch_bytes), ("unsplit", need_min)):
		plan.params.scratch_bytes = nbytes
		for t in (plan.dq, plan.dk, plan.dv):
			t.fill_(float("nan"))
		plan.backward()
		torch.cuda.synchronize()
		results[name] = [t.clone() for t in (plan.dq, plan.dk, plan.dv)]
	assert torch.equal(results["split"][0], results["unsplit"][0])
	for x, y, what in zip(results["split"][1:], results["unsplit"][1:], ("dk", "dv")):
		assert torch.isfinite(x.float()).all(), what
		rel = float((x.float() - y.float()).norm() / y.float().norm())
		assert rel < 2e-3, (what, rel)  # (one rounding step of bf16 is 2^-9 = 2e-3 of a value; most values agree exactly)


@pytest.mark.parametrize("order", [(1, 2, 4), (1, 4, 2), (5, 2), (3, 4), (1, 6)])
def test_backward_by_stages_matches_the_oracle(order):
	"""fa2_bwd_stages: the stand-alone delta pre-pass (bit 0), the dK/dV kernel (bit 1) and the dQ kernel (bit 2)
	launched separately, in either order after the pre-pass, and the dQ kernel that forms delta itself (5) followed
	by dK/dV - the launches the benchmark times one by one.  Every combination must give the gradients of fa2_bwd."""
	for D, dtype, causal, pdrop in ((128, torch.bfloat16, True, 0.0), (64, torch.float16, False, 0.0), (256, torch.bfloat16, True, 0.1)):
		B, S, Hq, Hkv = 2, 260, 4, 2
		q, k, v, do, _ = make_inputs(B, S, S, Hq, Hkv, D, dtype, 11)
		g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), causal=causal, p_drop=pdrop, seed=3)
		plan = op.Plan(_dev(q), _dev(k), _dev(v), dout=_dev(do), causal=causal, dropout_prob=pdrop, dropout_seed=3)
		plan.forward()
		want = [t.clone() for t in plan.backward()]
		for t in (plan.dq, plan.dk, plan.dv):
			t.fill_(float("nan"))
		plan.scratch.fill_(0xFF)  # delta must come from this sequence of calls, not from the full backward above
		for stages in order:
			plan.backward(stages)
		torch.cuda.synchronize()
		check_grads((plan.dq, plan.dk, plan.dv), g_ref, f"stages {order} D{D}")
		# delta from the pre-pass and delta formed inside the dQ kernel may differ in the last bit of an fp32 sum
		for name, a, b in zip(("dq", "dk", "dv"), (plan.dq, plan.dk, plan.dv), want):
			assert O.rel_l2(a.float().cpu().numpy(), b.float().cpu().numpy().astype(np.float64)) <= 1e-3, name


def test_strided_inputs_from_a_fused_qkv_buffer():
	B, S, Hq, Hkv, D = 2, 160, 4, 2, 128
	dtype = torch.bfloat16
	g = torch.Generator().manual_seed(11)
	fused = (torch.randn(B, S, Hq + 2 * Hkv, D, generator=g) * 0.5).to(dtype)
	do = torch.randn(B, S, Hq, D, generator=g).to(dtype)
	q, k, v = fused[:, :, :Hq], fused[:, :, Hq:Hq + Hkv], fused[:, :, Hq + Hkv:]
	o_ref, lse_ref = O.attention_fwd(f64(q), f64(k), f64(v), causal=True)
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), causal=True)
	fd = fused.to(DEV)
	qd, kd, vd = fd[:, :, :Hq], fd[:, :, Hq:Hq + Hkv], fd[:, :, Hq + Hkv:]
	assert not qd.is_contiguous()
	o, lse = op.fwd(qd, kd, vd, causal=True)
	gr = op.bwd(qd, kd, vd, o, lse, _dev(do), causal=True)
	check_forward(o, lse, o_ref, lse_ref, dtype, "strided")
	check_grads(gr, g_ref, "strided")


def test_gqa_equals_mha_on_repeated_kv():
	q, k, v, do, _ = make_inputs(1, 256, 256, 8, 2, 128, torch.bfloat16, 8)
	q, k, v, do = (_dev(t) for t in (q, k, v, do))
	o1, l1 = op.fwd(q, k, v, causal=True)
	kr, vr = k.repeat_interleave(4, dim=2), v.repeat_interleave(4, dim=2)
	o2, l2 = op.fwd(q, kr, vr, causal=True)
	assert torch.equal(o1, o2) and torch.equal(l1, l2)
	g1 = op.bwd(q, k, v, o1, l1, do, causal=True)
	g2 = op.bwd(q, kr, vr, o2, l2, do, causal=True)
	assert torch.equal(g1[0], g2[0])
	for a, b in ((g1[1], g2[1]), (g1[2], g2[2])):
		ref = b.float().reshape(1, 256, 2, 4, 128).sum(3)
		assert O.rel_l2(a.float().cpu().numpy(), ref.cpu().numpy()) < 5e-3


def test_facade_forward_and_autograd():
	"""FlashAttention(AttentionConfig(...)).forward / __call__ with gradients through the operator."""
	from jax_flash_attn2 import AttentionConfig, Backend, FlashAttention, Platform

	attn = FlashAttention(AttentionConfig(platform=Platform.HIP, backend=Backend.GPU))
	q, k, v, do, bias = make_inputs(2, 128, 128, 4, 2, 64, torch.bfloat16, 9, bias_shape=(2, 2, 128, 128))
	qd, kd, vd = (_dev(t).requires_grad_() for t in (q, k, v))
	out = attn.forward(qd, kd, vd, bias=_dev(bias), causal=True, dropout_prob=0.1, dropout_seed=7)
	out.backward(_dev(do))
	kw = dict(causal=True, p_drop=0.1, seed=7)
	o_ref, _ = O.attention_fwd(f64(q), f64(k), f64(v), f64(bias), **kw)
	g_ref = O.attention_bwd(f64(q), f64(k), f64(v), f64(do), f64(bias), **kw)
	assert np.abs(out.detach().float().cpu().numpy() - o_ref).max() <= TOL_O[torch.bfloat16]
	check_grads((qd.grad, kd.grad, vd.grad), g_ref, "facade")
	# 2-D padding mask, Sq == Sk; with Sq != Sk the mask is dropped and a single row is never causal
	mask = (torch.arange(128)[None, :] < torch.tensor([128, 50])[:, None]).to(DEV)
	o2 = attn(qd.detach(), kd.detach(), vd.detach(), attention_mask=mask)
	o2_ref, _ = O.attention_fwd(f64(q), f64(k), f64(v), seqlens=[128, 50])
	assert np.abs(o2.float().cpu().numpy() - o2_ref).max() <= TOL_O[torch.bfloat16]
	o3 = attn(qd.detach()[:, :1], kd.detach(), vd.detach(), attention_mask=mask, causal=True)
	o3_ref, _ = O.attention_fwd(f64(q)[:, :1], f64(k), f64(v), causal=False)
	assert np.abs(o3.float().cpu().numpy() - o3_ref).max() <= TOL_O[torch.bfloat16]
	with pytest.warns(UserWarning):
		o4 = FlashAttention(AttentionConfig(platform=Platform.TRITON, backend=Backend.GPU))(qd.detach(), kd.detach(), vd.detach())
	assert torch.equal(o4, attn(qd.detach(), kd.detach(), vd.detach()))


def test_graph_capture_and_replay():
	"""The library only enqueues kernels on the caller's stream (no allocation, no synchronisation), so a forward +
	backward can be captured into a HIP graph; every replay must reproduce the eager results bit for bit."""
	q, k, v, do, _ = make_inputs(2, 300, 300, 4, 2, 128, torch.bfloat16, 21)
	plan = op.Plan(_dev(q), _dev(k), _dev(v), dout=_dev(do), causal=True, dropout_prob=0.1, dropout_seed=9)
	plan.forward()
	plan.backward()
	torch.cuda.synchronize()
	want = [t.clone() for t in (plan.out, plan.lse, plan.dq, plan.dk, plan.dv)]
	graph = torch.cuda.CUDAGraph()
	with torch.cuda.graph(graph):
		plan.forward()
		plan.backward()
	for _ in range(3):
		for t in (plan.out, plan.lse, plan.dq, plan.dk, plan.dv):
			t.zero_()
		torch.cuda.synchronize()
		graph.replay()
		torch.cuda.synchronize()
		for got, ref in zip((plan.out, plan.lse, plan.dq, plan.dk, plan.dv), want):
			assert torch.equal(got, ref)


def test_concurrent_streams_and_threads():
	"""No mutable global state: calls from several host threads on several streams give the results of running
	them one after the other."""
	import threading

	cases = []
	for n, (S, D, causal) in enumerate(((260, 64, True), (384, 128, False), (200, 128, True), (512, 64, False))):
		q, k, v, do, _ = make_inputs(2, S, S, 4, 2, D, torch.bfloat16, 30 + n)
		plan = op.Plan(_dev(q), _dev(k), _dev(v), dout=_dev(do), causal=causal)
		plan.forward()
		plan.backward()
		torch.cuda.synchronize()
		cases.append((plan, [t.clone() for t in (plan.out, plan.dq, plan.dk, plan.dv)]))
	for plan, _ in cases:
		for t in (plan.out, plan.dq, plan.dk, plan.dv):
			t.zero_()
	torch.cuda.synchronize()

	def work(plan):
		stream = torch.cuda.Stream()
		with torch.cuda.stream(stream):
			for _ in range(5):
				plan.forward()
				plan.backward()
		stream.synchronize()

	threads = [threading.Thread(target=work, args=(plan,)) for plan, _ in cases]
	for t in threads:
		t.start()
	for t in threads:
		t.join()
	torch.cuda.synchronize()
	for plan, want in cases:
		for got, ref in zip((plan.out, plan.dq, plan.dk, plan.dv), want):
			assert torch.equal(got, ref)
