"""fa2_bwd_static (the backward entry point that allocates nothing: its scratch is a
buffer built into the library) against fa2_bwd on the same inputs, through the C ABI.

Both run the same kernels, so the results must be bit-identical.  Two calls in a row,
the second on a smaller input: the built-in buffer then still holds the first call's
delta beyond the rows the second call rewrites.
"""

import ctypes

import pytest
import torch

from _cases import make_inputs
from jax_flash_attn2 import _hip_op as op
from jax_flash_attn2 import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(B, S, Hq, Hkv, D, dtype, causal, p_drop=0.0, seed=0, data_seed=0):
	q, k, v, do, _ = make_inputs(B, S, S, Hq, Hkv, D, dtype, data_seed)
	plan = op.Plan(q.to(DEV), k.to(DEV), v.to(DEV), dout=do.to(DEV), causal=causal, dropout_prob=p_drop, dropout_seed=seed)
	plan.forward()
	want = [t.clone() for t in plan.backward()]
	for t in (plan.dq, plan.dk, plan.dv):
		t.fill_(float("nan"))
	# the built-in scratch replaces the caller's: hand the library none at all
	prm = plan.params
	scratch, nbytes = prm.scratch, prm.scratch_bytes
	prm.scratch, prm.scratch_bytes = None, 0
	try:
		_lib.check(plan.lib.fa2_bwd_static(ctypes.byref(prm), torch.cuda.current_stream(DEV).cuda_stream))
	finally:
		prm.scratch, prm.scratch_bytes = scratch, nbytes
	torch.cuda.synchronize()
	for name, a, b in zip(("dq", "dk", "dv"), (plan.dq, plan.dk, plan.dv), want):
		assert torch.equal(a, b), f"{name} differs between fa2_bwd_static and fa2_bwd (B{B} S{S} Hq{Hq} D{D})"


def test_static_scratch_backward_matches_fa2_bwd_twice_in_a_row():
	_both(2, 384, 8, 2, 128, torch.bfloat16, True)
	_both(1, 200, 4, 2, 128, torch.bfloat16, True, data_seed=1)
	_both(2, 130, 4, 4, 64, torch.float16, False, p_drop=0.1, seed=7, data_seed=2)


def test_static_scratch_backward_rejects_sizes_beyond_its_buffer():
	lib = _lib.load()
	q = torch.empty((1, 8, 1, 64), dtype=torch.bfloat16, device=DEV)
	plan = op.Plan(q, q, q, dout=q)
	prm = plan.params
	# B * Hq * Sq * 4 bytes just above 16 MiB; validation only reads the dimensions before it refuses
	prm.Sq = prm.Sk = (16 << 20) // 4 + 64
	rc = lib.fa2_bwd_static(ctypes.byref(prm), torch.cuda.current_stream(DEV).cuda_stream)
	assert rc == -13, rc
	assert b"16 MiB" in lib.fa2_strerror(rc)
