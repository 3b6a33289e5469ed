"""Shared helpers of the GPU parity tests: seeded inputs, oracle comparison, tolerances."""

import numpy as np
import torch

import fa2_oracle as O

# north-star tolerances: max-abs on O (against an fp32/fp64 evaluation), relative L2 on gradients
TOL_O = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
TOL_GRAD_REL_L2 = 1e-2
TOL_LSE = 1e-2


def make_inputs(B, Sq, Sk, Hq, Hkv, D, dtype, seed=0, bias_shape=None, scale=0.5, bias_dtype=None, qk_scale=None):
	"""Seeded CPU tensors, already rounded to `dtype`, so the oracle consumes the kernel's exact inputs.
	qk_scale: standard deviation of q and k when it differs from that of v (the scores of a head of
	dim D then have a standard deviation of qk_scale^2 at the default softmax scale)."""
	g = torch.Generator().manual_seed(seed)
	qs = scale if qk_scale is None else qk_scale
	q = (torch.randn(B, Sq, Hq, D, generator=g) * qs).to(dtype)
	k = (torch.randn(B, Sk, Hkv, D, generator=g) * qs).to(dtype)
	v = (torch.randn(B, Sk, Hkv, D, generator=g) * scale).to(dtype)
	do = torch.randn(B, Sq, Hq, D, generator=g).to(dtype)
	bias = None
	if bias_shape is not None:
		bias = torch.randn(*bias_shape, generator=g).to(bias_dtype or dtype)
	return q, k, v, do, bias


def f64(t):
	return None if t is None else t.to(torch.float64).numpy()


def check_forward(o, lse, o_ref, lse_ref, dtype, what=""):
	o = o.float().cpu().numpy()
	lse = lse.float().cpu().numpy()
	err = np.abs(o - o_ref).max()
	assert np.isfinite(o).all(), f"{what}: non-finite output"
	assert err <= TOL_O[dtype], f"{what}: O max-abs {err:.3e} > {TOL_O[dtype]}"
	fin = np.isfinite(lse_ref)
	assert np.array_equal(np.isneginf(lse), ~fin), f"{what}: -inf pattern of LSE differs"
	if fin.any():
		e = np.abs(lse[fin] - lse_ref[fin]).max()
		assert e <= TOL_LSE, f"{what}: LSE max-abs {e:.3e}"


def check_grads(got, ref, what="", stored=None):
	"""stored: the oracle's gradients with delta formed from O as the backward pass really receives it (rounded to
	16 bits) - the size of what legitimately survives where the exact gradient cancels to zero."""
	for n, (name, a, b) in enumerate(zip(("dq", "dk", "dv"), got, ref)):
		a = a.float().cpu().numpy()
		assert np.isfinite(a).all(), f"{what}: non-finite {name}"
		if np.abs(b).max() <= 1e-10:
			# a gradient that is zero up to fp64 rounding (e.g. a single key: dS = P (dP - delta) = 0) may come
			# back as rounding noise of delta
			# (delta is formed from O rounded to 16 bits: up to 2^-8 of |dP| survives the subtraction, summed over the rows)
			floor = 0.0 if stored is None else float(np.abs(stored[n]).max())
			assert np.abs(a).max() <= 1e-2 + 2.0 * floor, f"{what}: {name} should be zero (max-abs {np.abs(a).max():.3e}, rounding floor {floor:.3e})"
			continue
		e = O.rel_l2(a, b)
		assert e <= TOL_GRAD_REL_L2, f"{what}: {name} rel-L2 {e:.3e} > {TOL_GRAD_REL_L2}"
