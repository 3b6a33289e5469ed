#!/usr/bin/env python3
"""Writes the golden fixtures in this directory from the NumPy oracle
(oracle/fa2_oracle.py).  The reference ships no test vectors for this path, so
the fixtures guard the oracle itself against regressions and give the GPU
tests something to check without recomputing.  Inputs are bf16-representable
fp32 so that a 16-bit kernel consumes exactly the same numbers.

    python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "oracle"))
import fa2_oracle as O  # noqa: E402

CASES = {
	# name: (B, Sq, Sk, Hq, Hkv, D, causal, bias_shape, seqlens, p_drop, seed)
	"mha_d64": (1, 33, 33, 4, 4, 64, False, None, None, 0.0, 0),
	"gqa_causal_d64": (1, 33, 33, 4, 2, 64, True, None, None, 0.0, 0),
	"gqa_causal_d128_sq_lt_sk": (1, 16, 40, 4, 2, 128, True, None, None, 0.0, 0),
	"causal_sq_gt_sk_d64": (1, 40, 16, 2, 2, 64, True, None, None, 0.0, 0),
	"bias_b1_d64": (2, 33, 33, 4, 2, 64, False, (2, 1, 33, 33), None, 0.0, 0),
	"bias_group_causal_d128": (1, 20, 20, 4, 2, 128, True, (1, 2, 20, 20), None, 0.0, 0),
	"seqlens_d64": (3, 24, 24, 2, 2, 64, True, None, (24, 7, 0), 0.0, 0),
	"dropout_causal_d64": (1, 33, 33, 4, 2, 64, True, None, None, 0.1, 42),
	"dropout_d256": (1, 16, 16, 2, 2, 256, False, None, None, 0.25, (3 << 32) | 99),
}


def main():
	for idx, (name, (B, Sq, Sk, Hq, Hkv, D, causal, bshape, seqlens, p, seed)) in enumerate(sorted(CASES.items())):
		rng = np.random.default_rng(1000 + idx)
		q = O.round_bf16(rng.normal(size=(B, Sq, Hq, D)) * 0.5)
		k = O.round_bf16(rng.normal(size=(B, Sk, Hkv, D)) * 0.5)
		v = O.round_bf16(rng.normal(size=(B, Sk, Hkv, D)) * 0.5)
		dout = O.round_bf16(rng.normal(size=(B, Sq, Hq, D)))
		kw = dict(causal=causal, p_drop=p, seed=seed)
		out = dict(q=q, k=k, v=v, dout=dout, causal=causal, p_drop=p, seed=np.uint64(seed))
		if bshape:
			kw["bias"] = out["bias"] = O.round_bf16(rng.normal(size=bshape))
		if seqlens:
			kw["seqlens"] = out["seqlens"] = np.asarray(seqlens, np.int32)
		o, lse = O.attention_fwd(q, k, v, **kw)
		dq, dk, dv = O.attention_bwd(q, k, v, dout, **kw)
		out.update(o=o.astype(np.float32), lse=lse.astype(np.float32), dq=dq.astype(np.float32), dk=dk.astype(np.float32),
		           dv=dv.astype(np.float32))
		if p > 0:
			out["keep_bits"] = np.packbits(O.dropout_keep_mask(seed, p, B, Hq, Sq, Sk))
		np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
		print(name, "ok")


if __name__ == "__main__":
	main()
