#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step = one forward + one backward call through the C ABI (fa2_fwd, fa2_bwd)
on inputs already resident in HBM.  Default workload: the Llama-3-8B-style
prefill shape (B=4, S=4096, Hq=32, Hkv=8, D=128, bf16, causal).

Prints ONE JSON line: whole-step throughput in TFLOP/s (FlashAttention-2 FLOP
convention: fwd = 4*B*Hq*Sq*Sk*D, halved when causal; bwd = 2.5 x fwd), the
roofline entry of the dominant kernel (timed live with HIP events on the
launch stream) and a CPU baseline (the NumPy restatement of the reference's
JAX-platform blockwise algorithm on a bounded sample).
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "jax-flash-attn2_amd"))

PEAK_TFLOPS = {"bf16": 2516.6, "fp16": 2516.6}  # dense MFMA, 256 CU x 2.4 GHz x 4096 FLOP/clk/CU
HBM_PEAK_GBS = 8000.0

WORKLOADS = {
	# name: B, Sq, Sk, Hq, Hkv, D, dtype, causal, bias, dropout, backward
	"c1": dict(B=2, S=512, Hq=16, Hkv=4, D=64, dtype="fp16", causal=True, bias=False, p=0.0, bwd=False,
	           desc="README shape B2 Hq16 Hkv4 S512 D64 fp16 causal, forward only"),
	"c2": dict(B=4, S=4096, Hq=32, Hkv=8, D=128, dtype="bf16", causal=True, bias=False, p=0.0, bwd=True,
	           desc="Llama-3-8B prefill B4 S4096 Hq32 Hkv8 D128 bf16 causal, forward+backward"),
	"c3": dict(B=8, S=2048, Hq=16, Hkv=16, D=64, dtype="bf16", causal=False, bias=True, p=0.0, bwd=True,
	           desc="padded MHA B8 S2048 H16 D64 bf16, bias [B,1,S,S] with mask folded in, forward+backward"),
	"c3_split": dict(B=8, S=2048, Hq=16, Hkv=16, D=64, dtype="bf16", causal=False, bias=True, p=0.0, bwd=True, split_mask=True,
	                 desc="padded MHA B8 S2048 H16 D64 bf16, bias [B,1,S,S] and the per-row key lengths passed separately "
	                      "(kv_lens), forward+backward"),
	"c4": dict(B=1, S=32768, Hq=64, Hkv=8, D=128, dtype="bf16", causal=True, bias=False, p=0.0, bwd=True,
	           desc="long context B1 S32768 Hq64 Hkv8 D128 bf16 causal, forward+backward"),
	"c5": dict(B=8, S=2048, Hq=16, Hkv=16, D=256, dtype="bf16", causal=True, bias=False, p=0.1, bwd=True,
	           desc="dropout, wide heads B8 S2048 H16 D256 bf16 causal p=0.1 seed=42, forward+backward"),
}


def fwd_flops(w):
	f = 4.0 * w["B"] * w["Hq"] * w["S"] * w["S"] * w["D"]
	return f / 2 if w["causal"] else f


def make_inputs(w, device):
	import torch

	dt = torch.bfloat16 if w["dtype"] == "bf16" else torch.float16
	g = torch.Generator(device=device)
	B, S, Hq, Hkv, D = w["B"], w["S"], w["Hq"], w["Hkv"], w["D"]
	mul = 1.0 if w is WORKLOADS["c1"] else 0.5

	def rnd(seed, shape, m):
		g.manual_seed(seed)
		return (torch.randn(shape, generator=g, device=device, dtype=torch.float32) * m).to(dt)

	q = rnd(0, (B, S, Hq, D), mul)
	k = rnd(1, (B, S, Hkv, D), mul)
	v = rnd(2, (B, S, Hkv, D), mul)
	do = rnd(3, (B, S, Hq, D), 1.0)
	bias = kv_lens = None
	if w["bias"]:
		# bias[b,0,i,j] = 1/(1+|i-j|) ; keys beyond a per-row valid length get finfo.min
		i = torch.arange(S, device=device)
		base = 1.0 / (1.0 + (i[:, None] - i[None, :]).abs().float())
		g.manual_seed(4)
		lens = torch.randint(S // 2, S + 1, (B,), generator=g, device=device)
		valid = i[None, :] < lens[:, None]
		bias = base[None, None].expand(B, 1, S, S).clone()
		if w.get("split_mask"):
			bias = bias.to(dt)
			kv_lens = lens.to(torch.int32).contiguous()
		else:
			bias = torch.where(valid[:, None, None, :], bias, torch.full_like(bias, torch.finfo(dt).min)).to(dt)
	return q, k, v, do, bias, kv_lens


def event_time_ms(fn, iters, torch):
	"""Average duration of fn() over `iters` launches, HIP events on the current stream."""
	start = torch.cuda.Event(enable_timing=True)
	stop = torch.cuda.Event(enable_timing=True)
	start.record()
	for _ in range(iters):
		fn()
	stop.record()
	stop.synchronize()
	return start.elapsed_time(stop) / iters


def measured_traffic(workload, kernel):
	"""HBM bytes per launch of `kernel` from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE runs, or None."""
	path = os.path.join(ROOT, "profiles", f"{workload}_traffic.json")
	try:
		with open(path) as f:
			rec = json.load(f)
	except (OSError, ValueError):
		return None
	return rec.get("hbm_bytes_per_launch") if rec.get("kernel") == kernel else None


def mfma_peak(torch, dev):
	"""What the chip sustains on bf16 matrix products alone (random operands), and at which clock."""
	import ctypes

	# the measurement kernel lives in its own small library beside the product library
	path = os.path.join(ROOT, "jax-flash-attn2_amd", "libfa2_bench.so")
	if not os.path.exists(path):
		return None
	lib = ctypes.CDLL(path)
	lib.fa2_bench_mfma.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
	lib.fa2_bench_mfma.restype = ctypes.c_int
	wgs, iters = 1024, 2000
	buf = torch.zeros(16 + wgs * 2048, dtype=torch.uint8, device=dev)
	st = torch.cuda.current_stream(dev).cuda_stream

	def run(n):
		rc = lib.fa2_bench_mfma(buf.data_ptr(), buf.numel(), wgs, n, st)
		if rc:
			raise RuntimeError(f"fa2_bench_mfma failed ({rc})")

	run(iters)  # settle the clocks
	torch.cuda.synchronize()
	ms = event_time_ms(lambda: run(iters), 3, torch)
	ticks = buf[:16].cpu().view(torch.int64)
	flops = wgs * 8.0 * iters * 32 * 32768
	return {"tflops": flops / (ms * 1e-3) / 1e12, "clock_mhz": float(ticks[0]) / (float(ticks[1]) / 100.0),
	        "what": "v_mfma_f32_32x32x16_bf16 only, random operands, 8 waves/CU x 4 chains whose accumulators stay live "
	                "over the whole loop"}


def cpu_baseline(w):
	"""Reference JAX-platform algorithm (NumPy restatement) on a bounded sample of the workload."""
	sys.path.insert(0, os.path.join(ROOT, "oracle"))
	import numpy as np

	import fa2_oracle as O

	r = w["Hq"] // w["Hkv"]
	# bounded sample: at most two batch entries and 4096 positions of the workload, all heads
	# (10 - 20 s on 16 host cores for the workloads with S >= 4096)
	B, S, D = min(w["B"], 2), min(w["S"], 4096), w["D"]
	Hkv = w["Hkv"]
	Hq = Hkv * r
	rng = np.random.default_rng(0)
	q = rng.standard_normal((B, S, Hq, D), dtype=np.float32) * 0.5
	k = rng.standard_normal((B, S, Hkv, D), dtype=np.float32) * 0.5
	v = rng.standard_normal((B, S, Hkv, D), dtype=np.float32) * 0.5
	do = rng.standard_normal((B, S, Hq, D), dtype=np.float32)
	def timed(mask):
		t0 = time.perf_counter()
		if w["bwd"]:
			O.jax_platform_call(q, k, v, with_grads_for=do, mask=mask)
		else:
			O.jax_platform_call(q, k, v, mask=mask)
		return time.perf_counter() - t0

	cores = os.cpu_count() if not os.environ.get("OMP_NUM_THREADS") else int(os.environ["OMP_NUM_THREADS"])
	mult = 3.5 if w["bwd"] else 1.0
	what = f"B={B} Hq={Hq} Hkv={Hkv} S={S} D={D} fp32, {'fwd+bwd' if w['bwd'] else 'fwd'}, blocks 128x128"
	# as the reference's facade runs it: that branch never applies the causal mask, it computes the full S x S problem
	dt = timed(None)
	out = {
		"value": 4.0 * B * Hq * S * S * D * mult / dt / 1e12,
		"unit": "TFLOP/s",
		"cores": cores,
		"kind": "port",
		"sample": f"{what}, non-causal (the reference's JAX branch ignores causal), {dt:.1f} s",
		"seconds": dt,
	}
	if w["causal"]:
		# the same functions given a causal mask (they then skip the blocks above the diagonal); FLOPs counted as for the GPU
		tri = np.tril(np.ones((S, S), dtype=bool))[None, None]
		dtc = timed(tri)
		out["causal"] = {
			"value": 2.0 * B * Hq * S * S * D * mult / dtc / 1e12,
			"unit": "TFLOP/s",
			"sample": f"{what}, causal mask with block skipping, {dtc:.1f} s",
			"seconds": dtc,
		}
	return out


def reference_grid(torch, op, dev, args):
	"""Forward-only times over the shapes named by the result files under the reference's benchmarks/
	(`b=<B>-ub=<bias>-hdim=<D>-qh=<Hq>-kvh=<Hkv>-mode=fwd.csv`, rows seqlen 1024 ... 8192).  Those files record neither
	dtype, causal flag nor the bias shape: here bf16, non-causal, bias [B, Hq, S, S] (the most traffic a bias can bring)."""
	print("| B | bias | D | Hq | Hkv | S | ms | TFLOP/s |")
	print("|---|---|---|---|---|---|---|---|")
	for B in (1, 2, 4):
		for ub in (False, True):
			for D in (64, 128, 256):
				for Hq, Hkv in ((16, 8), (32, 16)):
					for S in (1024, 2048, 4096, 6144, 8192):
						w = dict(B=B, S=S, Hq=Hq, Hkv=Hkv, D=D, dtype="bf16", causal=False, bias=False, p=0.0, bwd=False)
						q, k, v, _, _, _ = make_inputs(w, dev)
						bias = torch.empty((B, Hq, S, S), dtype=torch.bfloat16, device=dev).normal_() if ub else None
						plan = op.Plan(q, k, v, bias=bias, causal=False)
						t_pre = time.perf_counter()
						while time.perf_counter() - t_pre < 0.1:
							plan.forward()
							torch.cuda.synchronize()
						ms = event_time_ms(plan.forward, max(3, min(args.steps, 20)), torch)
						print(f"| {B} | {'yes' if ub else 'no'} | {D} | {Hq} | {Hkv} | {S} | {ms:.4f} | {fwd_flops(w) / (ms * 1e-3) / 1e12:.0f} |", flush=True)
						del plan, q, k, v, bias


def main():
	ap = argparse.ArgumentParser()
	ap.add_argument("--gpus", type=int, default=1)
	ap.add_argument("--steps", type=int, default=50)
	ap.add_argument("--warmup", type=int, default=5)
	ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
	ap.add_argument("--no-cpu-baseline", action="store_true")
	ap.add_argument("--no-mfma-peak", action="store_true", help="skip the matrix-product-only microbenchmark")
	ap.add_argument("--no-power-check", action="store_true",
	                help="skip the rerun of the same launches on all-zero operands (tells whether the timed run was clock-throttled)")
	ap.add_argument("--copy-calibration", action="store_true",
	                help="also run a plain 1 GiB device copy (known traffic) so that rocprofv3 FETCH_SIZE / WRITE_SIZE "
	                     "readings of the attention kernels can be scaled")
	ap.add_argument("--reference-grid", action="store_true",
	                help="instead of one workload: forward times over the grid of shapes the reference's benchmarks/ folder "
	                     "holds results for (batch, bias, head dim, heads, sequence length); prints a markdown table")
	args = ap.parse_args()
	if args.gpus != 1:
		print("bench.py: this build measures ONE GPU; --gpus N with N > 1 is not supported "
		      "(attention shards over batch and KV-head groups without communication).", file=sys.stderr)
		sys.exit(2)

	import torch

	from jax_flash_attn2 import _hip_op as op

	if not torch.cuda.is_available():
		print("bench.py: no GPU visible", file=sys.stderr)
		sys.exit(1)
	dev = torch.device("cuda:0")
	if args.reference_grid:
		reference_grid(torch, op, dev, args)
		return
	w = WORKLOADS[args.workload]
	q, k, v, do, bias, kv_lens = make_inputs(w, dev)
	plan = op.Plan(q, k, v, dout=do if w["bwd"] else None, bias=bias, causal=w["causal"], dropout_prob=w["p"],
	               dropout_seed=42 if w["p"] > 0 else None, kv_lens=kv_lens)

	def step():
		plan.forward()
		if w["bwd"]:
			plan.backward()

	if args.copy_calibration:
		src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
		dst = torch.empty_like(src)
		for _ in range(3):
			dst.copy_(src)
		torch.cuda.synchronize()
		del src, dst

	# Untimed pre-roll: after idling the GPU needs some hundred milliseconds of work before its
	# clocks settle (the first steps after start-up run 10-15 % slower than the steady state).
	t_pre = time.perf_counter()
	while time.perf_counter() - t_pre < 0.5:
		for _ in range(5):
			step()
		torch.cuda.synchronize()

	for _ in range(args.warmup):
		step()
	torch.cuda.synchronize()
	t0 = time.perf_counter()
	for _ in range(args.steps):
		step()
	torch.cuda.synchronize()
	ms = (time.perf_counter() - t0) * 1e3 / args.steps

	ff = fwd_flops(w)
	if kv_lens is not None:
		# only the valid keys count as work
		ff *= float(kv_lens.float().mean()) / w["S"]
	total = ff * (3.5 if w["bwd"] else 1.0)
	tflops = total / (ms * 1e-3) / 1e12

	# Per-kernel durations: HIP events on the launch stream, recorded between the launches of whole steps, so each
	# kernel is timed in the place it has in a step (after the kernel that precedes it there, at the clock the step
	# runs at).  The backward of a step is two launches: the dQ kernel, which also forms delta (stages 5), then the
	# dK/dV kernel (stages 2) - together exactly the launches of fa2_bwd.
	it = max(3, min(args.steps, 20))
	names = ["fwd", "bwd_dq", "bwd_dkdv"] if w["bwd"] else ["fwd"]
	calls = {"fwd": plan.forward, "bwd_dq": lambda: plan.backward(5), "bwd_dkdv": lambda: plan.backward(2)}
	evs = [[torch.cuda.Event(enable_timing=True) for _ in range(len(names) + 1)] for _ in range(it)]
	for _ in range(2):
		step()
	for e in evs:
		e[0].record()
		for i, n in enumerate(names):
			calls[n]()
			e[i + 1].record()
	torch.cuda.synchronize()
	kern = {n: sum(e[i].elapsed_time(e[i + 1]) for e in evs) / it for i, n in enumerate(names)}
	alg = {"fwd": ff}
	if w["bwd"]:
		# 5-product convention: S, dP, dV, dK belong to the dK/dV kernel (4 x 0.5 fwd), dQ to the dQ kernel;
		# the dQ kernel's recomputation of S and dP is not counted.
		alg["bwd_dkdv"] = 2.0 * ff
		alg["bwd_dq"] = 0.5 * ff
	dom = max((n for n in kern if n in alg), key=lambda n: kern[n])
	peak = PEAK_TFLOPS[w["dtype"]]
	achieved = alg[dom] / (kern[dom] * 1e-3) / 1e12
	roofline = {
		"kernel": dom,
		"bound": "mfma",
		"achieved": achieved,
		"peak": peak,
		"unit": "TFLOP/s",
		"frac": achieved / peak,
		"traffic": measured_traffic(args.workload, dom),
		"traffic_source": "committed rocprofv3 FETCH_SIZE / WRITE_SIZE runs (profiles/), not measured in this run",
		"kernel_ms": {n: round(t, 4) for n, t in kern.items()},
		"kernel_tflops": {n: round(alg[n] / (kern[n] * 1e-3) / 1e12, 1) for n in kern if n in alg},
	}

	out = {
		"metric": "attention TFLOP/s fwd+bwd (bf16 causal)" if args.workload == "c2" else f"attention TFLOP/s ({args.workload})",
		"value": tflops,
		"unit": "TFLOP/s",
		"n_gpus": 1,
		"steps": args.steps,
		"warmup": args.warmup,
		"ms_per_step": ms,
		"higher_is_better": True,
		"scaling": "weak",
		"vs_baseline": None,
		"dtype": w["dtype"],
		"data": "synthetic",
		"config": {"workload": w["desc"]},
		"pct_of_mfma_peak": 100.0 * tflops / peak,
		"roofline": roofline,
	}
	if not args.no_power_check:
		# The same launches on all-zero q, k, v, dO: the instruction stream, the masks and the memory traffic are those
		# of the timed run, only the switching activity of the data is gone.  Where this runs faster, the timed run was
		# held below the 2.4 GHz clock by the chip's power limit, not by the kernels' instruction issue.
		for t in (q, k, v, do):
			t.zero_()
		t_pre = time.perf_counter()
		while time.perf_counter() - t_pre < 0.3:
			for _ in range(5):
				step()
			torch.cuda.synchronize()
		t0 = time.perf_counter()
		for _ in range(args.steps):
			step()
		torch.cuda.synchronize()
		ms0 = (time.perf_counter() - t0) * 1e3 / args.steps
		out["zero_operands"] = {"ms_per_step": ms0, "speedup_over_timed_run": ms / ms0,
		                        "what": "same launches, q = k = v = dO = 0 (identical instruction stream and traffic)"}
	if not args.no_mfma_peak:
		mp = mfma_peak(torch, dev)
		if mp is not None:
			out["mfma_peak_measured"] = mp
			roofline["frac_of_measured_peak"] = achieved / mp["tflops"]
	if not args.no_cpu_baseline:
		out["cpu_baseline"] = cpu_baseline(w)
	print(json.dumps(out))


if __name__ == "__main__":
	main()
