// Measurement aid, built into its own libfa2_bench.so (bench.py loads it; the product library does not
// contain it): what the matrix pipe of this chip sustains on nothing but v_mfma_f32_32x32x16_bf16 with
// random operands.  The attention kernels are priced against the data-sheet peak (2.4 GHz); under sustained
// matrix load the chip settles at a lower clock (power limit), and this number says where.  No counterpart
// in the reference.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "fa2_common.hpp"

namespace fa2 {

// 8 waves per workgroup (two per SIMD), 4 independent chains per wave.  The accumulators stay live over the
// whole loop - nothing is zeroed or read inside it, so the matrix pipe never drains - and are read once at the end.
// result[0..1] (workgroup 0): shader-clock cycles and 100 MHz wall-clock ticks of the loop.
__global__ __launch_bounds__(512) void mfma_peak_kernel(float* sink, unsigned long long* result, int iters) {
	unsigned long long c0 = clock64(), w0 = wall_clock64();
	bf16x8 a[8], b[8];
	uint32_t st = 0x9E3779B9u * (threadIdx.x + 1) + 0x85EBCA6Bu * (blockIdx.x + 1);
	auto next = [&]() {
		st = st * 1664525u + 1013904223u;
		return (float)(int)(st >> 8) * (1.0f / 8388608.0f) - 1.0f;  // uniform in [-1, 1)
	};
#pragma unroll
	for (int i = 0; i < 8; ++i)
#pragma unroll
		for (int e = 0; e < 8; ++e) {
			a[i][e] = (__bf16)next();
			b[i][e] = (__bf16)next();
		}
	f32x16 acc[4];
#pragma unroll
	for (int j = 0; j < 4; ++j)
#pragma unroll
		for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
	for (int it = 0; it < iters; ++it) {
#pragma unroll
		for (int u = 0; u < 8; ++u)
#pragma unroll
			for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + j) & 7], b[u], acc[j], 0, 0, 0);
	}
	float s = acc[0][0] + acc[1][1] + acc[2][2] + acc[3][3];
	if (blockIdx.x == 0 && threadIdx.x == 0) {
		result[0] = clock64() - c0;
		result[1] = wall_clock64() - w0;
	}
	sink[(size_t)blockIdx.x * 512 + threadIdx.x] = s;
}

}  // namespace fa2

// Launches `workgroups` workgroups of 8 waves that each run `iters` x 32 v_mfma_f32_32x32x16_bf16 on random operands
// and nothing else.  FLOPs = workgroups * 8 * iters * 32 * 32768; the caller times the launch.  scratch (device,
// >= 16 + workgroups * 2048 bytes): on completion its first two uint64 hold workgroup 0's shader-clock cycles and
// 100 MHz wall-clock ticks, i.e. the clock the chip sustained.  Returns 0, or -1 for bad arguments, -2 for a failed launch.
extern "C" int fa2_bench_mfma(void* scratch, size_t scratch_bytes, int workgroups, int iters, void* hip_stream) {
	if (!scratch || workgroups <= 0 || iters <= 0) return -1;
	if (scratch_bytes < 16 + (size_t)workgroups * 512 * sizeof(float)) return -1;
	unsigned long long* result = (unsigned long long*)scratch;
	float* sink = (float*)((char*)scratch + 16);
	hipLaunchKernelGGL(fa2::mfma_peak_kernel, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)hip_stream, sink, result, iters);
	return hipGetLastError() == hipSuccess ? 0 : -2;
}
