// Exports the dropout keep-mask the attention kernels apply, so that it can be
// checked bit-for-bit against the Philox definition.  Counterpart of
// `tl.rand(seed, offs) > p` in the reference forward
// (jax_flash_attn2/flash_attention_triton/_forward_triton.py:140-143).
#include "fa2_common.hpp"
#include "fa2_kernels.hpp"

namespace fa2 {

// one thread = four consecutive keys of one (b, h, i)
__global__ __launch_bounds__(256) void dropout_mask_kernel(uint8_t* keep, int B, int H, int Sq, int Sk, uint32_t k0,
                                                            uint32_t k1, uint32_t thr, const uint32_t* seed_dev) {
	if (seed_dev) {
		k0 = seed_dev[0];
		k1 = seed_dev[1];
	}
	int nj4 = (Sk + 3) >> 2;
	int64_t total = (int64_t)B * H * Sq * nj4;
	for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
		int j4 = (int)(idx % nj4);
		int64_t r = idx / nj4;
		int i = (int)(r % Sq);
		r /= Sq;
		int h = (int)(r % H);
		int b = (int)(r / H);
		u32x4 rnd = philox4x32_10((uint32_t)j4, (uint32_t)i, (uint32_t)h, (uint32_t)b, k0, k1);
		uint8_t* row = keep + (((int64_t)b * H + h) * Sq + i) * Sk;
#pragma unroll
		for (int e = 0; e < 4; ++e) {
			int j = 4 * j4 + e;
			if (j < Sk) row[j] = rnd[e] >= thr ? 1 : 0;
		}
	}
}

hipError_t launch_dropout_mask(uint8_t* keep, int B, int H, int Sq, int Sk, uint32_t k0, uint32_t k1, uint32_t thr,
                               const uint32_t* seed_dev, hipStream_t s) {
	int64_t total = (int64_t)B * H * Sq * ((Sk + 3) / 4);
	int64_t blocks = (total + 255) / 256;
	if (blocks > 65536) blocks = 65536;
	hipLaunchKernelGGL(dropout_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, keep, B, H, Sq, Sk, k0, k1, thr, seed_dev);
	return hipGetLastError();
}

}  // namespace fa2
