// Exports the dropout keep-mask the attention kernels apply, so that it can be
// checked bit-for-bit against the Philox definition.  Counterpart of
// `tl.rand(seed, offs) > p` in the reference forward
// (jax_flash_attn2/flash_attention_triton/_forward_triton.py:140-143).
#include "fa2_common.hpp"
#include "fa2_kernels.hpp"

namespace fa2 {

// one thread = one generator call: two adjacent rows x four consecutive keys of one (b, h)
__global__ __launch_bounds__(256) void dropout_mask_kernel(uint8_t* keep, int B, int H, int Sq, int Sk, uint32_t k0,
                                                            uint32_t k1, uint32_t thr, const uint32_t* seed_dev) {
	if (seed_dev) {
		k0 = seed_dev[0];
		k1 = seed_dev[1];
	}
	int nj4 = (Sk + 3) >> 2, ni2 = (Sq + 1) >> 1;
	int64_t total = (int64_t)B * H * ni2 * nj4;
	for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
		int j4 = (int)(idx % nj4);
		int64_t r = idx / nj4;
		int i2 = (int)(r % ni2);
		r /= ni2;
		int h = (int)(r % H);
		int b = (int)(r / H);
		u32x4 rnd = philox4x32_10((uint32_t)j4, (uint32_t)i2, (uint32_t)h, (uint32_t)b, k0, k1);
#pragma unroll
		for (int v = 0; v < 8; ++v) {
			int i = 2 * i2 + (v >> 2), j = 4 * j4 + (v & 3);
			if (i < Sq && j < Sk) keep[(((int64_t)b * H + h) * Sq + i) * Sk + j] = keep16(rnd[v >> 1], v & 1, thr) ? 1 : 0;
		}
	}
}

hipError_t launch_dropout_mask(uint8_t* keep, int B, int H, int Sq, int Sk, uint32_t k0, uint32_t k1, uint32_t thr,
                               const uint32_t* seed_dev, hipStream_t s) {
	int64_t total = (int64_t)B * H * ((Sq + 1) / 2) * ((Sk + 3) / 4);
	int64_t blocks = (total + 255) / 256;
	if (blocks > 65536) blocks = 65536;
	hipLaunchKernelGGL(dropout_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, keep, B, H, Sq, Sk, k0, k1, thr, seed_dev);
	return hipGetLastError();
}

}  // namespace fa2
