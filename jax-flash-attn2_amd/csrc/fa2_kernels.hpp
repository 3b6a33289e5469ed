// Host <-> kernel argument block and the launchers the C ABI dispatches to.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fa2 {

// Everything a kernel needs, by value.  Strides are in BYTES here (the C ABI
// takes element strides; the launcher converts).
struct KTensor {
	char* ptr;
	int64_t sb, ss, sh;
};

struct KArgs {
	KTensor q, k, v, o, dout, dq, dk, dv;
	float* lse;      // [B, Hq, Sq] natural-log logsumexp
	float* delta;    // [B, Hq, Sq] rowsum(dO * O)  (backward scratch)
	const char* bias;
	int64_t bias_sb, bias_sh, bias_sm;  // bytes
	int bias_dtype;  // FA2_FP16 / FA2_BF16 / FA2_FP32 / FA2_MASK_U8 (bytes: 0 = masked, taken as the bias mask_fill)
	int bias_group;  // head axis of bias indexed by kv-head
	int bias_vec4;   // rows are 4-element aligned: vector loads allowed
	float mask_fill; // FA2_MASK_U8: the additive value of a masked position = lowest finite value of the element type
	int bias_lds;    // bias tiles may be copied global->LDS in 16-byte pieces (see fa2_api.hip)
	char* dbias;     // backward, optional: fp32 [B, Hq, Sq, Sk] gradient of the additive term (dQ kernel variants with bias)
	int64_t dbias_sb, dbias_sh, dbias_sm;  // bytes
	int dbias_atomic;  // entries of dbias are shared by several (batch, q-head) pairs (stride 0 on an axis, or Hkv heads): accumulate with atomic adds
	const int32_t* seqlens;
	const int32_t* kv_lens;  // [B]: keys at or beyond kv_lens[b] are masked (query rows unaffected)
	int B, Sq, Sk, Hq, Hkv;
	int causal;      // (host side only: the kernels read win_right)
	int win_left, win_right;  // row i sees keys i + off - win_left .. i + off + win_right; a negative bound is none; causal = win_right 0
	float scale;
	float softcap;   // > 0: scores become softcap * tanh(scale * q.k / softcap) before bias and mask (kernel variants CAP)
	float cap_k1;    // scale / softcap
	uint32_t drop_k0, drop_k1, drop_thr;
	const uint32_t* seed_dev;  // when set: the Philox key (low word, high word) is read from device memory instead

	float drop_inv_keep;
	int mtiles;      // number of row tiles of the launched kernel
	int xcd_remap;   // 1: group-major placement of workgroups on the 8 XCDs
	                 // 2: batch-major placement, heads of a row tile adjacent (a bias shared by the heads stays in L2)
	// dK/dV kernel on small grids: the streamed steps of a key tile (q-heads of the KV group x query tiles) are split
	// over kv_hsplit workgroups, each leaving fp32 partial dK / dV in dkv_part [kv_hsplit][B][Hkv][Sk][2][D]; a reduce
	// kernel sums, scales and stores them.  1 = no split.
	int kv_hsplit;
	float* dkv_part;
	// dK/dV kernel: a workgroup takes the key tiles p and ntiles - 1 - p one after the other (causal self-attention;
	// a.mtiles then counts pairs); kv_ntiles: key tiles per (batch, kv-head)
	int kv_pair, kv_ntiles;
	int fold_half;   // forward / dQ: workgroup ids from this one on are visited backwards (0 = off; see decode_block())
	int interleave;  // xcd_remap 1: this many (batch, kv-head) groups of an XCD advance through their tiles together (1, 2 or 4)
	int stages;      // backward: bit 0 delta, bit 1 dK/dV, bit 2 dQ
	int dq_makes_delta;  // the dQ kernel computes delta itself (and stores it for the dK/dV kernel)
	// split forward (0 / 1 = off): key ranges of split_len keys, partial results in scratch
	int nsplit, split_len;
	int pack_gqa;     // split forward: one workgroup holds the rows of all q-heads of a kv-head
	float* o_part;    // [nsplit, B, Hq, Sq, D] fp32
	float* lse_part;  // [nsplit, B, Hq, Sq] fp32
};

// dtype: FA2_FP16 / FA2_BF16.  Return hipError_t of the launch.
hipError_t launch_fwd(int dtype, int D, bool bias, bool drop, KArgs& a, hipStream_t s);
hipError_t launch_bwd(int dtype, int D, bool bias, bool drop, KArgs& a, hipStream_t s);
hipError_t launch_dropout_mask(uint8_t* keep, int B, int H, int Sq, int Sk, uint32_t k0, uint32_t k1, uint32_t thr,
                               const uint32_t* seed_dev, hipStream_t s);

// Per-(dtype, D) translation units provide these.
#define FA2_DECL_FWD(TAG, DD) hipError_t launch_fwd_##TAG##_##DD(bool bias, bool drop, KArgs& a, hipStream_t s);
#define FA2_DECL_BWD(TAG, DD) hipError_t launch_bwd_##TAG##_##DD(bool bias, bool drop, KArgs& a, hipStream_t s);
FA2_DECL_FWD(bf16, 64)
FA2_DECL_FWD(bf16, 128)
FA2_DECL_FWD(bf16, 256)
FA2_DECL_FWD(fp16, 64)
FA2_DECL_FWD(fp16, 128)
FA2_DECL_FWD(fp16, 256)
FA2_DECL_BWD(bf16, 64)
FA2_DECL_BWD(bf16, 128)
FA2_DECL_BWD(bf16, 256)
FA2_DECL_BWD(fp16, 64)
FA2_DECL_BWD(fp16, 128)
FA2_DECL_BWD(fp16, 256)

}  // namespace fa2
