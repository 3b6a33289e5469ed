/*
 * fa2.h - C ABI of libfa2_hip.so: Flash-Attention-2 forward and backward for
 * AMD MI355X (gfx950), hand-written HIP kernels.
 *
 * This is the operator boundary of the hot path.  It takes the place of the
 * XLA custom calls that the reference emits through
 * eformer.callib.triton_call(...) at
 *   jax_flash_attn2/flash_attention_triton/_forward_triton.py:547-588   (forward)
 *   jax_flash_attn2/flash_attention_triton/_backward_triton.py:1049-1080 (delta pre-pass)
 *   jax_flash_attn2/flash_attention_triton/_backward_triton.py:1082-1154 (dK/dV/dQ)
 * Arrays become device pointers, Python scalars become struct fields, outputs
 * are caller-allocated buffers.  The library never allocates, frees or
 * synchronises; every launch goes to the caller's stream.
 *
 * Tensor layout (same as the reference API, flash_attention.py:186-187):
 *   q, o, dO, dq : [B, Sq, Hq,  D]     k, v, dk, dv : [B, Sk, Hkv, D]
 * with arbitrary element strides for batch / sequence / head and a unit
 * stride on D (the reference assumes the same, _forward_triton.py:296,304,312).
 * q-head h reads kv-head h / (Hq / Hkv)  (_forward_triton.py:263-264).
 */
#ifndef FA2_H_
#define FA2_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types; the values mirror dtype_index() in
 * jax_flash_attn2/flash_attention_triton/_utils.py:75-82. */
enum { FA2_FP16 = 1, FA2_BF16 = 2, FA2_FP32 = 3 /* bias only */, FA2_MASK_U8 = 4 /* bias only: boolean mask, see `bias` */ };

/* Return codes. 0 = success, negative = error; nothing is launched on error. */
enum {
	FA2_OK = 0,
	FA2_EINVAL_STRUCT = -1,   /* NULL params or struct_size < FA2_PARAMS_SIZE_V1  */
	FA2_EINVAL_DTYPE = -2,    /* q/k/v dtype not fp16/bf16 (_forward_triton.py:494-495) */
	FA2_EINVAL_SHAPE = -3,    /* non-positive dimension, or scale not finite and > 0 */
	FA2_EINVAL_HEADS = -4,    /* Hq % Hkv != 0 (flash_attention.py:189-193)      */
	FA2_EINVAL_PTR = -5,      /* required pointer is NULL or not 16-byte aligned */
	FA2_EINVAL_STRIDE = -6,   /* stride not a multiple of 8 elements, or a sequence
	                             stride that is negative or above 2^31 / 256 elements */
	FA2_EINVAL_DROPOUT = -7,  /* p_drop outside [0, 1)                           */
	FA2_EINVAL_BIAS = -8,     /* bias dtype / stride invalid                     */
	FA2_EINVAL_MASK = -9,     /* seqlens given together with bias or with Sq != Sk
	                             (_forward_triton.py:474-481)                    */
	FA2_EUNSUPPORTED = -10,   /* head dim not in {64, 128, 256}                  */
	FA2_ESCRATCH = -11,       /* backward scratch missing or too small           */
	FA2_EHIP = -12,           /* HIP runtime reported a launch error             */
	FA2_ESCRATCH_STATIC = -13 /* fa2_bwd_static: the call needs more than
	                             FA2_STATIC_SCRATCH_BYTES of scratch             */
};

typedef struct fa2_tensor {
	void* ptr;          /* device pointer, 16-byte aligned                */
	int64_t stride_b;   /* element stride between batches                 */
	int64_t stride_s;   /* element stride between sequence positions      */
	int64_t stride_h;   /* element stride between heads; D stride is 1    */
} fa2_tensor;

typedef struct fa2_params {
	uint32_t struct_size;   /* = sizeof(fa2_params) of the header the caller was built
	                           with (>= FA2_PARAMS_SIZE_V1), checked first */
	int32_t dtype;          /* FA2_FP16 | FA2_BF16 for q,k,v,o,dO,dq,dk,dv */
	int32_t B, Sq, Sk, Hq, Hkv, D;
	int32_t causal;         /* bottom-right aligned: j <= i + Sk - Sq
	                           (_forward_triton.py:127-132)                */
	float scale;            /* softmax scale, must be > 0; applied to the fp32 result of q.k^T,
	                           as the reference does (_forward_triton.py:281)  */
	float p_drop;           /* dropout probability in [0,1); realised in steps of 2^-16: an element is dropped
	                           with probability floor(p_drop * 65536) / 65536 and kept values are scaled by the
	                           reciprocal of the realised keep probability, so E[O] is exact (see fa2_dropout_mask) */
	uint64_t seed;          /* Philox key for the dropout keep-mask        */

	fa2_tensor q, k, v, o;  /* o is written by fa2_fwd, read by fa2_bwd    */
	float* lse;             /* [B, Hq, Sq] fp32, natural-log logsumexp; -inf for
	                           rows without any allowed key.  Written by fa2_fwd,
	                           read by fa2_bwd.                            */

	/* Optional additive bias [B|1, Hq|Hkv|1, Sq, Sk], unit stride on Sk.
	 * stride 0 on batch / head = broadcast (calc_bias_strides, _utils.py:151-193).
	 * bias_group != 0: the head axis has Hkv entries and q-head h reads entry
	 * h / (Hq/Hkv) (flash_attention.py:161-164 materialises this repeat).   */
	const void* bias;       /* NULL = no bias                              */
	int32_t bias_dtype;     /* FA2_FP16 | FA2_BF16 | FA2_FP32, or FA2_MASK_U8: `bias` then points to a
	                           boolean mask, one byte per position (0 = masked), same shape and stride
	                           rules with strides in bytes.  A masked position adds the lowest finite
	                           value of `dtype` to the score - exactly what the bias
	                           where(mask, 0, finfo(dtype).min) of README.md:188 does, at one byte
	                           per position instead of two or four */
	int32_t bias_group;
	int64_t bias_stride_b, bias_stride_h, bias_stride_m;

	/* Optional per-batch valid length (the reference's 2-D right-padded
	 * attention_mask reduced to lengths, _forward_triton.py:499-510): keys
	 * j >= seqlens[b] are masked, query rows i >= seqlens[b] give zeros.
	 * Requires Sq == Sk and no bias.                                       */
	const int32_t* seqlens; /* [B] int32 on device, NULL = all full        */

	/* Backward only. */
	fa2_tensor dout;        /* dO, read                                    */
	fa2_tensor dq, dk, dv;  /* written; dk/dv already summed over each KV group */
	/* Backward: required, >= fa2_bwd_scratch_bytes(p) bytes.  Forward: optional, see
	 * fa2_fwd_scratch_bytes().  256-byte aligned. */
	void* scratch;
	uint64_t scratch_bytes;

	/* --- fields added after the first version of this header (FA2_PARAMS_SIZE_V1 bytes);
	 *     a caller that passes the shorter struct_size gets zeros for them --- */

	/* Optional: the Philox key as a 64-bit value in DEVICE memory (8-byte aligned).  When
	 * non-NULL the kernels read it there and `seed` is ignored, so the key can be an
	 * ordinary runtime operand of the caller's graph - the reference passes its
	 * dropout_seed to the custom call as an operand, not as a compile-time constant
	 * (_forward_triton.py:553, _flash_attention.py:91-92) - and changing it needs neither a
	 * new parameter block nor, under XLA, a new executable.                              */
	const uint64_t* seed_dev;

	/* Optional per-batch number of valid KEYS: keys j >= kv_lens[b] are masked, query rows
	 * are not touched and causal / window stay aligned to the FULL Sk (row i is aligned with key i + Sk - Sq).
	 * This differs on purpose from the key_padding_mask of the reference's naive attention, which aligns its
	 * window to the number of valid keys (refrence_call.py:58-66): kv_lens describes padding at the end of a
	 * key axis whose positions keep their meaning (a KV cache, a bias that is indexed by absolute key), so
	 * shortening a batch row must not shift which keys a query row may see.  Callers that want the other
	 * alignment shift `window_left / window_right` by Sk - kv_len themselves (one batch row per call), or use
	 * `seqlens`, which shortens both axes.  Unlike `seqlens` it may be
	 * combined with a bias and with Sq != Sk (key padding of cross attention, or of a
	 * batch that also carries a bias); key tiles beyond the length are skipped, not
	 * masked.  A row left without any allowed key gives O = 0 and lse = -inf.       */
	const int32_t* kv_lens; /* [B] int32 on device, NULL = all Sk keys     */

	/* Optional sliding window (has_window != 0), the window_size of the reference's naive
	 * attention (refrence_call.py:32,55-75): query row i attends to keys
	 *   i + (Sk - Sq) - window_left  ..  i + (Sk - Sq) + window_right
	 * where a negative bound means no bound on that side.  `causal` sets the right bound to 0
	 * (refrence_call.py:36-37).  A row left without any key gives O = 0 and lse = -inf
	 * (the reference zeroes such rows, :80-82).  Key tiles outside the window are skipped.  */
	int32_t has_window, window_left, window_right;

	/* Optional tanh soft-capping of the scores (> 0): softcap * tanh(scale q.k / softcap) takes the
	 * place of scale q.k, before bias and masks, as in the reference's naive attention
	 * (refrence_call.py:33,48-51); the backward carries the factor 1 - tanh^2.  0 = off.      */
	float softcap;

	/* Optional gradient of the additive bias (backward only; requires `bias` or `softcap`, i.e. the kernel
	 * variants that carry an additive term).  fp32, element strides as given, unit stride on Sk, 16-byte aligned
	 * with strides that are multiples of 4.  The dQ kernel adds, per (batch b, q-head h),
	 *   P[i, j] * (dP[i, j] - delta[i])
	 * - the gradient with respect to the term added to the score (before the softmax scale reaches dQ / dK and
	 * before the 1 - tanh^2 factor of soft-capping) - to dbias[b, h', i, j], h' = h, or h / (Hq / Hkv) when
	 * bias_group is set.  Two layouts:
	 *   - one entry per (batch, q-head): [B, Hq, Sq, Sk] with non-zero batch and head strides.  Plain stores,
	 *     deterministic; B * Hq * Sq * Sk * 4 bytes.
	 *   - the shape of a broadcast bias: stride 0 on the batch and / or head axis, or Hkv heads with bias_group.
	 *     Entries shared by several (batch, q-head) pairs are accumulated with hardware fp32 atomic adds, so the
	 *     buffer is as small as the bias but the order of the additions - the last bits of the sums - is not fixed
	 *     from run to run, and the adds run at about 0.34 T adds/s.
	 * Positions of key tiles the kernel skips (beyond a length, outside the window or the causal range) are not
	 * touched: pass a zero-filled buffer in both layouts.  The reference returns no gradient for its bias
	 * (_flash_attention.py:88), so this has no counterpart there. */
	float* dbias;
	int64_t dbias_stride_b, dbias_stride_h, dbias_stride_m;
} fa2_params;

/* sizeof(fa2_params) in the first version of this header: up to and including scratch_bytes */
#define FA2_PARAMS_SIZE_V1 ((uint32_t)offsetof(fa2_params, seed_dev))

/* O = softmax(scale q k^T + bias, masked) v, with dropout; writes o and lse.
 * Replaces the `_attn_fwd` custom call (_forward_triton.py:547-588). */
int fa2_fwd(const fa2_params* p, void* hip_stream);

/* Optional scratch for fa2_fwd.  Non-zero for many keys under too few (batch, head, 64-row tile)
 * units to fill the chip - decoding, `Sq == 1` in flash_attention.py:239-242, from 512 keys, and
 * prompts at batch 1 with few heads from 1024 or 2048 keys: given `scratch` (256-byte aligned) of at least this many
 * bytes, fa2_fwd splits the keys into ranges handled by separate workgroups and merges the
 * partial results (same O and lse to rounding).  Without it the call runs unsplit. */
size_t fa2_fwd_scratch_bytes(const fa2_params* p);

/* dq, dk, dv from (q, k, v, o, lse, dO).  Replaces the `_attn_bwd_preprocess`
 * and `_attn_bwd` custom calls and the XLA reduce over the KV group
 * (_backward_triton.py:1049-1161). */
int fa2_bwd(const fa2_params* p, void* hip_stream);

/* fa2_bwd restricted to some of its kernels, for per-kernel timing:
 * bit 0 = delta pre-pass (`_attn_bwd_preprocess`, _backward_triton.py:79-147),
 * bit 1 = dK/dV kernel (`_attn_bwd_block_dkdv`, :257-435),
 * bit 2 = dQ kernel (`_attn_bwd_block_dq`, :519-709).  fa2_bwd == stages 7.
 * Bits 0 and 2 together (5, 7): the pre-pass is not launched on its own; the dQ
 * kernel forms delta from the O and dO rows it holds, leaves it in scratch and
 * runs before the dK/dV kernel - so stages 5 followed by stages 2 are exactly
 * the two launches of fa2_bwd.  Bit 0 alone launches the stand-alone pre-pass;
 * bit 1 or bit 2 without bit 0 read the delta an earlier call left in scratch. */
int fa2_bwd_stages(const fa2_params* p, void* hip_stream, int stages);

/* Bytes of scratch fa2_bwd needs for these dimensions (0 on invalid params). */
size_t fa2_bwd_scratch_bytes(const fa2_params* p);

/* Optional larger scratch for fa2_bwd / fa2_bwd_stages.  Non-zero when the dK/dV kernel's grid
 * (B * Hkv * ceil(Sk / 128) workgroups) would leave at least half of the chip idle, or - causal,
 * fewer than 512 workgroups of long key tiles - would leave it waiting for the longest: given
 * `scratch` of at least this many bytes (it includes fa2_bwd_scratch_bytes), the work of a key
 * tile - the q-heads of its KV group times the query tiles - is split over up to 8 workgroups
 * that leave fp32 partial dK / dV behind delta, and a third kernel sums them in a fixed order
 * (results stay deterministic).  With less scratch the backward runs unsplit.  The reference
 * has no counterpart: it sums dK / dV over the q-heads on the host side of its launcher
 * (_backward_triton.py:1156-1161).  0 when no split applies. */
size_t fa2_bwd_split_scratch_bytes(const fa2_params* p);

/* fa2_bwd for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  p->scratch / p->scratch_bytes are ignored: the
 * scratch (delta, [B, Hq, Sq] fp32) lives in a buffer of FA2_STATIC_SCRATCH_BYTES
 * built into the library, one copy per GPU, held until the process ends.  Calls
 * whose fa2_bwd_scratch_bytes() exceeds that limit (B * Hq * Sq > 4 Mi rows) fail
 * with FA2_ESCRATCH_STATIC and launch nothing.  The call itself allocates and
 * frees nothing and launches the same two kernels as fa2_bwd.  All calls on one
 * GPU share the buffer: two calls that overlap in time on the same GPU (different
 * streams or threads) race on it - order them.  The first call on each GPU looks
 * up the buffer's device address; make that call outside graph capture. */
#define FA2_STATIC_SCRATCH_BYTES (16u << 20)
int fa2_bwd_static(const fa2_params* p, void* hip_stream);

/* keep[b,h,i,j] (uint8, contiguous [B,Hq,Sq,Sk]) of the dropout mask the
 * kernels apply for (seed, p_drop); for validation against the Philox
 * definition: Philox-4x32-10 with key (seed low word, seed high word), one call per
 * two adjacent rows x four adjacent keys with counter (j >> 2, i >> 1, h, b); its four
 * words are eight 16-bit values (word w: value 2w in the low half, 2w + 1 in the high
 * half), element (i, j) owns value 4 (i & 1) + (j & 3) and is kept iff
 * value >= floor(p_drop * 65536).  Counterpart of `tl.rand(seed, offs) > p`
 * (_forward_triton.py:140-143). Uses B, Hq, Sq, Sk, p_drop, seed / seed_dev only. */
int fa2_dropout_mask(const fa2_params* p, uint8_t* keep, void* hip_stream);

/* Validate params exactly as fa2_fwd / fa2_bwd would, without launching
 * (host-only; usable without a GPU).  which: 0 = forward, 1 = backward. */
int fa2_validate(const fa2_params* p, int which);

const char* fa2_strerror(int code);
int fa2_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FA2_H_ */
