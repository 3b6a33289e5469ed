// C ABI of libfa2_hip.so: argument validation and kernel dispatch.
// Declarations and the reference call sites they replace: include/fa2.h.
#include "../../include/fa2.h"

#include <math.h>
#include <string.h>

#include <mutex>

#include "fa2_kernels.hpp"

// Scratch of fa2_bwd_static(): one copy per GPU the library runs on, held until the process
// ends.  In host code this name is only a handle for hipGetSymbolAddress(), never an address.
static __device__ __align__(256) unsigned char scratch[FA2_STATIC_SCRATCH_BYTES];

namespace {

using fa2::KArgs;
using fa2::KTensor;

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// Parameter blocks of earlier versions of the header are shorter (struct_size says which): they are
// completed with zeros.  Returns NULL for a NULL block or one shorter than the first version.
const fa2_params* complete(const fa2_params* p, fa2_params& local) {
	if (!p || p->struct_size < FA2_PARAMS_SIZE_V1) return nullptr;
	if (p->struct_size >= sizeof(fa2_params)) return p;
	memset(&local, 0, sizeof(local));
	memcpy(&local, p, p->struct_size);
	local.struct_size = sizeof(fa2_params);
	return &local;
}

int check_tensor(const fa2_tensor& t, bool required) {
	if (!t.ptr) return required ? FA2_EINVAL_PTR : FA2_OK;
	if (!aligned16(t.ptr)) return FA2_EINVAL_PTR;
	// 16-byte vector access along D needs every row start 16-byte aligned
	if (t.stride_b % 8 || t.stride_s % 8 || t.stride_h % 8) return FA2_EINVAL_STRIDE;
	// the tile copies address the rows of a tile (up to 128) with 32-bit byte offsets
	if (t.stride_s < 0 || t.stride_s > (int64_t)0x7fffffff / (2 * 128)) return FA2_EINVAL_STRIDE;
	return FA2_OK;
}

int esize(int dtype) { return dtype == FA2_FP32 ? 4 : dtype == FA2_MASK_U8 ? 1 : 2; }

KTensor conv(const fa2_tensor& t) {
	KTensor k;
	k.ptr = (char*)t.ptr;
	k.sb = t.stride_b * 2;
	k.ss = t.stride_s * 2;
	k.sh = t.stride_h * 2;
	return k;
}

// delta [B, Hq, Sq] fp32, rounded up to 256 bytes (p: a completed block)
size_t bwd_scratch_bytes(const fa2_params* p) {
	if (p->B <= 0 || p->Hq <= 0 || p->Sq <= 0) return 0;
	size_t n = (size_t)p->B * (size_t)p->Hq * (size_t)p->Sq * sizeof(float);
	return (n + 255) & ~(size_t)255;
}

// own_scratch: the backward brings its scratch itself (fa2_bwd_static), p->scratch is not looked at
int validate(const fa2_params* p, int which, bool own_scratch = false) {
	if (!p) return FA2_EINVAL_STRUCT;
	if (p->seed_dev && ((uintptr_t)p->seed_dev & 7)) return FA2_EINVAL_PTR;
	if (p->dtype != FA2_FP16 && p->dtype != FA2_BF16) return FA2_EINVAL_DTYPE;
	if (p->B <= 0 || p->Sq <= 0 || p->Sk <= 0 || p->Hq <= 0 || p->Hkv <= 0 || p->D <= 0) return FA2_EINVAL_SHAPE;
	if (p->Hq % p->Hkv) return FA2_EINVAL_HEADS;
	if (p->D != 64 && p->D != 128 && p->D != 256) return FA2_EUNSUPPORTED;
	if (!(p->p_drop >= 0.f && p->p_drop < 1.f)) return FA2_EINVAL_DROPOUT;
	if (!isfinite(p->scale) || !(p->scale > 0.f)) return FA2_EINVAL_SHAPE;
	if (!isfinite(p->softcap) || p->softcap < 0.f) return FA2_EINVAL_SHAPE;
	int rc;
	if ((rc = check_tensor(p->q, true))) return rc;
	if ((rc = check_tensor(p->k, true))) return rc;
	if ((rc = check_tensor(p->v, true))) return rc;
	if ((rc = check_tensor(p->o, true))) return rc;
	if (!p->lse || ((uintptr_t)p->lse & 3)) return FA2_EINVAL_PTR;
	if (p->bias) {
		if (p->bias_dtype != FA2_FP16 && p->bias_dtype != FA2_BF16 && p->bias_dtype != FA2_FP32 && p->bias_dtype != FA2_MASK_U8)
			return FA2_EINVAL_BIAS;
		if (((uintptr_t)p->bias % esize(p->bias_dtype)) != 0) return FA2_EINVAL_BIAS;
		if (p->bias_stride_b < 0 || p->bias_stride_h < 0 || p->bias_stride_m < p->Sk) return FA2_EINVAL_BIAS;
	}
	if (p->seqlens) {
		if (p->bias || p->Sq != p->Sk) return FA2_EINVAL_MASK;
		if ((uintptr_t)p->seqlens & 3) return FA2_EINVAL_PTR;
	}
	if (p->kv_lens && ((uintptr_t)p->kv_lens & 3)) return FA2_EINVAL_PTR;
	if (which == 1) {
		if ((rc = check_tensor(p->dout, true))) return rc;
		if ((rc = check_tensor(p->dq, true))) return rc;
		if ((rc = check_tensor(p->dk, true))) return rc;
		if ((rc = check_tensor(p->dv, true))) return rc;
		if (p->dbias) {
			if (!p->bias && !(p->softcap > 0.f)) return FA2_EINVAL_BIAS;
			if (!aligned16(p->dbias)) return FA2_EINVAL_BIAS;
			if (p->dbias_stride_b < 0 || p->dbias_stride_h < 0 || p->dbias_stride_m < p->Sk) return FA2_EINVAL_BIAS;
			if (p->dbias_stride_b % 4 || p->dbias_stride_h % 4 || p->dbias_stride_m % 4) return FA2_EINVAL_BIAS;
		}
		size_t need = bwd_scratch_bytes(p);
		if (own_scratch) {
			if (need > FA2_STATIC_SCRATCH_BYTES) return FA2_ESCRATCH_STATIC;
		} else if (!p->scratch || ((uintptr_t)p->scratch & 255) || p->scratch_bytes < need) {
			return FA2_ESCRATCH;
		}
	}
	return FA2_OK;
}

// an element is kept iff its 16-bit value is >= this
uint32_t drop_threshold(float p) {
	double t = floor((double)p * 65536.0);
	return t >= 65535.0 ? 0xFFFFu : (uint32_t)t;
}

void fill(const fa2_params* p, KArgs& a) {
	memset(&a, 0, sizeof(a));
	a.q = conv(p->q);
	a.k = conv(p->k);
	a.v = conv(p->v);
	a.o = conv(p->o);
	a.lse = p->lse;
	a.bias = (const char*)p->bias;
	if (p->bias) {
		int es = esize(p->bias_dtype);
		a.bias_sb = p->bias_stride_b * es;
		a.bias_sh = p->bias_stride_h * es;
		a.bias_sm = p->bias_stride_m * es;
		a.bias_dtype = p->bias_dtype;
		a.bias_group = p->bias_group ? 1 : 0;
		int valign = es == 4 ? 16 : es == 2 ? 8 : 4;
		// a masked position of a boolean mask adds the lowest finite value of the element type, which is what
		// where(mask, 0, finfo(dtype).min) passed as a bias would add
		a.mask_fill = p->dtype == FA2_BF16 ? -3.38953139e38f : -65504.f;
		a.bias_vec4 = (((uintptr_t)p->bias % valign) == 0 && a.bias_sb % valign == 0 && a.bias_sh % valign == 0 &&
		               a.bias_sm % valign == 0)
		                  ? 1
		                  : 0;
		// tiles of bias can be copied to LDS like K / V tiles: element type of q, 16-byte aligned
		// rows of whole 16-byte pieces (8 keys), row stride within the 32-bit offsets of the tile copies
		a.bias_lds = (p->bias_dtype == p->dtype && ((uintptr_t)p->bias % 16) == 0 && a.bias_sb % 16 == 0 && a.bias_sh % 16 == 0 &&
		              a.bias_sm % 16 == 0 && a.bias_sm >= 0 && a.bias_sm <= 0x7fffffff / 256 && p->Sk % 8 == 0)
		                 ? 1
		                 : 0;
	}
	a.seqlens = p->seqlens;
	a.kv_lens = p->kv_lens;
	a.B = p->B;
	a.Sq = p->Sq;
	a.Sk = p->Sk;
	a.Hq = p->Hq;
	a.Hkv = p->Hkv;
	a.causal = p->causal ? 1 : 0;
	// causal caps the right bound at 0, as the reference does (refrence_call.py:36-37)
	a.win_left = p->has_window && p->window_left >= 0 ? p->window_left : -1;
	a.win_right = p->causal ? 0 : (p->has_window && p->window_right >= 0 ? p->window_right : -1);
	a.scale = p->scale;
	a.softcap = p->softcap;
	a.cap_k1 = p->softcap > 0.f ? p->scale / p->softcap : 0.f;
	a.drop_k0 = (uint32_t)(p->seed & 0xFFFFFFFFull);
	a.drop_k1 = (uint32_t)(p->seed >> 32);
	a.seed_dev = (const uint32_t*)p->seed_dev;  // little-endian: low word first
	a.drop_thr = drop_threshold(p->p_drop);
	// kept values are scaled by the reciprocal of the probability the 16-bit threshold really gives,
	// (65536 - thr) / 65536, so that the expectation of the output is exact for every p
	a.drop_inv_keep = 65536.0f / (float)(65536u - a.drop_thr);
}

}  // namespace

namespace fa2 {

hipError_t launch_fwd(int dtype, int D, bool bias, bool drop, KArgs& a, hipStream_t s) {
	if (dtype == FA2_BF16) {
		if (D == 64) return launch_fwd_bf16_64(bias, drop, a, s);
		if (D == 128) return launch_fwd_bf16_128(bias, drop, a, s);
		return launch_fwd_bf16_256(bias, drop, a, s);
	}
	if (D == 64) return launch_fwd_fp16_64(bias, drop, a, s);
	if (D == 128) return launch_fwd_fp16_128(bias, drop, a, s);
	return launch_fwd_fp16_256(bias, drop, a, s);
}

hipError_t launch_bwd(int dtype, int D, bool bias, bool drop, KArgs& a, hipStream_t s) {
	if (dtype == FA2_BF16) {
		if (D == 64) return launch_bwd_bf16_64(bias, drop, a, s);
		if (D == 128) return launch_bwd_bf16_128(bias, drop, a, s);
		return launch_bwd_bf16_256(bias, drop, a, s);
	}
	if (D == 64) return launch_bwd_fp16_64(bias, drop, a, s);
	if (D == 128) return launch_bwd_fp16_128(bias, drop, a, s);
	return launch_bwd_fp16_256(bias, drop, a, s);
}

}  // namespace fa2

extern "C" {

int fa2_validate(const fa2_params* p, int which) {
	fa2_params lp;
	return validate(complete(p, lp), which ? 1 : 0);
}

size_t fa2_bwd_scratch_bytes(const fa2_params* p) {
	fa2_params lp;
	p = complete(p, lp);
	return p ? bwd_scratch_bytes(p) : 0;
}

// dK/dV on a small grid: B * Hkv * ceil(Sk / 128) workgroups that leave at least half of the chip idle - the steps a
// key tile streams (the q-heads of its KV group x the query tiles) are then split over up to 8 workgroups whose fp32
// partial dK / dV a reduce kernel sums.  Returns the number of parts (1 = no split).
static int bwd_step_split(const fa2_params* p) {
	if (p->Hkv <= 0 || p->Hq % p->Hkv) return 1;
	long wgs = (long)p->B * p->Hkv * ((p->Sk + 127) / 128);
	long steps = (long)(p->Hq / p->Hkv) * ((p->Sq + 127) / 128);  // of the longest key tile, in units of 128 rows
	long parts = wgs > 0 ? 256 / wgs : 1;  // fill the chip
	if (p->causal && wgs < 512) {
		// Causal key tiles differ in length (the first has all the steps, the last one row block's), and with one
		// workgroup per CU the longest sets the time.  Measured (D = 128, dK/dV kernel): up to 128 workgroups do best in
		// 8 parts, one per XCD, down to 16 steps a part (B4 Hq32 Hkv1 S4096 3.00 ms unsplit, 1.58 in 2, 1.07 in 8;
		// B2 Hq8 Hkv2 S4096 0.209 ms in 2, 0.172 in 8); above that about 1024 workgroups of at least 64 steps - up to
		// 256 workgroups at least 2 parts (B4 Hq32 Hkv2 S4096 1.56 ms unsplit, 1.06 in 2 or 4; B1 Hq32 Hkv8 S4096 0.39 /
		// 0.27 in 2 / 0.29 in 4; B1 H8 S4096, 32 steps, 0.103 / 0.090 in 2; B3 Hq32 Hkv4, 384 workgroups, 1.53 / 1.05
		// in 2 / 0.98 in 3; B1 H8 S6144, 384 of 48 steps, 0.163 / 0.185 in 2); from 512 on the launch order packs them
		// unsplit.
		long bal;
		if (wgs <= 128) {
			bal = steps / 16;
		} else if (wgs <= 256) {
			bal = steps / 64 > 2 ? steps / 64 : 2;
			if (bal > 4) bal = 4;
			if (bal > steps / 16) bal = steps / 16;
		} else {
			bal = (1024 + wgs / 2) / wgs;
			if (bal > steps / 64) bal = steps / 64;
		}
		if (bal > 8) bal = 8;
		if (bal > parts) parts = bal;
	}
	if (parts > 8) parts = 8;
	// (the partial sums and their reduction have a fixed cost - about 5 us: measured, a key tile of fewer than 8 such steps
	// is faster unsplit, and a part should have at least two)
	if (steps < 8) return 1;
	if (parts > steps / 2) parts = steps / 2;
	return parts >= 2 ? (int)parts : 1;
}

static size_t bwd_split_part_bytes(const fa2_params* p, int hs) {
	return (size_t)hs * (size_t)p->B * (size_t)p->Hkv * (size_t)p->Sk * 2 * (size_t)p->D * sizeof(float);
}

size_t fa2_bwd_split_scratch_bytes(const fa2_params* p) {
	fa2_params lp;
	p = complete(p, lp);
	if (!p) return 0;
	size_t base = bwd_scratch_bytes(p);
	if (!base || p->Sk <= 0 || p->D <= 0) return 0;
	int hs = bwd_step_split(p);
	return hs > 1 ? base + bwd_split_part_bytes(p, hs) : 0;
}

// Key ranges for a split forward: few query rows (one row tile of 64), too few (batch, head)
// pairs to fill the chip, many keys.  Returns the number of ranges (1 = no split).
// the rows of all q-heads of a kv-head fit one row tile: they share one workgroup (and one pass over K, V)
static bool fwd_pack_gqa(const fa2_params* p) {
	return p->Hkv > 0 && p->Hq % p->Hkv == 0 && p->Hq > p->Hkv && (long)(p->Hq / p->Hkv) * p->Sq <= 64;
}

static int fwd_split_plan(const fa2_params* p, int* split_len) {
	*split_len = 0;
	// workgroups of an unsplit launch of this kernel variant (row tiles of 64)
	long base = fwd_pack_gqa(p) ? (long)p->B * p->Hkv : (long)p->B * p->Hq * ((p->Sq + 63) / 64);
	int tiles = (p->Sk + 63) / 64;
	// A query longer than one row tile runs unsplit on the 128-row kernel, which a quarter of the chip's worth of
	// units already keeps busy over a short key range: the second launch pays from 16 key tiles on up to 128 units
	// and from 32 above (measured at D=64: 256 units over 16 tiles 0.0185 ms unsplit, 0.0203 ms split; over 32 tiles
	// 0.0316 and 0.0235).
	int min_tiles = p->Sq <= 64 ? 8 : (base <= 128 ? 16 : 32);
	if (base >= 512 || tiles < min_tiles) return 1;
	long want = (1024 + base - 1) / base;
	if (want > tiles / 4) want = tiles / 4;
	if (want > 64) want = 64;
	if (want < 2) return 1;
	int per = (int)((tiles + want - 1) / want);
	*split_len = per * 64;
	return (tiles + per - 1) / per;
}

// p: a completed block.  The split forward knows no window and no soft-capping: such calls run unsplit and
// need no scratch (the same predicate decides the launch in fa2_fwd).
static size_t fwd_scratch_bytes(const fa2_params* p) {
	if (p->B <= 0 || p->Hq <= 0 || p->Sq <= 0 || p->Sk <= 0 || p->D <= 0) return 0;
	if (p->has_window || p->softcap > 0.f) return 0;
	int len;
	int n = fwd_split_plan(p, &len);
	if (n <= 1) return 0;
	size_t rows = (size_t)n * (size_t)p->B * (size_t)p->Hq * (size_t)p->Sq;
	return (rows * ((size_t)p->D + 1) * sizeof(float) + 255) & ~(size_t)255;
}

size_t fa2_fwd_scratch_bytes(const fa2_params* p) {
	fa2_params lp;
	p = complete(p, lp);
	return p ? fwd_scratch_bytes(p) : 0;
}

int fa2_fwd(const fa2_params* p, void* hip_stream) {
	fa2_params lp;
	p = complete(p, lp);
	int rc = validate(p, 0);
	if (rc) return rc;
	KArgs a;
	fill(p, a);
	// optional scratch: with enough of it a short query over many keys runs split over key ranges
	size_t need = fwd_scratch_bytes(p);
	if (need && p->scratch && ((uintptr_t)p->scratch & 255) == 0 && p->scratch_bytes >= need) {
		a.nsplit = fwd_split_plan(p, &a.split_len);
		a.pack_gqa = fwd_pack_gqa(p) ? 1 : 0;
		size_t rows = (size_t)a.nsplit * (size_t)p->B * (size_t)p->Hq * (size_t)p->Sq;
		a.o_part = (float*)p->scratch;
		a.lse_part = a.o_part + rows * (size_t)p->D;
	}
	hipError_t e = fa2::launch_fwd(p->dtype, p->D, p->bias != nullptr || p->softcap > 0.f, p->p_drop > 0.f, a, (hipStream_t)hip_stream);
	return e == hipSuccess ? FA2_OK : FA2_EHIP;
}

int fa2_bwd(const fa2_params* p, void* hip_stream) { return fa2_bwd_stages(p, hip_stream, 7); }

static int bwd_launch(const fa2_params* p, void* hip_stream, int stages, void* scratch_ptr, size_t scratch_bytes) {
	KArgs a;
	fill(p, a);
	a.stages = stages & 7;
	// optional: with enough scratch behind delta the dK/dV kernel of a small grid runs split over the q-heads of a group
	a.kv_hsplit = 1;
	a.dkv_part = nullptr;
	{
		int hs = bwd_step_split(p);
		size_t base = bwd_scratch_bytes(p);
		if (hs > 1 && scratch_bytes >= base + bwd_split_part_bytes(p, hs)) {
			a.kv_hsplit = hs;
			a.dkv_part = (float*)((char*)scratch_ptr + base);
		}
	}
	a.dout = conv(p->dout);
	a.dq = conv(p->dq);
	a.dk = conv(p->dk);
	a.dv = conv(p->dv);
	a.delta = (float*)scratch_ptr;
	a.dbias = (char*)p->dbias;
	a.dbias_sb = p->dbias_stride_b * 4;
	a.dbias_sh = p->dbias_stride_h * 4;
	a.dbias_sm = p->dbias_stride_m * 4;
	a.dbias_atomic = p->dbias && ((p->dbias_stride_b == 0 && p->B > 1) || (p->dbias_stride_h == 0 && p->Hq > 1) ||
	                              (p->bias_group && p->Hq > p->Hkv))
	                     ? 1
	                     : 0;
	hipError_t e = fa2::launch_bwd(p->dtype, p->D, p->bias != nullptr || p->softcap > 0.f, p->p_drop > 0.f, a, (hipStream_t)hip_stream);
	return e == hipSuccess ? FA2_OK : FA2_EHIP;
}

int fa2_bwd_stages(const fa2_params* p, void* hip_stream, int stages) {
	fa2_params lp;
	p = complete(p, lp);
	int rc = validate(p, 1);
	if (rc) return rc;
	return bwd_launch(p, hip_stream, stages, p->scratch, (size_t)p->scratch_bytes);
}

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch_ptr(void** out) {
	constexpr int kMaxDevices = 64;
	static void* ptrs[kMaxDevices];
	static std::mutex mu;
	int dev = -1;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FA2_EHIP;
	std::lock_guard<std::mutex> lock(mu);
	if (!ptrs[dev]) {
		void* ptr = nullptr;
		if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return FA2_EHIP;
		ptrs[dev] = ptr;
	}
	*out = ptrs[dev];
	return FA2_OK;
}

int fa2_bwd_static(const fa2_params* p, void* hip_stream) {
	fa2_params lp;
	p = complete(p, lp);
	int rc = validate(p, 1, /*own_scratch=*/true);
	if (rc) return rc;
	void* ptr = nullptr;
	if ((rc = static_scratch_ptr(&ptr))) return rc;
	// delta is written in full by the first kernel before the second reads it: nothing to clear
	return bwd_launch(p, hip_stream, 7, ptr, (size_t)FA2_STATIC_SCRATCH_BYTES);
}

int fa2_dropout_mask(const fa2_params* p, uint8_t* keep, void* hip_stream) {
	fa2_params lp;
	p = complete(p, lp);
	if (!p) return FA2_EINVAL_STRUCT;
	if (p->seed_dev && ((uintptr_t)p->seed_dev & 7)) return FA2_EINVAL_PTR;
	if (p->B <= 0 || p->Sq <= 0 || p->Sk <= 0 || p->Hq <= 0) return FA2_EINVAL_SHAPE;
	if (!(p->p_drop >= 0.f && p->p_drop < 1.f)) return FA2_EINVAL_DROPOUT;
	if (!keep) return FA2_EINVAL_PTR;
	hipError_t e = fa2::launch_dropout_mask(keep, p->B, p->Hq, p->Sq, p->Sk, (uint32_t)(p->seed & 0xFFFFFFFFull),
	                                        (uint32_t)(p->seed >> 32), drop_threshold(p->p_drop), (const uint32_t*)p->seed_dev,
	                                        (hipStream_t)hip_stream);
	return e == hipSuccess ? FA2_OK : FA2_EHIP;
}

const char* fa2_strerror(int code) {
	switch (code) {
		case FA2_OK: return "ok";
		case FA2_EINVAL_STRUCT: return "params is NULL or struct_size is smaller than the first version of fa2_params";
		case FA2_EINVAL_DTYPE: return "Only support fp16 and bf16";
		case FA2_EINVAL_SHAPE: return "dimensions must be positive and the softmax scale finite and positive";
		case FA2_EINVAL_HEADS: return "query heads must be divisible by key/value heads";
		case FA2_EINVAL_PTR: return "required pointer is NULL or misaligned";
		case FA2_EINVAL_STRIDE: return "strides must be multiples of 8 elements and the sequence stride in [0, 2^31 / 256] elements";
		case FA2_EINVAL_DROPOUT: return "dropout probability must be in [0, 1)";
		case FA2_EINVAL_BIAS: return "bias dtype or strides invalid";
		case FA2_EINVAL_MASK: return "Attention mask is not supported along with attention bias or with QSeq != KSeq";
		case FA2_EUNSUPPORTED: return "head dim must be 64, 128 or 256";
		case FA2_ESCRATCH: return "backward scratch buffer missing, misaligned or too small";
		case FA2_EHIP: return "HIP launch failed";
		case FA2_ESCRATCH_STATIC: return "fa2_bwd_static: B * Hq * Sq * 4 bytes exceed the 16 MiB built-in scratch";
		default: return "unknown error";
	}
}

int fa2_version(void) { return 100; }

}  // extern "C"
