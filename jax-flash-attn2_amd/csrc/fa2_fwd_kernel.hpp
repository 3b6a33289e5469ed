// Forward kernel: O = softmax(scale Q K^T + bias, masked) V, plus the row
// logsumexp.  Takes the place of `_attn_fwd` / `_attn_fwd_inner`
// (jax_flash_attn2/flash_attention_triton/_forward_triton.py:60-164, 213-459).
//
// One workgroup = NW waves = one tile of BM = NW*QB*32 query rows of one
// (batch, q-head).  K/V tiles of BN = 64 keys are streamed through a double
// buffer in LDS by direct global->LDS loads.  Everything is computed
// transposed so that no intermediate ever leaves registers:
//   S^T[kv, q] = K[kv, :] . Q[q, :]      A = K fragment from LDS, B = Q in registers
//   O^T[d,  q] = V^T[d, kv] . P^T[kv, q] A = V through transposed LDS reads,
//                                        B = P^T = the S^T accumulator, packed to 16 bits
// In both accumulators a lane owns ONE query row (column l%32), so the online
// softmax needs only in-lane reductions plus one exchange with lane l^32, and
// rescaling O is a multiply by a per-lane scalar.
#pragma once
#include <type_traits>

#include "fa2_common.hpp"
#include "fa2_kernels.hpp"

namespace fa2 {

// experiment switch: wave priority raised around the clusters of matrix products (0 = off)
#ifndef FA2_SETPRIO
#define FA2_SETPRIO 0
#endif

constexpr int kFwdBN = 64;
// with bias: the running row maximum is only raised when exceeded by more than this (log2 units)
constexpr float kRescaleSlack = 8.f;
// without bias: largest partial row sum of one tile of P = exp2(c1 S - c1 m) taken without looking at
// the row maximum (fp16 holds values up to 65504)
constexpr float kFastSum = 16384.f;
constexpr int kNumCU = 256;  // compute units of the MI355X (tile-size choice for small grids)

// blockIdx.x -> (row tile, q-head, batch).  With xcd_remap the workgroups of
// one (batch, kv-head) - which share K and V - are kept on one XCD (hardware
// deals consecutive workgroup ids round-robin over the 8 XCDs), so K/V are
// fetched from HBM once per XCD L2 instead of once per L2 of every XCD.
// Row tiles are visited last-first: under a causal mask the last tiles are
// the longest, and starting them first shortens the tail of the launch.
// The hardware hands the workgroups of an XCD to its four shader engines in strict rotation and waits for a free CU
// on the engine whose turn it is: when adjacent workgroups differ in length, CUs of the other engines stand idle
// meanwhile (measured on causal multi-head attention with one q-head per kv-head: 15 us on average between two
// workgroups of a CU, a quarter of the launch).  Under a causal mask or a window the work of a tile depends on its
// index, so the launch order makes every aligned run of four workgroups of an XCD the same tile index: of the
// `heads` equal-length items a group has per tile (r q-heads for the forward and dQ kernels, 1 for dK/dV) and, where
// those are fewer than four, of `e` groups that advance together.  Returns e (1, 2 or 4); per_xcd = groups per XCD.
// Groups that advance together also stream their operands together (K and V in the forward and dQ kernels, Q and dO
// of the group's q-heads in dK/dV: stream_bytes per group): e is kept small enough for these to stay within reach of
// the XCD's 4 MiB L2 - with four groups of 8 MiB each the dK/dV kernel fetched twice as much from memory for no gain.
inline int launch_order(const KArgs& a, int heads, int per_xcd, int64_t stream_bytes) {
	if (a.win_right < 0 && a.win_left < 0) return 1;  // every tile sees all keys: equal lengths anyway
	int e = heads % 4 == 0 ? 1 : (heads % 2 == 0 ? 2 : 4);
	while (e > 1 && (per_xcd % e || e * stream_bytes > (8 << 20))) e >>= 1;
	return e;
}

// Workgroup ids of the first half of a causal grid that runs two 4-wave workgroups per CU (see decode_block), else 0.
// two_per_cu: the kernel variant leaves room for two workgroups on a CU (registers, LDS).  Measured with and without,
// B2 Hq8 Hkv2 S4096 D128 forward 0.086 / 0.109 ms (unfolded, the two batch rows put their long tiles on the same CUs),
// a single group B1 Hq8 S8192 0.163 / 0.168 ms.
inline int fold_half_of(const KArgs& a, int nw, int64_t total, bool two_per_cu) {
	if (!two_per_cu || nw != 4 || !a.causal || a.win_left >= 0 || a.xcd_remap > 1) return 0;
	if (total <= kNumCU || total > 2 * kNumCU || total % 16) return 0;
	return (int)(total / 2);
}

FA2_DEV void decode_block(const KArgs& a, int& mt, int& h, int& b, int id = (int)blockIdx.x) {
	if (a.fold_half && id >= a.fold_half) {
		// A causal grid of two workgroups per CU, all resident at once: the first half of the workgroup ids takes the
		// first place of every CU, the second half the second place in the same order of CUs.  The first half runs
		// from the longest tile down; the second half is visited backwards, so that the CU with the longest tile of
		// the first half gets the shortest of the second (on every XCD for itself when groups are placed by XCD).
		if (a.xcd_remap)
			id = (((a.fold_half >> 3) + ((a.fold_half >> 2) - 1 - (id >> 3))) << 3) | (id & 7);
		else
			id = a.fold_half + (2 * a.fold_half - 1 - id);
	}
	if (a.xcd_remap == 2) {
		// A bias without a head axis is re-read by every head: one batch per XCD, and on an
		// XCD the heads of one row tile next to each other, so that the tile of bias they all
		// read is fetched into that XCD's L2 once.
		int xcd = id & 7, j = id >> 3;
		int per_batch = a.mtiles * a.Hq;
		b = (j / per_batch) * 8 + xcd;
		int rem = j % per_batch;
		mt = a.mtiles - 1 - rem / a.Hq;
		h = rem % a.Hq;
		return;
	}
	if (a.xcd_remap == 3) {
		// The same sharing of a head-less bias, for batch rows of different key lengths: the unit (batch, row tile)
		// with its heads adjacent stays on one XCD, but the units of one batch go round the XCDs (batch b, tile t
		// on XCD (b + t) % 8), so that a short batch row does not leave its XCD idle.
		int xcd = id & 7, j = id >> 3;
		int u = j / a.Hq, nb8 = a.B >> 3;
		int tile = u / nb8;
		h = j % a.Hq;
		mt = a.mtiles - 1 - tile;
		b = ((xcd - tile) & 7) + 8 * (u % nb8);
		return;
	}
	int r = a.Hq / a.Hkv;
	int per_group = a.mtiles * r;
	int grp, within;
	if (a.xcd_remap) {
		int xcd = id & 7, j = id >> 3;
		// a.interleave = e groups of an XCD advance together: e r adjacent workgroups are the same row tile (see launch_order())
		int e = a.interleave;
		int sgi = j / (e * per_group), rem = j % (e * per_group);
		int t = rem / (e * r), rem2 = rem % (e * r);
		grp = (sgi * e + rem2 / r) * 8 + xcd;
		within = t * r + rem2 % r;
	} else {
		grp = id / per_group;
		within = id % per_group;
	}
	int hk = grp % a.Hkv;
	b = grp / a.Hkv;
	mt = a.mtiles - 1 - within / r;
	h = hk * r + within % r;
}

// four consecutive bias values bias[row][col..col+3] as floats.  dtype 4: the row holds bytes of a boolean
// mask; a zero byte stands for the additive value `fill`, anything else for 0.
FA2_DEV f32x4 load_bias4(const char* rowp, int col, int dtype, bool vec_ok, int ncols, float fill) {
	f32x4 out;
	if (vec_ok && col + 3 < ncols) {
		if (dtype == 3) {
			out = *(const f32x4*)(rowp + (int64_t)col * 4);
		} else if (dtype == 2) {
			bf16x4 t = *(const bf16x4*)(rowp + (int64_t)col * 2);
			out = to_f32x4(t);
		} else if (dtype == 1) {
			f16x4 t = *(const f16x4*)(rowp + (int64_t)col * 2);
			out = __builtin_convertvector(t, f32x4);
		} else {
			uint32_t t = *(const uint32_t*)(rowp + col);
#pragma unroll
			for (int e = 0; e < 4; ++e) out[e] = ((t >> (8 * e)) & 0xffu) ? 0.f : fill;
		}
	} else {
#pragma unroll
		for (int e = 0; e < 4; ++e) {
			float x = 0.f;
			if (col + e < ncols) {
				if (dtype == 3)
					x = *(const float*)(rowp + (int64_t)(col + e) * 4);
				else if (dtype == 2)
					x = to_f32(*(const __bf16*)(rowp + (int64_t)(col + e) * 2));
				else if (dtype == 1)
					x = (float)*(const _Float16*)(rowp + (int64_t)(col + e) * 2);
				else
					x = *(const uint8_t*)(rowp + col + e) ? 0.f : fill;
			}
			out[e] = x;
		}
	}
	return out;
}

// SPLIT: the keys are cut into a.nsplit ranges of a.split_len keys (a multiple of the tile);
// workgroup (tile, split) handles one range and leaves a normalised partial result (O as
// fp32 and its logsumexp) in scratch for fwd_combine_kernel.  For few query rows and many
// keys (decoding, short cross-attention queries), where one workgroup per row tile would
// leave most of the chip idle.
// BLDS: the bias goes through LDS (the launcher has checked element type, alignment and the key
// count); otherwise every lane loads its bias values from global memory.
// CAP: tanh soft-capping of the scores (refrence_call.py:48-51), on the path with bias; the bias itself may be absent.
template <typename T, int D, int NW, int QB, int WPS, bool BIAS, bool DROP, bool SPLIT = false, bool BLDS = false, bool CAP = false>
__global__ __launch_bounds__(NW * 64, WPS) void fwd_kernel(const KArgs a) {
	static_assert(!CAP || (BIAS && !BLDS && !SPLIT), "soft-capping runs on the plain path with bias");
	typedef typename T::V8 V8;
	constexpr int BM = NW * QB * 32;
	constexpr int BN = kFwdBN;
	constexpr int KB = BN / 32;   // 32-key blocks per tile
	constexpr int KS = D / 16;    // MFMA k-steps along D
	constexpr int DB = D / 32;    // 32-wide blocks of the head dim
	constexpr int NT = NW * 64;
	constexpr int TILE_BYTES = BN * D * 2;

	// Bias tiles (BM rows x 64 keys, element type of q) go through LDS as well when there is
	// room: read from global memory one row per lane, a wave's load touches 32 cache lines.
	constexpr bool BIAS_LDS = BIAS && BLDS && (D <= 128 || !SPLIT);
	constexpr int BIAS_BYTES = BIAS_LDS ? BM * BN * 2 : 0;
	static_assert(BN == 64, "bias tiles use the 64-element row geometry");
	__shared__ __attribute__((aligned(1024))) char smem[4 * TILE_BYTES + 2 * BIAS_BYTES];
	FA2_LDS char* lds = (FA2_LDS char*)smem;
	// layout: K[0] K[1] V[0] V[1] bias[0] bias[1]

	int mt, h, b, split = 0;
	// pack (split kernel only): the rows of the tile are the Sq rows of ALL r q-heads of one
	// kv-head (row = head_in_group * Sq + position), so that K and V are streamed once per
	// group instead of once per q-head; every lane then has its own q-head.
	bool pack = false;
	if constexpr (SPLIT) {
		split = (int)blockIdx.x % a.nsplit;
		pack = a.pack_gqa != 0;
		if (pack) {
			int id2 = (int)blockIdx.x / a.nsplit;
			b = id2 / a.Hkv;
			h = (id2 % a.Hkv) * (a.Hq / a.Hkv);
			mt = 0;
		} else {
			decode_block(a, mt, h, b, (int)blockIdx.x / a.nsplit);
		}
	} else {
		decode_block(a, mt, h, b);
	}
	const int hk = h / (a.Hq / a.Hkv);
	const int tid = threadIdx.x, lane = tid & 63;
	// the wave index as an explicitly scalar value: everything derived from it (tile bounds, loop trip counts,
	// "nothing to do for this wave") then stays in scalar registers and scalar branches
	const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, c = lane & 31;
	// dropout key: from the parameter block, or from device memory when the caller keeps it there
	uint32_t drop_k0 = a.drop_k0, drop_k1 = a.drop_k1;
	if constexpr (DROP) {
		if (a.seed_dev) {
			drop_k0 = a.seed_dev[0];
			drop_k1 = a.seed_dev[1];
		}
	}

	int sq_eff = a.Sq, sk_eff = a.Sk;
	if (a.seqlens) {
		int len = a.seqlens[b];
		len = len < 0 ? 0 : (len > a.Sk ? a.Sk : len);
		sq_eff = len < a.Sq ? len : a.Sq;
		sk_eff = len;
	}
	const int off = sk_eff - sq_eff;  // causal: key j allowed for row i iff j <= i + off
	if (a.kv_lens) {  // key padding only: the causal alignment keeps counting from the full key count
		int len = a.kv_lens[b];
		len = len < 0 ? 0 : len;
		sk_eff = len < sk_eff ? len : sk_eff;
	}
	const int m0 = mt * BM;
	const int wm0 = m0 + w * (QB * 32);

	// Row i may look at keys i + off - win_left .. i + off + win_right (each bound only when >= 0;
	// causal is win_right = 0): the sliding window of refrence_call.py:55-75, bottom-right aligned.
	const int wr = a.win_right, wl = a.win_left;
	constexpr int kNoKey = -(1 << 30);
	// keys this row tile can see (of this workgroup's range of keys)
	int kv_end = sk_eff;
	if (wr >= 0) {
		int last_row = (m0 + BM - 1 < sq_eff - 1) ? m0 + BM - 1 : sq_eff - 1;
		int e = last_row + off + wr + 1;
		kv_end = e < kv_end ? e : kv_end;
	}
	if (m0 >= sq_eff) kv_end = 0;
	int t_begin = 0;
	if constexpr (SPLIT) {
		int kv_begin = split * a.split_len;  // a multiple of BN
		int e = kv_begin + a.split_len;
		kv_end = e < kv_end ? e : kv_end;
		t_begin = kv_begin / BN;
		if (kv_end <= kv_begin) kv_end = 0;
	} else if (wl >= 0) {
		int first_key = m0 + off - wl;  // first key the tile's first row sees
		if (first_key > 0) t_begin = first_key / BN;
	}
	const int ntiles = kv_end > 0 ? (kv_end + BN - 1) / BN : 0;  // one past the last tile

	// per-lane first and last allowed key for each of this lane's rows
	int jmax[QB], jmin[QB];
	int qrow[QB];
	int hl[QB];  // this lane's q-head
#pragma unroll
	for (int qb = 0; qb < QB; ++qb) {
		int i = wm0 + 32 * qb + c;
		hl[qb] = h;
		if (pack) {
			int r = a.Hq / a.Hkv;
			int hh = i / a.Sq;
			i -= hh * a.Sq;
			if (hh >= r) {  // beyond the group's rows: no such row
				hh = r - 1;
				i = a.Sq;
			}
			hl[qb] = h + hh;
		}
		qrow[qb] = i;
		int jm = sk_eff - 1;
		if (wr >= 0) jm = (i + off + wr < jm) ? i + off + wr : jm;
		if (i >= sq_eff) jm = -1;
		jmax[qb] = jm;
		jmin[qb] = wl >= 0 ? i + off - wl : kNoKey;
	}
	// wave-uniform bounds over the wave's rows: wave_jmin / wave_jmax = smallest / largest last key,
	// wave_lmin / wave_lmax = smallest / largest first key
	int wave_jmin, wave_jmax, wave_lmin = kNoKey, wave_lmax = kNoKey;
	{
		int first = wm0, last = wm0 + QB * 32 - 1;
		if (first >= sq_eff) {
			wave_jmin = wave_jmax = -1;
		} else {
			wave_jmax = sk_eff - 1;
			wave_jmin = sk_eff - 1;
			int lastv = last < sq_eff - 1 ? last : sq_eff - 1;
			if (wr >= 0) {
				wave_jmax = (lastv + off + wr < wave_jmax) ? lastv + off + wr : wave_jmax;
				wave_jmin = (first + off + wr < wave_jmin) ? first + off + wr : wave_jmin;
			}
			if (wl >= 0) {
				wave_lmin = first + off - wl;
				wave_lmax = lastv + off - wl;
			}
			if (last >= sq_eff) wave_jmin = -1;
		}
		if (pack) {  // rows of several heads: every tile takes the masked path
			wave_jmin = -1;
			wave_jmax = wm0 < (a.Hq / a.Hkv) * a.Sq ? sk_eff - 1 : -1;
		}
	}

	const char* kbase = a.k.ptr + (int64_t)b * a.k.sb + (int64_t)hk * a.k.sh;
	const char* vbase = a.v.ptr + (int64_t)b * a.v.sb + (int64_t)hk * a.v.sh;

	TileLoader<D, BN, NT> kload, vload;
	kload.init(a.k.ss, tid);
	vload.init(a.v.ss, tid);
	// prologue: first K/V tile in flight while Q is fetched
	if (ntiles > t_begin) {
		int nb = t_begin * BN, bsel = t_begin & 1;
		int rows = sk_eff - nb < BN ? sk_eff - nb : BN;
		kload.load(lds + bsel * TILE_BYTES, kbase + (int64_t)nb * a.k.ss, a.k.ss, rows, tid);
		vload.load(lds + (2 + bsel) * TILE_BYTES, vbase + (int64_t)nb * a.v.ss, a.v.ss, rows, tid);
	}

	// Q fragments (B operand of S^T): lane holds Q[row c][16ks + 8g .. +7]
	V8 qf[QB][KS];
	{
#pragma unroll
		for (int qb = 0; qb < QB; ++qb) {
			const char* qbase = a.q.ptr + (int64_t)b * a.q.sb + (int64_t)hl[qb] * a.q.sh;
			int i = qrow[qb] < a.Sq ? qrow[qb] : a.Sq - 1;
			const char* rp = qbase + (int64_t)i * a.q.ss + g * 16;
#pragma unroll
			for (int ks = 0; ks < KS; ++ks) qf[qb][ks] = *(const V8*)(rp + ks * 32);
		}
	}

	// Without bias the score only feeds exp2: P = exp2(c1 * q.k - c1 * m) with m the row's running
	// reference in units of the raw dot product.  The factor c1 = scale * log2(e) is applied to the
	// fp32 accumulator, as the reference scales the fp32 result of its dot (_forward_triton.py:281).
	constexpr bool FOLD = !BIAS;
	float nmc[QB];  // -c1 * m of the lane's row (0 while the row has seen no key)
	// The Q fragments must have arrived before the loop over key tiles starts.  Otherwise the
	// compiler places its waits for these loads (s_waitcnt vmcnt) at their first uses inside the
	// loop, where the same counter also counts the tile copies in flight: every such wait would
	// then stall the matrix products until the copies of the NEXT tile have landed.
#pragma unroll
	for (int qb = 0; qb < QB; ++qb)
#pragma unroll
		for (int ks = 0; ks < KS; ++ks) asm volatile("; Q fragment present" : "+v"(qf[qb][ks]));

	f32x16 oacc[QB][DB];
	float mrow[QB], lrow[QB];
#pragma unroll
	for (int qb = 0; qb < QB; ++qb) {
		nmc[qb] = 0.f;
		mrow[qb] = -INFINITY;
		lrow[qb] = 0.f;
#pragma unroll
		for (int db = 0; db < DB; ++db)
#pragma unroll
			for (int i = 0; i < 16; ++i) oacc[qb][db][i] = 0.f;
	}

	const float c1 = BIAS ? a.scale : a.scale * kLog2e;  // score -> softmax domain
	const char* bias_base = nullptr;
	if constexpr (BIAS) {
		int hb = a.bias_group ? hk : h;
		bias_base = a.bias + (int64_t)b * a.bias_sb + (int64_t)hb * a.bias_sh;
	}
	constexpr bool bias_lds = BIAS_LDS;
	TileLoader<64, BM, NT> bload;
	int brows = 0, boff_lane = 0, bkey16 = 0;
	if constexpr (BIAS_LDS) {
		brows = a.Sq - m0 < BM ? a.Sq - m0 : BM;
		bload.init(a.bias_sm, tid, brows);
		// this lane's row of the tile: byte offset of its chunk 0 (+ 8 bytes for the upper half-wave) and swizzle key
		int row = w * (QB * 32) + c;
		boff_lane = row * 128 + 8 * g + (t_begin & 1) * BIAS_BYTES;
		bkey16 = swz<64>(row) << 4;
		if (bias_lds && ntiles > t_begin)
			bload.load(lds + 4 * TILE_BYTES + (t_begin & 1) * BIAS_BYTES, bias_base + (int64_t)m0 * a.bias_sm + (int64_t)t_begin * BN * 2,
			           a.bias_sm, brows, tid, (a.Sk - t_begin * BN) >> 3);
	}

	// Per-lane LDS byte offsets with the swizzle folded in, so that every fragment
	// read in the loop is base + register + immediate.
	//   K fragment (ks):      row c (+32 kb), chunk 2ks+g
	//   V fragment (kk, db):  rows 16kk + 4g + (lane&15)/4 (+8), 8 bytes at column 32db + 16((lane>>4)&1) + 4(lane&3)
	// The offsets carry the buffer (K[1] / V[1] / bias[1] lie a power of two behind K[0] / V[0] / bias[0])
	// and are flipped after every tile, so that the reads need no address arithmetic in the loop.
	const int buf0 = t_begin & 1;
	// (the swizzle touches the low four bits of the chunk index only: chunks 16 and up - head dim 256 - are the same
	// offsets 256 bytes further on, an immediate of the read instead of eight more registers)
	constexpr int KR = KS < 8 ? KS : 8, DR = DB < 4 ? DB : 4;
	int koff[KR];
#pragma unroll
	for (int ks = 0; ks < KR; ++ks) koff[ks] = tile_off<D>(c, 2 * ks + g) + buf0 * TILE_BYTES;
	int voff[DR][2];
	{
		int i16 = lane & 15;
		int vrow = 4 * g + (i16 >> 2);
		int vcol = 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
#pragma unroll
		for (int db = 0; db < DR; ++db) {
			int col = 32 * db + vcol;
			voff[db][0] = tile_off<D>(vrow, col >> 3) + ((col & 4) << 1) + (2 + buf0) * TILE_BYTES;
			voff[db][1] = tile_off<D>(vrow + 8, col >> 3) + ((col & 4) << 1) + (2 + buf0) * TILE_BYTES;
		}
	}

	// One K/V tile.  MASKED = some element of the tile is masked for this wave.
	auto tile_body = [&](auto masked_tag, int n0) {
		constexpr bool MASKED = decltype(masked_tag)::value;
		// bias tile, fetched ahead of the matrix products
		f32x4 bv[BIAS ? KB : 1][BIAS ? QB : 1][4];
		if (BIAS_LDS && bias_lds) {
			static_assert(!BIAS_LDS || QB == 1, "");
#pragma unroll
			for (int kb = 0; kb < KB; ++kb)
#pragma unroll
				for (int aa = 0; aa < 4; ++aa) {
					typename T::V4 x = *(const FA2_LDS typename T::V4*)(lds + 4 * TILE_BYTES + boff_lane + (((kb * 4 + aa) << 4) ^ bkey16));
					bv[kb][0][aa] = to_f32x4(x);
				}
		} else if constexpr (BIAS) {
#pragma unroll
			for (int qb = 0; qb < QB; ++qb) {
				int i = qrow[qb] < a.Sq ? qrow[qb] : a.Sq - 1;
				const char* rowp = bias_base + (int64_t)i * a.bias_sm;
				if (SPLIT && !a.bias_group) rowp += (int64_t)(hl[qb] - h) * a.bias_sh;  // (packed rows: the lane's own head)
#pragma unroll
				for (int kb = 0; kb < KB; ++kb)
#pragma unroll
					for (int aa = 0; aa < 4; ++aa) {
						if (CAP && a.bias == nullptr)
							bv[kb][qb][aa] = f32x4{0.f, 0.f, 0.f, 0.f};
						else
							bv[kb][qb][aa] = load_bias4(rowp, n0 + 32 * kb + 8 * aa + 4 * g, a.bias_dtype, a.bias_vec4, a.Sk, a.mask_fill);
					}
			}
		}

		// S^T = K Q^T
		f32x16 s[KB][QB];
		auto compute_s = [&]() __attribute__((always_inline)) {
#pragma unroll
			for (int kb = 0; kb < KB; ++kb)
#pragma unroll
				for (int qb = 0; qb < QB; ++qb)
#pragma unroll
					for (int i = 0; i < 16; ++i) s[kb][qb][i] = 0.f;
			__builtin_amdgcn_sched_barrier(0);
#pragma unroll
			for (int ks = 0; ks < KS; ++ks)
#pragma unroll
				for (int kb = 0; kb < KB; ++kb) {
					V8 kf = *(const FA2_LDS V8*)(lds + koff[ks % KR] + (ks / KR) * 256 + kb * (32 * D * 2));
#pragma unroll
					for (int qb = 0; qb < QB; ++qb) s[kb][qb] = mfma32(kf, qf[qb][ks], s[kb][qb]);
				}
			// issue order: a few fragment reads ahead, then one read per product, so that the
			// LDS latency is paid once per tile instead of once per product
			{
				constexpr int NR = KS * KB, PF = D == 256 ? 4 : (NR < 8 ? NR : 8);  // (head dim 256: registers are short)
				__builtin_amdgcn_sched_group_barrier(0x100, PF, 0);
#pragma unroll
				for (int i = 0; i < NR - PF; ++i) {
					__builtin_amdgcn_sched_group_barrier(0x008, QB, 0);
					__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
				}
				__builtin_amdgcn_sched_group_barrier(0x008, PF * QB, 0);
			}
			__builtin_amdgcn_sched_barrier(0);
		};

		// V fragments for O^T += V^T P^T, fetched in batches of NF; the first batch is in
		// flight during the softmax, each further one during the products of the previous.
		constexpr int KK = BN / 16;
		constexpr int NFR = KK * DB;                                  // fragments of a tile: 16-key step fi / DB, d-block fi % DB
		constexpr int NF = D == 256 ? 4 : (NFR < 8 ? NFR : 8);        // fragments per batch (head dim 256: registers are short)
		constexpr int NBATCH = NFR / NF;
		u32x4 vfr[2][NF];
		auto issue_v = [&](auto batch_tag, u32x4(&dst)[NF]) {
			constexpr int BI = decltype(batch_tag)::value;
#pragma unroll
			for (int u = 0; u < NF; ++u) {
				const int fi = BI * NF + u, st = fi / DB, db = fi % DB;
				dst[u] = lds_tr_issue_rt<D>(lds + voff[db % DR][0] + (db / DR) * 256, lds + voff[db % DR][1] + (db / DR) * 256, st);
			}
		};

		// online softmax, one query row per lane
		V8 pf[QB][BN / 16];
#if FA2_SETPRIO
		__builtin_amdgcn_s_setprio(FA2_SETPRIO);
#endif
		compute_s();
#if FA2_SETPRIO
		__builtin_amdgcn_s_setprio(0);
#endif
		issue_v(std::integral_constant<int, 0>{}, vfr[0]);
		// packs P (held in s) to the B operand of the second product
		auto pack_p = [&](int qb) __attribute__((always_inline)) {
#pragma unroll
			for (int kb = 0; kb < KB; ++kb)
#pragma unroll
				for (int hf = 0; hf < 2; ++hf) {
					const f32x16& r = s[kb][qb];
					pf[qb][2 * kb + hf] = pack8<T>(r[8 * hf + 0], r[8 * hf + 1], r[8 * hf + 2], r[8 * hf + 3], r[8 * hf + 4],
					                               r[8 * hf + 5], r[8 * hf + 6], r[8 * hf + 7]);
				}
		};
		// Dropout on the packed P (the row sums have been taken before): word m of a packed operand holds the keys
		// 8 (2 hf + m / 2) + 4 g + 2 (m % 2), + 1 of the block - the two values of word m % 2 of the generator's words for that
		// group of four keys.
		// (split forward: the rows of a tile may belong to several heads - no sharing of generator calls between lanes)
		auto drop_p = [&](int qb) __attribute__((always_inline)) {
			if constexpr (DROP) {
				const uint32_t thr2 = a.drop_thr * 0x10001u;
#pragma unroll
				for (int kb = 0; kb < KB; ++kb)
#pragma unroll
					for (int hf = 0; hf < 2; ++hf) {
						uint32_t dw[2][2];
						dropout_words_rowlane_half<!SPLIT>(n0 + 32 * kb + 4 * g, (uint32_t)qrow[qb], (uint32_t)hl[qb], (uint32_t)b, drop_k0, drop_k1, hf, dw);
						u32x4 x = __builtin_bit_cast(u32x4, pf[qb][2 * kb + hf]);
#pragma unroll
						for (int m = 0; m < 4; ++m) x[m] = keep_pair16(x[m], dw[m >> 1][m & 1], thr2);
						pf[qb][2 * kb + hf] = __builtin_bit_cast(V8, x);
					}
			}
		};
		if constexpr (FOLD) {
			// Fast path: P = exp2(c1 S - c1 m) against the reference m the rows
			// already have, packed to 16 bits at once - no row maximum, and the scores stay in their
			// registers.  It stands when every partial row sum of the tile stays below kFastSum (then no
			// P exceeds it either: 16-bit P and the fp32 sums hold that without loss) and no row meets
			// its first keys in this tile.  Otherwise (decided for the wave as a whole) the tile takes
			// the path with the row maximum, from the scores that are still there.
			constexpr bool FAST = true;
			float lt[QB];
			bool slow = true;
			if constexpr (FAST) {
				// (a row that meets its first keys here has no reference yet: what the fast path makes of it is discarded)
				bool over = false;
#pragma unroll
				for (int qb = 0; qb < QB; ++qb) {
					float ls4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
					for (int kb = 0; kb < KB; ++kb)
#pragma unroll
						for (int hf = 0; hf < 2; ++hf) {
							float pv[8];
#pragma unroll
							for (int e = 0; e < 8; ++e) pv[e] = __builtin_fmaf(s[kb][qb][8 * hf + e], c1, nmc[qb]);
#pragma unroll
							for (int e = 0; e < 8; ++e) {
								float p = exp2_fast(pv[e]);
								if constexpr (MASKED) {
									int j = n0 + 32 * kb + 8 * (2 * hf + (e >> 2)) + 4 * g + (e & 3);
									p = ((j <= jmax[qb]) & (j >= jmin[qb])) ? p : 0.f;
								}
								ls4[e & 3] += p;
								pv[e] = p;
							}
							pf[qb][2 * kb + hf] = pack8<T>(pv[0], pv[1], pv[2], pv[3], pv[4], pv[5], pv[6], pv[7]);
						}
					lt[qb] = (ls4[0] + ls4[1]) + (ls4[2] + ls4[3]);
					// (a NaN sum - from inf or NaN inputs - also takes the other path, which propagates it)
					over = over || !(lt[qb] <= kFastSum) || (mrow[qb] == -INFINITY && jmax[qb] >= n0 && jmin[qb] < n0 + BN);
				}
				slow = __builtin_amdgcn_ballot_w64(over) != 0;
			}
			if (slow) {
#pragma unroll
				for (int qb = 0; qb < QB; ++qb) {
					// four independent partial maxima (and, below, partial sums): a chain of dependent
					// vector-ALU operations pays the full pipeline latency at every link
					float mx4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
					for (int kb = 0; kb < KB; ++kb)
#pragma unroll
						for (int i = 0; i < 16; ++i) {
							float x = s[kb][qb][i];
							if constexpr (MASKED) {
								int j = n0 + 32 * kb + 8 * (i >> 2) + 4 * g + (i & 3);
								x = ((j <= jmax[qb]) & (j >= jmin[qb])) ? x : -INFINITY;
							}
							s[kb][qb][i] = x;
							mx4[i & 3] = __builtin_fmaxf(mx4[i & 3], x);
						}
					float mx = __builtin_fmaxf(__builtin_fmaxf(mx4[0], mx4[1]), __builtin_fmaxf(mx4[2], mx4[3]));
					mx = pair_max(mx);
					// the row maximum becomes the reference whenever it exceeds it
					if (mx > mrow[qb]) {
						// (first keys of the row: l = 0 and O = 0, alpha = exp2(-inf) = 0 leaves them so)
						const float alpha = exp2_fast((mrow[qb] - mx) * c1);
						mrow[qb] = mx;
						nmc[qb] = -mx * c1;
						lrow[qb] *= alpha;
#pragma unroll
						for (int db = 0; db < DB; ++db)
#pragma unroll
							for (int i = 0; i < 16; ++i) oacc[qb][db][i] *= alpha;
					}
					float ls4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
					for (int kb = 0; kb < KB; ++kb)
#pragma unroll
						for (int i = 0; i < 16; ++i) {
							float p = exp2_fast(__builtin_fmaf(s[kb][qb][i], c1, nmc[qb]));
							ls4[i & 3] += p;
							s[kb][qb][i] = p;
						}
					lt[qb] = (ls4[0] + ls4[1]) + (ls4[2] + ls4[3]);
					pack_p(qb);
				}
			}
#pragma unroll
			for (int qb = 0; qb < QB; ++qb) lrow[qb] += lt[qb];
		} else {
#pragma unroll
			for (int qb = 0; qb < QB; ++qb) {
				float mx4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
				for (int kb = 0; kb < KB; ++kb)
#pragma unroll
					for (int i = 0; i < 16; ++i) {
						float x;
						if constexpr (CAP)
							x = __builtin_fmaf(tanh_fast(s[kb][qb][i] * a.cap_k1), a.softcap, bv[kb][qb][i >> 2][i & 3]);
						else
							x = __builtin_fmaf(s[kb][qb][i], c1, bv[kb][qb][i >> 2][i & 3]);
						if constexpr (MASKED) {
							int j = n0 + 32 * kb + 8 * (i >> 2) + 4 * g + (i & 3);
							x = ((j <= jmax[qb]) & (j >= jmin[qb])) ? x : -INFINITY;
						}
						s[kb][qb][i] = x;
						mx4[i & 3] = __builtin_fmaxf(mx4[i & 3], x);
					}
				float mx = __builtin_fmaxf(__builtin_fmaxf(mx4[0], mx4[1]), __builtin_fmaxf(mx4[2], mx4[3]));
				mx = pair_max(mx);
				float ls4[4] = {0.f, 0.f, 0.f, 0.f};
				// natural units with bias.  The running reference m of a row is only raised when some
				// row of the wave exceeds it by more than kRescaleSlack (log2 units): until then
				// P = exp2(x - m) may grow to 2^slack, which fp32 sums and 16-bit P hold without loss,
				// and the O accumulators are left alone.
				const float slack = kRescaleSlack * kLn2;
				if (__builtin_amdgcn_ballot_w64(mx > mrow[qb] + slack) != 0) {
					float m_new = __builtin_fmaxf(mrow[qb], mx);
					float m_use = m_new == -INFINITY ? 0.f : m_new;
					float alpha = exp2_fast((mrow[qb] - m_use) * kLog2e);
					mrow[qb] = m_new;
					lrow[qb] *= alpha;
#pragma unroll
					for (int db = 0; db < DB; ++db)
#pragma unroll
						for (int i = 0; i < 16; ++i) oacc[qb][db][i] *= alpha;
				}
				const float m_use = mrow[qb] == -INFINITY ? 0.f : mrow[qb];
				// (x - m) log2(e) as one fused multiply-add, x log2(e) - m log2(e) - unless some row's reference is so
				// large that m log2(e) leaves the fp32 range: a row whose keys all carry the finfo.min "mask" bias of
				// the bf16 type (-3.39e38).  Such a wave (rare) subtracts first.
				if (__builtin_amdgcn_ballot_w64(__builtin_fabsf(m_use) > 1e37f) == 0) {
					const float nm2 = -m_use * kLog2e;
#pragma unroll
					for (int kb = 0; kb < KB; ++kb)
#pragma unroll
						for (int i = 0; i < 16; ++i) {
							float p = exp2_fast(__builtin_fmaf(s[kb][qb][i], kLog2e, nm2));
							ls4[i & 3] += p;
							s[kb][qb][i] = p;
						}
				} else {
#pragma unroll
					for (int kb = 0; kb < KB; ++kb)
#pragma unroll
						for (int i = 0; i < 16; ++i) {
							float p = exp2_fast((s[kb][qb][i] - m_use) * kLog2e);
							ls4[i & 3] += p;
							s[kb][qb][i] = p;
						}
				}
				lrow[qb] += (ls4[0] + ls4[1]) + (ls4[2] + ls4[3]);
				pack_p(qb);
			}
		}
#pragma unroll
		for (int qb = 0; qb < QB; ++qb) drop_p(qb);

		// O^T += V^T P^T
		auto pv_batch = [&](auto batch_tag) {
			constexpr int BI = decltype(batch_tag)::value;
			if constexpr (BI + 1 < NBATCH) issue_v(std::integral_constant<int, BI + 1>{}, vfr[(BI + 1) & 1]);
#pragma unroll
			for (int u = 0; u < NF; ++u) {
				const int fi = BI * NF + u, st = fi / DB, db = fi % DB;
#pragma unroll
				for (int qb = 0; qb < QB; ++qb) oacc[qb][db] = mfma32(as_frag<T>(vfr[BI & 1][u]), pf[qb][st], oacc[qb][db]);
			}
		};
		__builtin_amdgcn_sched_barrier(0);
#if FA2_SETPRIO
		__builtin_amdgcn_s_setprio(FA2_SETPRIO);
#endif
		static_for<0, NBATCH>(pv_batch);
		// issue order: every product of a batch but the last is followed by the two transposed reads
		// of one fragment of the next batch (left to itself the compiler's order, and with it the
		// kernel's duration, changes with unrelated edits)
#pragma unroll
		for (int i = 0; i < (NBATCH - 1) * NF; ++i) {
			__builtin_amdgcn_sched_group_barrier(0x008, QB, 0);
			__builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
		}
		__builtin_amdgcn_sched_group_barrier(0x008, NF * QB, 0);
		__builtin_amdgcn_sched_barrier(0);
#if FA2_SETPRIO
		__builtin_amdgcn_s_setprio(0);
#endif
	};

	// Head dim 256 runs one wave per SIMD, so the softmax overlaps the matrix products only if the wave interleaves
	// them itself.  A tile without masking is handled as two halves of 32 keys, in four phases of KS products each:
	//   phase 0   S_0 = K_0 Q^T         |  (dropout: the generator calls of half 0)
	//   phase 1   S_1 = K_1 Q^T         |  P_0 from S_0   (dropout: mask on P_0, first rounds of the calls of half 1)
	//   phase 2   O^T += V_0^T P_0^T    |  P_1 from S_1   (dropout: their last rounds, mask on P_1)
	//   phase 3   O^T += V_1^T P_1^T
	// The vector-ALU work is cut into pieces that follow the products one by one, and every product is preceded by the
	// LDS read of a fragment PA products further on (a scheduling barrier after every slot pins that order).  The
	// softmax is the path without the row maximum, applied per half; a half that needs the maximum after all (decided
	// for the wave as a whole) takes it from its scores, which are still in their registers, before its P is used.
	// (Head dim 128 takes the same path in its four-wave workgroups, where two waves share a SIMD: B4 H32 S4096 causal forward 0.531 -> 0.511 ms,
	// B8 S2048 0.307 -> 0.294 ms; nothing at S 8192 or without a causal mask, and the eight-wave workgroups of long context
	// measured 0.4 % slower and stay on the plain tile body.  With dropout the generator's pieces need sixteen slots a phase.)
	constexpr bool PIPE = (D == 256 || (D == 128 && !DROP)) && NW == 4 && QB == 1 && FOLD && !SPLIT;
	auto tile_pipe = [&](int n0) {
		if constexpr (PIPE) {
			constexpr int NFR = KS;  // fragments = products of a phase: KS of K for a half, 2 sixteen-key steps x DB of V
			constexpr int RING = 8, PA = DROP ? 4 : 7;  // (dropout: the generator needs the registers)
			static_assert(2 * DB == KS && KS % RING == 0 && PA < RING, "");
			u32x4 fr[RING];
			f32x16 sc[2];
			u32x4 pp[2][2];  // [half][16-key step]: P packed to 16 bits
			float bx[4], lsum[4];
			auto read_k = [&](int hf, int f) __attribute__((always_inline)) {
				fr[f % RING] = __builtin_bit_cast(u32x4, *(const FA2_LDS V8*)(lds + koff[f % KR] + (f / KR) * 256 + hf * (32 * D * 2)));
			};
			auto read_v = [&](int hf, int f) __attribute__((always_inline)) {
				const int db = f % DB;
				fr[f % RING] = lds_tr_issue_rt<D>(lds + voff[db % DR][0] + (db / DR) * 256, lds + voff[db % DR][1] + (db / DR) * 256, 2 * hf + f / DB);
			};
			auto prod_s = [&](int hf, int f) __attribute__((always_inline)) {
				f32x16 zero;
#pragma unroll
				for (int i = 0; i < 16; ++i) zero[i] = 0.f;
				sc[hf] = mfma32(as_frag<T>(fr[f % RING]), qf[0][f], f == 0 ? zero : sc[hf]);
			};
			auto prod_o = [&](int hf, int f) __attribute__((always_inline)) {
				oacc[0][f % DB] = mfma32(as_frag<T>(fr[f % RING]), as_frag<T>(pp[hf][f / DB]), oacc[0][f % DB]);
			};
			// piece pc (0 .. 7) of the softmax of a half: values 4 q .. 4 q + 3 (q = pc / 2); first the exponents and two
			// exp2, then two exp2, the sums and the packing - a result is consumed some instructions after it was produced
			auto soft_piece = [&](int hf, int pc) __attribute__((always_inline)) {
				const int q = pc >> 1;
				if ((pc & 1) == 0) {
#pragma unroll
					for (int e = 0; e < 4; ++e) bx[e] = __builtin_fmaf(sc[hf][4 * q + e], c1, nmc[0]);
					bx[0] = exp2_fast(bx[0]);
					bx[1] = exp2_fast(bx[1]);
				} else {
					bx[2] = exp2_fast(bx[2]);
					bx[3] = exp2_fast(bx[3]);
#pragma unroll
					for (int e = 0; e < 4; ++e) lsum[e] = q == 0 ? bx[e] : lsum[e] + bx[e];
					pp[hf][q >> 1][2 * (q & 1)] = pack2<typename T::V2>(bx[0], bx[1]);
					pp[hf][q >> 1][2 * (q & 1) + 1] = pack2<typename T::V2>(bx[2], bx[3]);
				}
			};
			// after the pieces of a half: does the path without the maximum stand?  Otherwise the half is done again
			// from its scores with the row maximum (raising the reference and rescaling l and O where it exceeds it).
			auto soft_finish = [&](int hf) __attribute__((always_inline)) {
				float lt = (lsum[0] + lsum[1]) + (lsum[2] + lsum[3]);
				// (a NaN sum - from inf or NaN inputs - also takes the other path, which propagates it)
				const bool over = !(lt <= kFastSum) || mrow[0] == -INFINITY;
				if (__builtin_amdgcn_ballot_w64(over) != 0) {
					float mx4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
					for (int i = 0; i < 16; ++i) mx4[i & 3] = __builtin_fmaxf(mx4[i & 3], sc[hf][i]);
					float mx = pair_max(__builtin_fmaxf(__builtin_fmaxf(mx4[0], mx4[1]), __builtin_fmaxf(mx4[2], mx4[3])));
					if (mx > mrow[0]) {
						const float alpha = exp2_fast((mrow[0] - mx) * c1);
						mrow[0] = mx;
						nmc[0] = -mx * c1;
						lrow[0] *= alpha;
#pragma unroll
						for (int db = 0; db < DB; ++db)
#pragma unroll
							for (int i = 0; i < 16; ++i) oacc[0][db][i] *= alpha;
					}
					float ls4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
					for (int i = 0; i < 16; ++i) {
						float pv = exp2_fast(__builtin_fmaf(sc[hf][i], c1, nmc[0]));
						ls4[i & 3] += pv;
						sc[hf][i] = pv;
					}
#pragma unroll
					for (int h2 = 0; h2 < 2; ++h2)
						pp[hf][h2] = __builtin_bit_cast(u32x4, pack8<T>(sc[hf][8 * h2 + 0], sc[hf][8 * h2 + 1], sc[hf][8 * h2 + 2], sc[hf][8 * h2 + 3],
						                                                  sc[hf][8 * h2 + 4], sc[hf][8 * h2 + 5], sc[hf][8 * h2 + 6], sc[hf][8 * h2 + 7]));
					lt = (ls4[0] + ls4[1]) + (ls4[2] + ls4[3]);
				}
				lrow[0] += lt;
			};
			// Dropout: the two generator calls of a half (one per 16-key step; see dropout_words_rowlane_half), one after the
			// other, as pieces of two rounds each, and the mask on the packed P (see drop_p in the other tile body).
			uint32_t cs[4], dwp[2][2][2][2];  // state of the call in flight; words [half][call][group of four keys][word]
			const bool odd = qrow[0] & 1;
			const uint32_t thr2 = a.drop_thr * 0x10001u;
			// piece pc of call u of half hf: 0 .. 4 = rounds 2 pc, 2 pc + 1 (the counter is set up with the first), 5 = exchange
			auto gen_piece = [&](int hf, int u, auto pt) __attribute__((always_inline)) {
				if constexpr (DROP) {
					constexpr int pc = decltype(pt)::value;
					if constexpr (pc == 0) {
						cs[0] = (uint32_t)((n0 + 32 * hf + 4 * g + 8 * (2 * u + (odd ? 1 : 0))) >> 2);
						cs[1] = (uint32_t)qrow[0] >> 1;
						cs[2] = (uint32_t)hl[0];
						cs[3] = (uint32_t)b;
					}
					if constexpr (pc < 5) {
						philox4x32_rounds<2 * pc, 2 * pc + 2>(cs, drop_k0, drop_k1);
					} else {
						uint32_t own0 = odd ? cs[2] : cs[0], own1 = odd ? cs[3] : cs[1];
						uint32_t got0 = quad_swap1(odd ? cs[0] : cs[2]), got1 = quad_swap1(odd ? cs[1] : cs[3]);
						dwp[hf][u][0][0] = odd ? got0 : own0;
						dwp[hf][u][0][1] = odd ? got1 : own1;
						dwp[hf][u][1][0] = odd ? own0 : got0;
						dwp[hf][u][1][1] = odd ? own1 : got1;
					}
				}
			};
			auto mask_piece = [&](int hf, int u) __attribute__((always_inline)) {
				if constexpr (DROP) {
#pragma unroll
					for (int m = 0; m < 4; ++m) pp[hf][u][m] = keep_pair16(pp[hf][u][m], dwp[hf][u][m >> 1][m & 1], thr2);
				}
			};
			// one phase: NFR slots of (read ahead, product, vector-ALU piece)
			auto phase = [&](auto&& read_cur, auto&& prod, auto&& read_next, auto&& valu) __attribute__((always_inline)) {
				__builtin_amdgcn_sched_barrier(0);
				static_for<0, NFR>([&](auto jt) __attribute__((always_inline)) {
					constexpr int j = decltype(jt)::value;
					if constexpr (j + PA < NFR)
						read_cur(j + PA);
					else
						read_next(j + PA - NFR);
					prod(j);
					__builtin_amdgcn_sched_barrier(0);
					valu(jt);
					__builtin_amdgcn_sched_barrier(0);
				});
			};
			auto none = [&](auto) __attribute__((always_inline)) {};
			// (dropout: both calls of half 0 run in phase 0, the first call of half 1 at the end of phase 1, its second at the end of phase 2;
			// the mask of a half is applied once its P is final: after soft_finish, before the phase that uses it)
			auto gv0 = [&](auto jt) __attribute__((always_inline)) {
				constexpr int j = decltype(jt)::value;
				if constexpr (j < 12) gen_piece(0, j / 6, std::integral_constant<int, j % 6>{});
			};
			// the eight softmax pieces of half hf behind the products of a phase (the scores' last product is then at least two
			// products back): with sixteen slots one piece behind each of the products 2 .. 9, with eight slots (head dim 128)
			// behind the products 2 .. 7, two each behind the first two (other distributions measured the same)
			auto soft_slot = [&](int hf, auto jt) __attribute__((always_inline)) {
				constexpr int j = decltype(jt)::value;
				if constexpr (NFR >= 10) {
					if constexpr (j >= 2 && j < 10) soft_piece(hf, j - 2);
				} else if constexpr (j == 2 || j == 3) {
					soft_piece(hf, 2 * (j - 2));
					soft_piece(hf, 2 * (j - 2) + 1);
				} else if constexpr (j >= 4) {
					soft_piece(hf, j);
				}
			};
			auto sv0 = [&](auto jt) __attribute__((always_inline)) {
				constexpr int j = decltype(jt)::value;
				soft_slot(0, jt);
				if constexpr (j >= 10) gen_piece(1, 0, std::integral_constant<int, j - 10>{});
			};
			auto sv1 = [&](auto jt) __attribute__((always_inline)) {
				constexpr int j = decltype(jt)::value;
				soft_slot(1, jt);
				if constexpr (j >= 10) gen_piece(1, 1, std::integral_constant<int, j - 10>{});
			};
#pragma unroll
			for (int f = 0; f < PA; ++f) read_k(0, f);
			phase([&](int f) __attribute__((always_inline)) { read_k(0, f); }, [&](int f) __attribute__((always_inline)) { prod_s(0, f); },
			      [&](int f) __attribute__((always_inline)) { read_k(1, f); }, gv0);
			phase([&](int f) __attribute__((always_inline)) { read_k(1, f); }, [&](int f) __attribute__((always_inline)) { prod_s(1, f); },
			      [&](int f) __attribute__((always_inline)) { read_v(0, f); }, sv0);
			soft_finish(0);
			mask_piece(0, 0);
			mask_piece(0, 1);
			phase([&](int f) __attribute__((always_inline)) { read_v(0, f); }, [&](int f) __attribute__((always_inline)) { prod_o(0, f); },
			      [&](int f) __attribute__((always_inline)) { read_v(1, f); }, sv1);
			soft_finish(1);
			mask_piece(1, 0);
			mask_piece(1, 1);
			phase([&](int f) __attribute__((always_inline)) { read_v(1, f); }, [&](int f) __attribute__((always_inline)) { prod_o(1, f); }, none, none);
			__builtin_amdgcn_sched_barrier(0);
		}
	};

	// One pipeline step: publish tile t, start the copies of tile t + 1, compute.
	auto step = [&](auto masked_tag, int t) {
		const int n0 = t * BN;
		const int buf = t & 1;
		wait_async_loads();
		__syncthreads();
		if (t + 1 < ntiles) {
			int n1 = n0 + BN;
			int rows = sk_eff - n1 < BN ? sk_eff - n1 : BN;
			kload.load(lds + (buf ^ 1) * TILE_BYTES, kbase + (int64_t)n1 * a.k.ss, a.k.ss, rows, tid);
			vload.load(lds + (2 + (buf ^ 1)) * TILE_BYTES, vbase + (int64_t)n1 * a.v.ss, a.v.ss, rows, tid);
			if constexpr (BIAS_LDS) {
				if (bias_lds)
					bload.load(lds + 4 * TILE_BYTES + (buf ^ 1) * BIAS_BYTES, bias_base + (int64_t)m0 * a.bias_sm + (int64_t)n1 * 2,
					           a.bias_sm, brows, tid, (a.Sk - n1) >> 3);
			}
		}
		bool skip = false;
		if constexpr (decltype(masked_tag)::value) skip = n0 > wave_jmax || n0 + BN - 1 < wave_lmin;  // whole tile masked for this wave (uniform)
		if (!skip) {
			if constexpr (PIPE && !decltype(masked_tag)::value)
				tile_pipe(n0);
			else
				tile_body(masked_tag, n0);
		}
		// the other buffers next time
#pragma unroll
		for (int ks = 0; ks < KR; ++ks) koff[ks] ^= TILE_BYTES;
#pragma unroll
		for (int db = 0; db < DR; ++db) {
			voff[db][0] ^= TILE_BYTES;
			voff[db][1] ^= TILE_BYTES;
		}
		if constexpr (BIAS_LDS) boff_lane ^= BIAS_BYTES;
	};
	// Tiles that lie entirely inside every row's range of allowed keys need no mask.  They
	// run in a loop of their own, so that the steady-state loop is a single
	// straight-line body; the tiles on the window's left edge come before them, the tiles
	// on the causal diagonal / right edge / ragged end after.
	int t_lo = wave_lmax > 0 ? (wave_lmax + BN - 1) / BN : 0;  // first tile at or right of every row's first key
	t_lo = t_lo < t_begin ? t_begin : (t_lo > ntiles ? ntiles : t_lo);
	int t_full = (wave_jmin + 1) / BN;
	t_full = t_full < t_lo ? t_lo : (t_full > ntiles ? ntiles : t_full);
	for (int t = t_begin; t < t_lo; ++t) step(std::true_type{}, t);
	for (int t = t_lo; t < t_full; ++t) step(std::false_type{}, t);
	for (int t = t_full; t < ntiles; ++t) step(std::true_type{}, t);

	// epilogue: normalise, store O (lane: row c, four consecutive d per store) and LSE
	char* obase = a.o.ptr + (int64_t)b * a.o.sb + (int64_t)h * a.o.sh;
#pragma unroll
	for (int qb = 0; qb < QB; ++qb) {
		float lt = pair_sum(lrow[qb]);
		float inv = lt > 0.f ? 1.f / lt : 0.f;
		if constexpr (DROP) inv *= a.drop_inv_keep;
		int i = qrow[qb];
		if constexpr (SPLIT) {
			// partial result of this key range: [split][b][h][i][D] fp32 and [split][b][h][i]
			if (i < a.Sq) {
				int64_t row = (((int64_t)split * a.B + b) * a.Hq + hl[qb]) * a.Sq + i;
				float* rp = a.o_part + row * D;
#pragma unroll
				for (int db = 0; db < DB; ++db)
#pragma unroll
					for (int aa = 0; aa < 4; ++aa) {
						const f32x16& r = oacc[qb][db];
						f32x4 o4 = {r[4 * aa] * inv, r[4 * aa + 1] * inv, r[4 * aa + 2] * inv, r[4 * aa + 3] * inv};
						*(f32x4*)(rp + 32 * db + 8 * aa + 4 * g) = o4;
					}
				if (g == 0) {
					float lse = -INFINITY;
					if (lt > 0.f) lse = BIAS ? mrow[qb] + log2_fast(lt) * kLn2 : (mrow[qb] * c1 + log2_fast(lt)) * kLn2;
					a.lse_part[row] = lse;
				}
			}
			continue;
		}
		if (i < a.Sq) {
			char* rp = obase + (int64_t)i * a.o.ss;
#pragma unroll
			for (int db = 0; db < DB; ++db)
#pragma unroll
				for (int aa = 0; aa < 4; ++aa) {
					const f32x16& r = oacc[qb][db];
					u32x2 pk = {pack2<typename T::V2>(r[4 * aa] * inv, r[4 * aa + 1] * inv),
					            pack2<typename T::V2>(r[4 * aa + 2] * inv, r[4 * aa + 3] * inv)};
					*(u32x2*)(rp + (32 * db + 8 * aa + 4 * g) * 2) = pk;
				}
			if (g == 0) {
				float lse;
				if (lt > 0.f)
					lse = BIAS ? mrow[qb] + log2_fast(lt) * kLn2 : (mrow[qb] * c1 + log2_fast(lt)) * kLn2;
				else
					lse = -INFINITY;
				a.lse[((int64_t)b * a.Hq + h) * a.Sq + i] = lse;
			}
		}
	}
}

// O = sum_s exp(lse_s - lse) O_s, lse = log sum_s exp(lse_s) over the key ranges of a split forward.
// One thread per (row, 8 head-dim values); HBM-bound and small.
template <typename T, int D>
__global__ __launch_bounds__(256) void fwd_combine_kernel(const KArgs a) {
	constexpr int TPR = D / 8;
	constexpr int RPB = 256 / TPR;
	int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
	int part = threadIdx.x % TPR;
	int64_t nrows = (int64_t)a.B * a.Hq * a.Sq;
	if (row >= nrows) return;
	int i = (int)(row % a.Sq);
	int64_t bh = row / a.Sq;
	int h = (int)(bh % a.Hq), b = (int)(bh / a.Hq);
	float m = -INFINITY;
	for (int s = 0; s < a.nsplit; ++s) m = __builtin_fmaxf(m, a.lse_part[(int64_t)s * nrows + row]);
	float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
	float tot = 0.f;
	if (m > -INFINITY) {
		for (int s = 0; s < a.nsplit; ++s) {
			float wgt = exp2_fast((a.lse_part[(int64_t)s * nrows + row] - m) * kLog2e);
			tot += wgt;
			const float* op = a.o_part + ((int64_t)s * nrows + row) * D + part * 8;
			f32x4 x0 = *(const f32x4*)op, x1 = *(const f32x4*)(op + 4);
#pragma unroll
			for (int e = 0; e < 4; ++e) {
				acc[e] += wgt * x0[e];
				acc[4 + e] += wgt * x1[e];
			}
		}
	}
	float inv = tot > 0.f ? 1.f / tot : 0.f;
	char* rp = a.o.ptr + (int64_t)b * a.o.sb + (int64_t)h * a.o.sh + (int64_t)i * a.o.ss + part * 16;
	*(typename T::V8*)rp = pack8<T>(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv, acc[4] * inv, acc[5] * inv, acc[6] * inv,
	                                acc[7] * inv);
	if (part == 0) a.lse[row] = tot > 0.f ? m + log2_fast(tot) * kLn2 : -INFINITY;
}

template <typename T, int D>
struct FwdCfg {
	// D <= 128: 8 waves, two per SIMD (<= 256 registers each): while one waits on LDS or
	// on a matrix product the other issues.  D = 256 needs the whole register file.
	// (the launcher prefers two independent workgroups of 4 waves per CU where the K and V of a head fit an XCD's L2,
	// see launch_fwd_t)
	static constexpr int NW = D <= 128 ? 8 : 4;
	static constexpr int QB = 1;
	static constexpr int WPS = 1;
	static constexpr int BM = NW * QB * 32;
};

// Split forward: 2 waves x 32 rows per workgroup (the query is short), nsplit key ranges each.
template <typename T, int D>
hipError_t launch_fwd_split_t(bool bias, bool drop, KArgs& a, hipStream_t s) {
	constexpr int NW = D == 256 ? 4 : 2, BM = NW * 32;  // (D = 256: four waves, the tile copies need the threads)
	a.mtiles = (a.Sq + BM - 1) / BM;
	int groups = a.B * a.Hkv;
	a.xcd_remap = (groups % 8 == 0) ? 1 : 0;
	a.interleave = 1;
	dim3 grid((unsigned)((a.pack_gqa ? a.B * a.Hkv : a.mtiles * a.B * a.Hq) * a.nsplit)), block(NW * 64);
	const bool blds = bias && a.bias_lds && D <= 128 && !a.pack_gqa;
	if (blds && drop)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, 1, 1, true, true, true, true>), grid, block, 0, s, a);
	else if (blds)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, 1, 1, true, false, true, true>), grid, block, 0, s, a);
	else if (bias && drop)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, 1, 1, true, true, true>), grid, block, 0, s, a);
	else if (bias)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, 1, 1, true, false, true>), grid, block, 0, s, a);
	else if (drop)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, 1, 1, false, true, true>), grid, block, 0, s, a);
	else
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, 1, 1, false, false, true>), grid, block, 0, s, a);
	int64_t nrows = (int64_t)a.B * a.Hq * a.Sq;
	constexpr int RPB = 256 / (D / 8);
	hipLaunchKernelGGL((fwd_combine_kernel<T, D>), dim3((unsigned)((nrows + RPB - 1) / RPB)), dim3(256), 0, s, a);
	return hipGetLastError();
}

// One tile configuration: NW waves x 32 rows per workgroup (WPS: launch bound, waves per SIMD).
template <typename T, int D, int NW, int WPS>
hipError_t launch_fwd_cfg(bool bias, bool drop, KArgs& a, hipStream_t s) {
	constexpr int QB = 1, BM = NW * QB * 32;
	a.mtiles = (a.Sq + BM - 1) / BM;
	int groups = a.B * a.Hkv;
	a.xcd_remap = (groups % 8 == 0) ? 1 : 0;
	a.interleave = a.xcd_remap ? launch_order(a, a.Hq / a.Hkv, groups / 8, (int64_t)a.Sk * D * 4) : 1;
	if (bias && a.bias_sh == 0 && a.B % 8 == 0) a.xcd_remap = a.kv_lens ? 3 : 2;
	dim3 grid((unsigned)(a.mtiles * a.B * a.Hq)), block(NW * 64);
	a.fold_half = fold_half_of(a, NW, (int64_t)grid.x, D == 64 || WPS == 2);
	const bool blds = bias && a.bias_lds;
	if (a.softcap > 0.f && drop)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, true, true, false, false, true>), grid, block, 0, s, a);
	else if (a.softcap > 0.f)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, true, false, false, false, true>), grid, block, 0, s, a);
	else if (blds && drop)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, true, true, false, true>), grid, block, 0, s, a);
	else if (blds)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, true, false, false, true>), grid, block, 0, s, a);
	else if (bias && drop)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, true, true>), grid, block, 0, s, a);
	else if (bias)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, true, false>), grid, block, 0, s, a);
	else if (drop)
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, false, true>), grid, block, 0, s, a);
	else
		hipLaunchKernelGGL((fwd_kernel<T, D, NW, QB, WPS, false, false>), grid, block, 0, s, a);
	return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_fwd_t(bool bias, bool drop, KArgs& a, hipStream_t s) {
	if (a.nsplit > 1) return launch_fwd_split_t<T, D>(bias, drop, a, s);
	typedef FwdCfg<T, D> C;
	if constexpr (C::NW == 8) {
		// A grid that leaves at least half of the chip idle (small batch x heads, short sequences): workgroups of
		// 128 rows instead of 256, twice as many of them, still at most one per CU.
		int64_t wgs = (int64_t)((a.Sq + 127) / 128) * a.B * a.Hq;
		if (wgs <= kNumCU) return launch_fwd_cfg<T, D, 4, 1>(bias, drop, a, s);
		// Larger grids: two independent 128-row workgroups per CU instead of one of 256 rows - the same eight waves, but
		// one workgroup computes while the other loads its Q, waits for its first tiles or stores its result, and a
		// causal tile of 128 rows wastes less on the diagonal.  They read K and V twice as often, so only where the K
		// and V of a head stay in an XCD's L2 (4 MiB; B1 H4 S16384 D = 128, 8 MiB a head: 0.372 -> 0.568 ms).
		// D = 64 keeps below 256 registers a wave in every variant and gains everywhere (B32 S512 H12 0.053 -> 0.045 ms,
		// B128 S197 0.071 -> 0.056 ms, B4 S4096 Hq32 causal 0.377 -> 0.330 ms); D = 128 needs an instantiation bound to
		// 256 registers, which the variants with bias do not fit.  Its four-wave workgroups run their unmasked tiles
		// through the pipelined path; with that they gain under a causal mask up to the 4 MiB (Hq32 Hkv8: B8 S2048 0.330 ->
		// 0.303 ms, B4 S4096 0.563 -> 0.516 ms, B2 S8192 0.974 -> 0.965 ms, B2 S6144 Hq16 0.298 -> 0.280 ms; S16384 + 1 %) and
		// without a mask up to 4096 keys (B8 S2048 0.520 -> 0.502 ms, B4 S4096 0.958 -> 0.953 ms; S8192 + 1 %).
		// (With dropout the tiles keep the plain body and the limits measured for it: under a causal mask 2 MiB once the
		// grid exceeds two workgroups per CU - B2 Hq32 S8192 0.953 -> 0.971 ms - and without a mask 1024 keys, where the
		// start and end of a workgroup weigh most - B16 S1024 0.316 -> 0.297 ms.)
		const int64_t kv_limit = D == 64   ? (4 << 20)
		                         : a.causal ? ((drop && wgs > 2 * kNumCU) ? (2 << 20) : (4 << 20))
		                                    : (drop ? 1024 * D * 4 : (2 << 20));
		if ((int64_t)a.Sk * D * 4 <= kv_limit && (D == 64 || (!bias && !(a.softcap > 0.f))))
			return launch_fwd_cfg<T, D, 4, (D == 128 ? 2 : 1)>(bias, drop, a, s);
	}
	return launch_fwd_cfg<T, D, C::NW, C::WPS>(bias, drop, a, s);
}

}  // namespace fa2
