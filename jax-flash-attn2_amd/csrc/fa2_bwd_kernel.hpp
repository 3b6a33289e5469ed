// Backward kernels: delta pre-pass, dK/dV kernel, dQ kernel.  They take the
// place of `_attn_bwd_preprocess` and `_attn_bwd` with its two roles
// (jax_flash_attn2/flash_attention_triton/_backward_triton.py:79-147, 150-435,
// 438-709, 712-945) and of the XLA sum over each KV group (:1156-1161).
//
// P is recomputed from the saved logsumexp.  With dropout, the same
// position-keyed Philox mask as the forward is regenerated.
//
// dK/dV kernel: one workgroup = NW waves x 32 keys of one (batch, KV head);
// K and V rows live in registers; Q and dO tiles of the r = Hq/Hkv query
// heads of the group are streamed through LDS, so dK and dV accumulate over
// the whole group in registers - no atomics and no per-q-head temporary.
//   S  [q, kv] = Q K^T          A = Q from LDS,            B = K in registers
//   dP [q, kv] = dO V^T         A = dO from LDS,           B = V in registers
//   dV^T[d,kv] += dO^T P        A = dO, transposed LDS read, B = P  (S accumulator packed)
//   dK^T[d,kv] += Q^T  dS       A = Q,  transposed LDS read, B = dS
//
// dQ kernel: one workgroup = one tile of query rows of one (batch, q-head),
// K/V tiles streamed exactly as in the forward.
//   S^T [kv, q] = K Q^T ; dP^T[kv, q] = V dO^T     (Q, dO in registers)
//   dQ^T[d,  q] += K^T dS^T     A = K, transposed LDS read, B = dS^T packed
#pragma once
#include "fa2_common.hpp"
#include "fa2_fwd_kernel.hpp"
#include "fa2_kernels.hpp"

namespace fa2 {

// ---------------------------------------------------------------------------
// delta[b,h,i] = sum_d O[b,i,h,d] * dO[b,i,h,d]     (HBM-bound; reads O and dO once)
// ---------------------------------------------------------------------------
template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const KArgs a) {
	constexpr int TPR = D / 8;          // threads per row, 8 elements each
	constexpr int RPB = 256 / TPR;      // rows per block
	int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
	int part = threadIdx.x % TPR;
	int64_t nrows = (int64_t)a.B * a.Sq * a.Hq;
	float acc = 0.f;
	int h = 0, b = 0, i = 0;
	if (row < nrows) {
		h = (int)(row % a.Hq);
		int64_t r = row / a.Hq;
		i = (int)(r % a.Sq);
		b = (int)(r / a.Sq);
		typename T::V8 o = *(const typename T::V8*)(a.o.ptr + b * a.o.sb + (int64_t)i * a.o.ss + (int64_t)h * a.o.sh + part * 16);
		typename T::V8 d = *(const typename T::V8*)(a.dout.ptr + b * a.dout.sb + (int64_t)i * a.dout.ss + (int64_t)h * a.dout.sh + part * 16);
#pragma unroll
		for (int e = 0; e < 8; ++e) acc += (float)o[e] * (float)d[e];
	}
#pragma unroll
	for (int sft = TPR / 2; sft >= 1; sft >>= 1) acc += __shfl_xor(acc, sft, 64);
	if (row < nrows && part == 0) a.delta[((int64_t)b * a.Hq + h) * a.Sq + i] = acc;
}

// ---------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------
// BIAS_T: the bias has the element type of q / k / v (no run-time type dispatch per value)
// CAP: tanh soft-capping of the scores (see the forward kernel); the bias itself may then be absent
// One key tile `nt` of (batch b, kv-head hk): the whole life of its dK / dV accumulators.  hsi / hsplit: this workgroup's
// share when the streamed steps of the tile are split over workgroups.  `order`: the order in which the streamed
// (q-head, query tile) steps are visited -
//   0  head by head, query tiles ascending inside a head;
//   1  query tile by query tile ascending, the r q-heads inside a tile (starting with head `rot`);
//   2  the same with the query tiles descending.
// With 1 and 2 every workgroup of a KV group that walks in the same direction is at the same query tile at the same
// time, whatever its key tile - the tiles of Q / dO they stream are then fetched from memory once per XCD.
// What depends on the batch row only: valid rows / keys and the causal alignment, the dropout key.
struct DkdvRow {
	int sq_eff, sk_eff, off;
	uint32_t drop_k0, drop_k1;
};

template <bool DROP>
FA2_DEV DkdvRow dkdv_row(const KArgs& a, int b) {
	DkdvRow rw;
	rw.sq_eff = a.Sq;
	rw.sk_eff = a.Sk;
	if (a.seqlens) {
		int len = a.seqlens[b];
		len = len < 0 ? 0 : (len > a.Sk ? a.Sk : len);
		rw.sq_eff = len < a.Sq ? len : a.Sq;
		rw.sk_eff = len;
	}
	rw.off = rw.sk_eff - rw.sq_eff;
	if (a.kv_lens) {  // key padding only: the causal alignment keeps counting from the full key count
		int len = a.kv_lens[b];
		len = len < 0 ? 0 : len;
		rw.sk_eff = len < rw.sk_eff ? len : rw.sk_eff;
	}
	// dropout key: from the parameter block, or from device memory when the caller keeps it there
	rw.drop_k0 = a.drop_k0;
	rw.drop_k1 = a.drop_k1;
	if constexpr (DROP) {
		if (a.seed_dev) {
			rw.drop_k0 = a.seed_dev[0];
			rw.drop_k1 = a.seed_dev[1];
		}
	}
	return rw;
}

// K, V rows of this lane's key of key tile nt as B operands: the lane holds X[key][16 ks + 8 g .. + 7].
template <typename T, int D, int NW>
FA2_DEV void dkdv_load_kv(const KArgs& a, int nt, int hk, int b, typename T::V8 (&kf)[D / 16], typename T::V8 (&vf)[D / 16]) {
	typedef typename T::V8 V8;
	const int tid = threadIdx.x, lane = tid & 63;
	const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, c = lane & 31;
	const int jcol = nt * (NW * 32) + 32 * w + c;
	int j = jcol < a.Sk ? jcol : a.Sk - 1;
	const char* kp = a.k.ptr + (int64_t)b * a.k.sb + (int64_t)hk * a.k.sh + (int64_t)j * a.k.ss + g * 16;
	const char* vp = a.v.ptr + (int64_t)b * a.v.sb + (int64_t)hk * a.v.sh + (int64_t)j * a.v.ss + g * 16;
#pragma unroll
	for (int ks = 0; ks < D / 16; ++ks) {
		kf[ks] = *(const V8*)(kp + ks * 32);
		vf[ks] = *(const V8*)(vp + ks * 32);
	}
}

// WALKS: `order` is a run-time value (the paired kernel); otherwise the tile is walked head by head and `order_rt` is not looked at.
template <typename T, int D, int NW, int QB, bool BIAS, bool DROP, bool BIAS_T, bool CAP, bool WALKS>
FA2_DEV void bwd_dkdv_tile(const KArgs& a, const int nt, const int hk, const int b, const int hsi, const int hsplit, const int order_rt,
                           const int rot, const DkdvRow& rw) {
	const int order = WALKS ? order_rt : 0;
	static_assert(!CAP || (BIAS && !BIAS_T), "soft-capping runs on the plain path with bias");
	typedef typename T::V8 V8;
	constexpr int BN = NW * 32;     // keys per workgroup
	constexpr int BMQ = QB * 32;    // query rows per streamed tile
	constexpr int KS = D / 16;
	constexpr int DB = D / 32;
	constexpr int NT = NW * 64;
	constexpr int TILE_BYTES = BMQ * D * 2;
	constexpr int STAT_BYTES = BMQ * 4;
	// Register files pinned by hand (K / V fragments and the dK / dV accumulators in AGPRs, the
	// S / dP accumulators in VGPRs) when the AGPR file holds the former; the bias and dropout
	// variants need the registers for other things and leave the choice to the compiler.
	constexpr bool KV_AGPR = 2 * KS * 4 + 2 * DB * 16 <= 256 && !BIAS && !DROP;
	// On that path the elementwise stage is shortened: the chains of S and dP start from
	// -lse / (scale log2(e)) and -delta instead of 0, so that P = exp2(c1 * S accumulator) and
	// dS = P * (dP accumulator).  The factor c1 = scale * log2(e) is applied to the fp32
	// accumulator, as the reference scales the fp32 result of its dot (_backward_triton.py:554-559).
	constexpr bool FOLD = KV_AGPR;
	// Head dim 64 with bias, no dropout (matrix products through the compiler's builtins): the chain of dP still starts
	// from -delta of the block's rows - the start value is the four LDS reads of the statistics as they are, the
	// subtraction per value goes away (one of about eight vector-ALU instructions per value of a kernel that is bound by them).
	constexpr bool FOLD_DEL = !FOLD && BIAS && !DROP && D == 64;
	// Where the register files are left to the compiler it chooses accumulation registers for S / dP as well - results
	// that the vector ALU consumes - and copies them out value by value; at head dim 256, where dK / dV fill the
	// accumulation registers, it also moves 32 registers of dK / dV out of the way and back in every block (96 extra
	// vector-ALU instructions per block of 16 values).  For the variants named here the products of S / dP are therefore
	// issued as inline assembly with the accumulator pinned to vector registers.
	constexpr bool S_VGPR = !KV_AGPR && ((D == 256 && !BIAS) || (D == 128 && BIAS && !DROP));  // (the other variants run out of vector registers in the pinned form)

	// A bias in the element type of q is streamed through LDS as tiles of BMQ rows x BN keys
	// where LDS has the room (the launcher then guarantees 16-byte aligned rows and whole key
	// tiles): fetched one key per lane from global memory, every value is a 2-byte load of its own.
	// (D = 128: LDS has room only with 64-row tiles, which the launcher chooses for bias.  D = 256, 32-row tiles: through
	// LDS the dK/dV kernel of B2 H16 S4096 with a bias per head takes 1.37 ms, with a load per value 4.12 ms.)
	constexpr bool BIAS_LDS = BIAS && BIAS_T && 4 * TILE_BYTES + 4 * STAT_BYTES + 2 * BMQ * BN * 2 <= 160 * 1024;
	constexpr int BIAS_BYTES = BIAS_LDS ? BMQ * BN * 2 : 0;
	static_assert(BN == 128, "bias tiles use the 128-element row geometry");
	// Q[0] dO[0] Q[1] dO[1] | lse[0] lse[1] delta[0] delta[1] | bias[0] bias[1]
	// (buffer 1 of each kind lies a power of two behind buffer 0: the per-lane read addresses below
	// carry the buffer in that one bit and are flipped once per step, so that every read in the
	// loop is register + immediate with no address arithmetic)
	__shared__ __attribute__((aligned(1024))) char smem[4 * TILE_BYTES + 4 * STAT_BYTES + 2 * BIAS_BYTES];
	FA2_LDS char* lds = (FA2_LDS char*)smem;
	FA2_LDS char* stat = lds + 4 * TILE_BYTES;
	FA2_LDS char* lds_bias = lds + 4 * TILE_BYTES + 4 * STAT_BYTES;

	const int tid = threadIdx.x, lane = tid & 63;
	// the wave index as an explicitly scalar value: everything derived from it (tile bounds, loop trip counts,
	// "nothing to do for this wave") then stays in scalar registers and scalar branches
	const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, c = lane & 31;
	const uint32_t drop_k0 = rw.drop_k0, drop_k1 = rw.drop_k1;
	const int r = a.Hq / a.Hkv;
	const int sq_eff = rw.sq_eff, sk_eff = rw.sk_eff, off = rw.off;
	const int n0 = nt * BN;
	const int wn0 = n0 + 32 * w;
	const int jcol = wn0 + c;  // this lane's key

	// K, V rows of this lane's key as B operands: lane holds X[jcol][16ks + 8g .. +7]
	V8 kf[KS], vf[KS];
	dkdv_load_kv<T, D, NW>(a, nt, hk, b, kf, vf);
	// The fragments must have arrived before the loop over streamed tiles starts.  Otherwise the compiler places its
	// waits for these loads (s_waitcnt vmcnt) at their first uses inside the loop - it does not see the wait that
	// publishes a tile - where the same counter also counts the tile copies in flight: every step would then wait
	// for the copies of the NEXT tile before its first product.  (With KV_AGPR the loads go straight into
	// accumulation registers, where the inline-assembly products read them.)
#pragma unroll
	for (int ks = 0; ks < KS; ++ks) {
		if constexpr (KV_AGPR)
			asm volatile("; K / V fragment present" : "+a"(kf[ks]), "+a"(vf[ks]));
		else
			asm volatile("; K / V fragment present" : "+v"(kf[ks]), "+v"(vf[ks]));
	}


	f32x16 dk[DB], dv[DB];
#pragma unroll
	for (int db = 0; db < DB; ++db)
#pragma unroll
		for (int i = 0; i < 16; ++i) dk[db][i] = dv[db][i] = 0.f;

	// Row i may look at keys i + off - win_left .. i + off + win_right (each bound only when >= 0; causal is
	// win_right = 0), so key j is seen by rows j - off - win_right .. j - off + win_left.
	const int wr = a.win_right, wl = a.win_left;
	// query tiles that see at least one key of this workgroup
	int q_lo = 0;
	if (wr >= 0) {
		int first = n0 - off - wr;  // first row allowed to see key n0
		q_lo = first > 0 ? first / BMQ : 0;
	}
	int q_hi = (sq_eff + BMQ - 1) / BMQ;  // exclusive
	if (wl >= 0) {
		int last = n0 + BN - 1 - off + wl;  // last row allowed to see the workgroup's last key
		int e = last >= 0 ? last / BMQ + 1 : 0;
		q_hi = e < q_hi ? e : q_hi;
	}
	if (n0 >= sk_eff) q_hi = q_lo;
	// rows that may see this lane's key: row_lo .. row_hi (none when the key itself is beyond the valid ones)
	int row_lo = wr >= 0 ? jcol - off - wr : -(1 << 30);
	int row_hi = sq_eff - 1;
	if (wl >= 0) row_hi = jcol - off + wl < row_hi ? jcol - off + wl : row_hi;
	if (jcol >= sk_eff) row_lo = 1 << 30;
	const int nq = q_hi > q_lo ? q_hi - q_lo : 0;
	const int steps = nq * r;
	// this workgroup's share of the steps (all of them unless the launch splits the steps of a key tile over `hsplit` workgroups)
	const int s_lo = hsplit > 1 ? (int)((int64_t)steps * hsi / hsplit) : 0;
	const int s_hi = hsplit > 1 ? (int)((int64_t)steps * (hsi + 1) / hsplit) : steps;

	const float c1 = BIAS ? a.scale : a.scale * kLog2e;
	const float inv_scale = 1.f / a.scale;

	TileLoader<D, BMQ, NT> qload, doload;
	qload.init(a.q.ss, tid);
	doload.init(a.dout.ss, tid);
	TileLoader<128, BMQ, NT> bload;
	if constexpr (BIAS_LDS) bload.init(a.bias_sm, tid);
	// Streamed tile `step` in the order `order` asks for (see above).  Head by head is what a workgroup with one key
	// tile does: walking the query tiles outermost there measured 2 - 3 % slower (the workgroups of a KV group differ in
	// length and drift apart either way).  The two query-tile-outermost orders belong to the paired tiles of
	// bwd_dkdv_kernel, where all workgroups are equally long and stay together.
	auto decode_step = [&](int step, int& hq, int& m0) __attribute__((always_inline)) {
		int hi, i;
		if (order == 0) {
			hi = step / nq;
			i = step - hi * nq;
		} else {
			int t = step / r;
			hi = step - t * r + rot;
			hi = hi >= r ? hi - r : hi;
			i = order == 2 ? nq - 1 - t : t;
		}
		// (explicitly scalar: the results feed address arithmetic in branches that only some lanes take, and values the
		// compiler has to merge across such a branch end up in vector registers - every multiply of the tile's base
		// address then runs on the vector ALU)
		hq = __builtin_amdgcn_readfirstlane(hk * r + hi);
		m0 = __builtin_amdgcn_readfirstlane((q_lo + i) * BMQ);
	};
	// start the copies of streamed tile `step` (rows beyond Sq are fetched from the last valid row)
	// base addresses of a streamed tile, as explicitly scalar values (computed in uniform control flow, ahead of the
	// branch in which some lanes fetch the statistics)
	struct TileBase {
		const char *q, *dout, *bias;
	};
	auto tile_base = [&](int hq, int m0) __attribute__((always_inline)) {
		TileBase t;
		t.q = TileLoader<D, BMQ, NT>::uniform(a.q.ptr + (int64_t)b * a.q.sb + (int64_t)hq * a.q.sh + (int64_t)m0 * a.q.ss);
		t.dout = TileLoader<D, BMQ, NT>::uniform(a.dout.ptr + (int64_t)b * a.dout.sb + (int64_t)hq * a.dout.sh + (int64_t)m0 * a.dout.ss);
		t.bias = nullptr;
		if constexpr (BIAS_LDS) {
			int hb = a.bias_group ? hk : hq;
			t.bias = TileLoader<D, BMQ, NT>::uniform(a.bias + (int64_t)b * a.bias_sb + (int64_t)hb * a.bias_sh + (int64_t)m0 * a.bias_sm + (int64_t)n0 * 2);
		}
		return t;
	};
	auto issue_tile = [&](int step, const TileBase& tb, int m0, FA2_LDS char* qdst, FA2_LDS char* dodst) __attribute__((always_inline)) {
		int rows = a.Sq - m0 < BMQ ? a.Sq - m0 : BMQ;
		qload.load(qdst, tb.q, a.q.ss, rows, tid);
		doload.load(dodst, tb.dout, a.dout.ss, rows, tid);
		if constexpr (BIAS_LDS) bload.load(lds_bias + ((step - s_lo) & 1) * BIAS_BYTES, tb.bias, a.bias_sm, rows, tid, (a.Sk - n0) >> 3);
	};
	// per-row statistics of a tile: thread t < BMQ fetches lse, t in [BMQ, 2 BMQ) fetches delta.
	// The value is only touched again in store_stat(), a whole step later: nothing here may wait for the load.
	const int stat_row = tid % BMQ;
	const float* stat_src = tid < BMQ ? a.lse : a.delta;
	auto fetch_stat = [&](int hq, int m0) -> float {
		float x = 0.f;
		if (tid < 2 * BMQ) {
			int i = m0 + stat_row;
			i = i < a.Sq ? i : a.Sq - 1;
			x = stat_src[((int64_t)b * a.Hq + hq) * a.Sq + i];
		}
		return x;
	};
	// lse in the units the elementwise stage wants, both negated where they start the chains
	// (lse: -lse / (scale log2(e)) ... in the units of the raw dot product where it starts the chain of S, else -lse log2(e),
	// the addend of the fused multiply-add that forms the exponent; delta: negated where it starts the chain of dP)
	const float stat_mul = tid < BMQ ? (FOLD ? -inv_scale : -kLog2e) : ((FOLD || FOLD_DEL) ? -1.f : 1.f);
	auto store_stat = [&](float x, int buf) {
		if (tid < 2 * BMQ) {
			int which = tid / BMQ;
			// (kept finite: lse of a row whose keys all carry the finfo.min "mask" bias of the bf16 type is -3.39e38)
			*(FA2_LDS float*)(stat + (2 * which + buf) * STAT_BYTES + stat_row * 4) = __builtin_fminf(x * stat_mul, 3.0e38f);
		}
	};

	// per-lane LDS byte offsets (swizzle folded in) of the fragments read in the loop
	// (the swizzle touches the low four bits of the chunk index only: chunks 16 and up - head dim 256 - are the same
	// offsets 256 bytes further on, an immediate of the read instead of more registers)
	constexpr int KR = KS < 8 ? KS : 8, DR = DB < 4 ? DB : 4;
	int poff[KR];
#pragma unroll
	for (int ks = 0; ks < KR; ++ks) poff[ks] = tile_off<D>(c, 2 * ks + g);
	int toff[DR][2];
	{
		int i16 = lane & 15;
		int trow = 4 * g + (i16 >> 2);
		int tcol = 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
#pragma unroll
		for (int db = 0; db < DR; ++db) {
			int col = 32 * db + tcol;
			toff[db][0] = tile_off<D>(trow, col >> 3) + ((col & 4) << 1);
			toff[db][1] = tile_off<D>(trow + 8, col >> 3) + ((col & 4) << 1);
		}
	}

	int soff = 16 * g;  // statistics: this half-wave's four rows of a quad (+ the buffer, flipped per step)

	// bias tile (rows of 128 keys): this lane's 8-byte piece of rows 4 g + i16 / 4 (+ 8) at its wave's 32 keys
	int boffq[2] = {0, 0};
	if constexpr (BIAS_LDS) {
		int i16 = lane & 15;
		int trow = 4 * g + (i16 >> 2);
		int col = 32 * w + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
		boffq[0] = tile_off<128>(trow, col >> 3) + ((col & 4) << 1);
		boffq[1] = tile_off<128>(trow + 8, col >> 3) + ((col & 4) << 1);
	}

	// One streamed tile of BMQ query rows of q-head hq.  MASKED = some (row, key)
	// of this wave's 32 keys x BMQ rows is masked.
	auto tile_body = [&](auto masked_tag, int hq, int m0) __attribute__((always_inline)) {
		constexpr bool MASKED = decltype(masked_tag)::value;
		const char* bias_base = nullptr;
		if constexpr (BIAS) {
			int hb = a.bias_group ? hk : hq;
			int jc = jcol < a.Sk ? jcol : a.Sk - 1;
			int es = a.bias_dtype == 3 ? 4 : a.bias_dtype == 4 ? 1 : 2;
			bias_base = a.bias + (int64_t)b * a.bias_sb + (int64_t)hb * a.bias_sh + (int64_t)jc * es;
		}
		// The tile's QB blocks of 32 rows go through three stages,
		//   A(i): S_i = Q_i K^T, dP_i = dO_i V^T          (2 KS matrix products)
		//   B(i): P_i, dS_i from S_i, dP_i, lse, delta      (elementwise, 16 values per lane)
		//   C(i): dV^T += dO_i^T P_i, dK^T += Q_i^T dS_i   (4 DB matrix products)
		// software-pipelined: pipeline stage k runs A(k), B(k-1) and C(k-2) together, cut
		// into NSLOT slots.  A slot issues one product of A(k), one of C(k-2), the LDS reads
		// of the fragments that the slot PA places further on will use (so every read has PA
		// slots to complete and the LDS traffic is spread evenly), and its share of the
		// elementwise math of B(k-1) - the vector ALU and the LDS work in the shadow of the
		// matrix pipe.  A scheduling barrier after every slot pins that order.
		constexpr int NSLOT = 2 * KS;     // = 4 DB
		constexpr int PA = 4;             // read-ahead distance in slots
		constexpr int RING = PA + 1;
		static_assert(NSLOT % 16 == 0 || 16 % NSLOT == 0, "");
		f32x16 s[2], dp[2];
		u32x4 pbits[2][2], sbits[2][2];   // [block parity][16-row half]: P and dS packed to 16 bits
		V8 afr[RING];                     // fragments of Q_i / dO_i for the products of A
		u32x4 cfr[RING];                  // transposed fragments of dO_i / Q_i for the products of C
		f32x4 lse4[4], del4[4];
		f32x16 cstart[2];                 // start values of the chains of S and dP (inline-assembly path)
		float bv[2][BIAS && !BIAS_LDS ? 16 : 1];  // [block parity]: bias values, fetched one stage ahead of their use
		u32x2 bvr[2][BIAS_LDS ? 4 : 1];           // the same from LDS: [block parity][quad], 4 values of 16 bits

		// fragment of product j of A(qb): even j -> Q (S), odd j -> dO (dP), k-step j / 2
		auto issue_A = [&](int qb, int j) __attribute__((always_inline)) {
			// (poff carries the buffer; dO lies one tile behind Q)
			afr[(qb * NSLOT + j) % RING] = *(const FA2_LDS V8*)(lds + poff[(j >> 1) % KR] + ((j >> 1) / KR) * 256 + ((j & 1) ? TILE_BYTES : 0) + qb * (32 * D * 2));
		};
		// fragment of product j of C(qb): half j / (2 DB); inside a half even -> dO^T (dV), odd -> Q^T (dK)
		auto issue_C = [&](int qb, int j) __attribute__((always_inline)) {
			int hf = j / (2 * DB), rr = j % (2 * DB), db = rr >> 1;
			const FA2_LDS char* base = lds + ((rr & 1) ? 0 : TILE_BYTES) + qb * (32 * D * 2);
			cfr[(qb * NSLOT + j) % RING] = lds_tr_issue_rt<D>(base + toff[db % DR][0] + (db / DR) * 256, base + toff[db % DR][1] + (db / DR) * 256, hf);
		};
		// statistics of rows 8 aa + 4 g .. + 3 of block qb
		auto issue_stat = [&](int qb, int aa) __attribute__((always_inline)) {
			lse4[aa] = *(const FA2_LDS f32x4*)(stat + soff + (32 * qb + 8 * aa) * 4);
			if constexpr (!FOLD_DEL) del4[aa] = *(const FA2_LDS f32x4*)(stat + soff + 2 * STAT_BYTES + (32 * qb + 8 * aa) * 4);
		};
		// FOLD_DEL: -delta of rows 8 aa + 4 g .. + 3 of block qb, the start value of its chain of dP (read a stage ahead of the statistics)
		f32x4 cdel4[FOLD_DEL ? 4 : 1];
		auto issue_del = [&](int qb, int aa) __attribute__((always_inline)) {
			if constexpr (FOLD_DEL) cdel4[aa] = *(const FA2_LDS f32x4*)(stat + soff + 2 * STAT_BYTES + (32 * qb + 8 * aa) * 4);
		};
		// statistics of the quads whose phase 0 runs in slot j
		auto issue_stat_for_slot = [&](int qb, int j) __attribute__((always_inline)) {
			if constexpr (NSLOT >= 16) {
				if (j % (NSLOT / 4) == 0) issue_stat(qb, j / (NSLOT / 4));
			} else {
				constexpr int QPS = 16 / NSLOT;
				if (j % 4 == 0)
					for (int e = 0; e < QPS; ++e) issue_stat(qb, (j / 4) * QPS + e);
			}
		};
		auto load_bias = [&](int qb, int i) __attribute__((always_inline)) {
			if constexpr (BIAS && !BIAS_LDS) {
				int row = m0 + 32 * qb + 8 * (i >> 2) + 4 * g + (i & 3);
				row = row < a.Sq ? row : a.Sq - 1;
				const char* pp = bias_base + (int64_t)row * a.bias_sm;
				if (CAP && a.bias == nullptr)
					bv[qb & 1][i] = 0.f;
				else if constexpr (BIAS_T)
					bv[qb & 1][i] = to_f32(*(const typename T::E*)pp);
				else
					bv[qb & 1][i] = a.bias_dtype == 3   ? *(const float*)pp
					                : a.bias_dtype == 2 ? to_f32(*(const __bf16*)pp)
					                : a.bias_dtype == 1 ? (float)*(const _Float16*)pp
					                                    : (*(const uint8_t*)pp ? 0.f : a.mask_fill);
			}
		};
		// bias values of block qb that belong to slot j when the 16 of them are spread over a stage
		auto load_bias_for_slot = [&](int qb, int j) __attribute__((always_inline)) {
			if constexpr (BIAS_LDS) {
				// quad j (rows 8 j + 4 g + e of the block, this lane's key): one transposed read
				if (j < 4) {
					typedef __attribute__((__vector_size__(4 * sizeof(short)))) short v4s;
					v4s x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA2_LDS v4s*)(lds_bias + boffq[j & 1] + (j >> 1) * (16 * 256) + qb * (32 * 256)));
					bvr[qb & 1][j] = __builtin_bit_cast(u32x2, x);
				}
			} else if constexpr (BIAS) {
				if constexpr (NSLOT >= 16) {
					if (j % (NSLOT / 16) == 0) load_bias(qb, j / (NSLOT / 16));
				} else {
#pragma unroll
					for (int e = 0; e < 16 / NSLOT; ++e) load_bias(qb, j * (16 / NSLOT) + e);
				}
			}
		};
		auto mfma_A = [&](int qb, int j, f32x16& sa, f32x16& dpa) __attribute__((always_inline)) {
			int ks = j >> 1, r = (qb * NSLOT + j) % RING;
			if constexpr (KV_AGPR) {
				// the chains start from -lse and -delta of the block's rows (accumulator element i
				// belongs to row 8 (i / 4) + 4 g + i % 4, which is element i % 4 of quarter i / 4)
				if (j == 0) {
					cstart[0] = __builtin_shufflevector(__builtin_shufflevector(lse4[0], lse4[1], 0, 1, 2, 3, 4, 5, 6, 7), __builtin_shufflevector(lse4[2], lse4[3], 0, 1, 2, 3, 4, 5, 6, 7), 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
					mfma32_vc(sa, afr[r], kf[ks], cstart[0]);
				} else if (j == 1) {
					cstart[1] = __builtin_shufflevector(__builtin_shufflevector(del4[0], del4[1], 0, 1, 2, 3, 4, 5, 6, 7), __builtin_shufflevector(del4[2], del4[3], 0, 1, 2, 3, 4, 5, 6, 7), 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
					mfma32_vc(dpa, afr[r], vf[ks], cstart[1]);
				}
				else if (j & 1)
					mfma32_va<true>(dpa, afr[r], vf[ks]);
				else
					mfma32_va<true>(sa, afr[r], kf[ks]);
			} else if constexpr (S_VGPR) {
				if (j == 0)
					mfma32_vz(sa, afr[r], kf[ks]);
				else if (j == 1)
					mfma32_vz(dpa, afr[r], vf[ks]);
				else if (j & 1)
					mfma32_va<false>(dpa, afr[r], vf[ks]);
				else
					mfma32_va<false>(sa, afr[r], kf[ks]);
			} else {
				// too many registers to pin: leave the register files to the compiler
				f32x16 zero;
#pragma unroll
				for (int i = 0; i < 16; ++i) zero[i] = 0.f;
				if (j & 1) {
					f32x16 c0 = zero;
					if constexpr (FOLD_DEL)
						c0 = __builtin_shufflevector(__builtin_shufflevector(cdel4[0], cdel4[1], 0, 1, 2, 3, 4, 5, 6, 7), __builtin_shufflevector(cdel4[2], cdel4[3], 0, 1, 2, 3, 4, 5, 6, 7), 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
					dpa = mfma32(afr[r], vf[ks], j == 1 ? c0 : dpa);
				} else
					sa = mfma32(afr[r], kf[ks], j == 0 ? zero : sa);
			}
		};
		auto mfma_C = [&](int qb, int j, u32x4(&pbi)[2], u32x4(&sbi)[2]) __attribute__((always_inline)) {
			int hf = j / (2 * DB), rr = j % (2 * DB), db = rr >> 1, r = (qb * NSLOT + j) % RING;
			if constexpr (KV_AGPR) {
				if (rr & 1)
					mfma32_aa(dk[db], as_frag<T>(cfr[r]), as_frag<T>(sbi[hf]));
				else
					mfma32_aa(dv[db], as_frag<T>(cfr[r]), as_frag<T>(pbi[hf]));
			} else {
				if (rr & 1)
					dk[db] = mfma32(as_frag<T>(cfr[r]), as_frag<T>(sbi[hf]), dk[db]);
				else
					dv[db] = mfma32(as_frag<T>(cfr[r]), as_frag<T>(pbi[hf]), dv[db]);
			}
		};
		// B(qb) as 16 micro-steps: quad q (values 4q .. 4q+3, rows 8q + 4g + e) goes through
		//   phase 0: x = S c1 - lse, y = dP - delta     phase 1: P = exp2(x) (mask, dropout)
		//   phase 2: dS = P y                            phase 3: pack P and dS to 16 bits
		// Every micro-step is four independent operations per instruction kind, and the phases
		// of a quad sit in different slots: a vector-ALU result is only consumed many cycles
		// after it was issued (back-to-back dependent vector operations would each wait for
		// the previous one's full pipeline latency).
		float bx[4][4], by[4][4];
		float bt[4][4];  // CAP: tanh of the scaled score, for the factor 1 - tanh^2 of its derivative
		// dropout keep bits of a quad (bit e = value 4q + e), produced while the previous quad is processed.
		// One generator call yields the values of 2 adjacent rows x 4 adjacent keys, and the 4 lanes of a
		// DPP quad hold 4 adjacent keys: one call per lane covers the 2 x 4 rows of the quads q and q + 1 (q even) -
		// lane t evaluates the rows 2 (t & 1), 2 (t & 1) + 1 of quad q + t / 2, reduces its 8 values to 8 keep bits
		// (bit = value index = 4 (row & 1) + (key & 3)), and the quad exchanges them (DPP broadcasts).  The call is
		// cut into 4 parts (rounds 0-2, 3-5, 6-7, 8-9 + exchange) that run in the four micro-step slots of the
		// quad before q; the odd quads' slots stay free of generator work.
		uint32_t keepw[4] = {0u, 0u, 0u, 0u};
		uint32_t phs[2][4];
		auto keep_bit = [&](int qb, int q, int part, int u = 0) __attribute__((always_inline)) {
			if constexpr (DROP) {
				if (q & 1) return;
				uint32_t(&cs)[4] = phs[u];
				if (part == 0) {
					const int t = c & 3;
					cs[0] = (uint32_t)(jcol >> 2);
					cs[1] = (uint32_t)((m0 + 32 * qb + 8 * (q + (t >> 1)) + 4 * g + 2 * (t & 1)) >> 1);
					cs[2] = (uint32_t)hq;
					cs[3] = (uint32_t)b;
					philox4x32_rounds<0, 3>(cs, drop_k0, drop_k1);
				} else if (part == 1) {
					philox4x32_rounds<3, 6>(cs, drop_k0, drop_k1);
				} else if (part == 2) {
					philox4x32_rounds<6, 8>(cs, drop_k0, drop_k1);
				} else {
					philox4x32_rounds<8, 10>(cs, drop_k0, drop_k1);
					uint32_t mine = 0;
#pragma unroll
					for (int v = 0; v < 8; ++v) mine |= keep16(cs[v >> 1], v & 1, a.drop_thr) ? (1u << v) : 0u;
					// rows e = 0, 1 of quad q were evaluated by lane 0 of the quad, e = 2, 3 by lane 1; quad q + 1: lanes 2, 3
					uint32_t r0 = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0x00, 0xf, 0xf, false);
					uint32_t r1 = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0x55, 0xf, 0xf, false);
					uint32_t r2 = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0xaa, 0xf, 0xf, false);
					uint32_t r3 = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0xff, 0xf, 0xf, false);
					const uint32_t sh = (uint32_t)(c & 3);  // this lane's key among the call's four
					keepw[q & 3] = ((r0 >> sh) & 1u) | (((r0 >> (4 + sh)) & 1u) << 1) | (((r1 >> sh) & 1u) << 2) | (((r1 >> (4 + sh)) & 1u) << 3);
					keepw[(q + 1) & 3] = ((r2 >> sh) & 1u) | (((r2 >> (4 + sh)) & 1u) << 1) | (((r3 >> sh) & 1u) << 2) | (((r3 >> (4 + sh)) & 1u) << 3);
				}
			}
		};
		auto micro_B = [&](int qb, int q, int phase, int e0, int e1, const f32x16& sa, const f32x16& dpa, u32x4(&pbo)[2], u32x4(&sbo)[2])
		                   __attribute__((always_inline)) {
			if constexpr (FOLD) {
				// the accumulators already hold q.k - lse / (scale log2(e)) and dP - delta
				if (phase == 0) {
#pragma unroll
					for (int e = e0; e < e1; ++e) bx[q][e] = sa[4 * q + e] * c1;
				} else if (phase == 1) {
#pragma unroll
					for (int e = e0; e < e1; ++e) {
						float p = exp2_fast(bx[q][e]);
						if constexpr (MASKED) {
							int row = m0 + 32 * qb + 8 * q + 4 * g + e;
							bool ok = (row >= row_lo) & (row <= row_hi);  // (no short-circuit: that would be a divergent branch per value)
							p = ok ? p : 0.f;
						}
						bx[q][e] = p;
					}
				} else if (phase == 2) {
#pragma unroll
					for (int e = e0; e < e1; ++e) by[q][e] = bx[q][e] * dpa[4 * q + e];
				} else if (phase == 3) {
					int hf = q >> 1, m = (q & 1) * 2;
#pragma unroll
					for (int e = e0; e < e1; e += 2) {
						pbo[hf][m + e / 2] = pack2<typename T::V2>(bx[q][e], bx[q][e + 1]);
						sbo[hf][m + e / 2] = pack2<typename T::V2>(by[q][e], by[q][e + 1]);
					}
				}
			} else if (phase == 0) {
#pragma unroll
				for (int e = e0; e < e1; ++e) {
					int i = 4 * q + e;
					if constexpr (BIAS)
						if constexpr (BIAS_LDS) {
							float bvl = to_f32x4(__builtin_bit_cast(typename T::V4, bvr[qb & 1][q]))[e];
							bx[q][e] = __builtin_fmaf(__builtin_fmaf(sa[i], c1, bvl), kLog2e, lse4[q][e]);
						} else if constexpr (CAP) {
							bt[q][e] = tanh_fast(sa[i] * a.cap_k1);
							bx[q][e] = __builtin_fmaf(__builtin_fmaf(bt[q][e], a.softcap, bv[qb & 1][i]), kLog2e, lse4[q][e]);
						} else {
							bx[q][e] = __builtin_fmaf(__builtin_fmaf(sa[i], c1, bv[qb & 1][i]), kLog2e, lse4[q][e]);
						}
					else
						bx[q][e] = __builtin_fmaf(sa[i], c1, lse4[q][e]);
				}
			} else if (phase == 1) {
#pragma unroll
				for (int e = e0; e < e1; ++e) {
					// dP is read here, not in phase 0: the last product of its chain is then at
					// least two matrix products back
					if constexpr (!DROP) by[q][e] = FOLD_DEL ? dpa[4 * q + e] : dpa[4 * q + e] - del4[q][e];
					float p = exp2_fast(bx[q][e]);
					int row = m0 + 32 * qb + 8 * q + 4 * g + e;
					if constexpr (MASKED) {
						bool ok = (row >= row_lo) & (row <= row_hi);  // (no short-circuit: that would be a divergent branch per value)
						p = ok ? p : 0.f;
					}
					bx[q][e] = p;
					if constexpr (DROP) {
						bool keep = (keepw[q & 3] >> e) & 1u;
						// by = dP keep / (1 - p_drop) - delta ; bx keeps P, the dropped P goes to dV
						by[q][e] = keep ? __builtin_fmaf(dpa[4 * q + e], a.drop_inv_keep, -del4[q][e]) : -del4[q][e];
						bx[q][e] = keep ? p : -p;  // sign bit marks a dropped value (P >= 0)
					}
				}
			} else if (phase == 2) {
#pragma unroll
				for (int e = e0; e < e1; ++e) {
					by[q][e] = __builtin_fabsf(bx[q][e]) * by[q][e];
					if constexpr (CAP) by[q][e] *= __builtin_fmaf(-bt[q][e], bt[q][e], 1.f);
				}
			} else {
				int hf = q >> 1, m = (q & 1) * 2;
#pragma unroll
				for (int e = e0; e < e1; e += 2) {
					float p0 = bx[q][e], p1 = bx[q][e + 1];
					if constexpr (DROP) {
						p0 = p0 < 0.f ? 0.f : p0;
						p1 = p1 < 0.f ? 0.f : p1;
					}
					pbo[hf][m + e / 2] = pack2<typename T::V2>(p0, p1);
					sbo[hf][m + e / 2] = pack2<typename T::V2>(by[q][e], by[q][e + 1]);
				}
			}
		};

		// reads that the first PA slots of stage 0 use
#pragma unroll
		for (int j = 0; j < PA; ++j) issue_A(0, j);
		if constexpr (FOLD) {
#pragma unroll
			for (int aa = 0; aa < 4; ++aa) issue_stat(0, aa);
		}
		if constexpr (FOLD_DEL) {
#pragma unroll
			for (int aa = 0; aa < 4; ++aa) issue_del(0, aa);
		}

		auto stage = [&](auto k_tag) __attribute__((always_inline)) {
			constexpr int k = decltype(k_tag)::value;
			constexpr bool HAS_A = k < QB, HAS_B = k >= 1 && k - 1 < QB, HAS_C = k >= 2 && k - 2 < QB;
			constexpr bool NEXT_A = k + 1 < QB, NEXT_B = k + 1 >= 1 && k < QB, NEXT_C = k + 1 >= 2 && k - 1 < QB;
			// One row block per step (head dim 256): nothing else is in flight, so the products of C start half a stage
			// early - those of the block's first 16 rows (its slots 0 .. H - 1) run beside the elementwise math of its last
			// 16 rows in the second half of stage 1, the rest in a stage 2 of half the length.
			constexpr bool HALF = QB == 1;
			constexpr int H = NSLOT / 2;
			constexpr int NS = (HALF && k == 2) ? H : NSLOT;
			__builtin_amdgcn_sched_barrier(0);
			// (a stage that starts with the elementwise math of a block whose last products - inline assembly - were the
			// previous stage's last instructions: their results need their wait states)
			if constexpr (S_VGPR && HAS_B && !HAS_A) asm volatile("s_nop 15" ::: "memory");
#pragma unroll
			for (int j = 0; j < NS; ++j) {
				// this slot's product of C, if any: block and slot index within that block's C
				const bool has_c = HALF ? ((k == 1 && j >= H) || k == 2) : HAS_C;
				const int cblk = HALF ? 0 : k - 2, jc = HALF ? (k == 1 ? j - H : j + H) : j;
				// LDS reads for the slot PA places ahead (in this stage or the next one)
				{
					int jn = j + PA;
					if (jn < NSLOT) {
						if constexpr (HAS_A) issue_A(k, jn);
						if constexpr (HAS_C && !HALF) issue_C(k - 2, jn);
						if constexpr (HAS_B && !FOLD) {
							issue_stat_for_slot(k - 1, jn);
						}
					} else {
						int jj = jn - NSLOT;
						if constexpr (NEXT_A) issue_A(k + 1, jj);
						if constexpr (NEXT_C && !HALF) issue_C(k - 1, jj);
						if constexpr (NEXT_B && !FOLD) {
							issue_stat_for_slot(k, jj);
						}
					}
					if constexpr (HALF && k >= 1) {
						// (stage 1 slot t is slot t - H of C, stage 2 slot t is slot t + H)
						int cn = k == 1 ? j + PA - H : j + PA + H;
						if (cn >= 0 && cn < NSLOT) issue_C(0, cn);
					}
					// the start values of the chains of the next block, in the last four slots
					if constexpr (FOLD && NEXT_A) {
						if (j >= NSLOT - 4) issue_stat(k + 1, j - (NSLOT - 4));
					}
					if constexpr (FOLD_DEL && NEXT_A) {
						if (j >= NSLOT - 4) issue_del(k + 1, j - (NSLOT - 4));
					}
				}
				// first half of the slot: product of A, first half of the micro-step(s) of B;
				// second half: product of C, second half of the micro-step(s) - each matrix
				// product is followed by vector-ALU work, never directly by another product
				auto b_half = [&](int e0, int e1) __attribute__((always_inline)) {
					if constexpr (HAS_B) {
						if constexpr (NSLOT >= 16) {
							if (j % (NSLOT / 16) == NSLOT / 16 - 1) {
								int ms = j / (NSLOT / 16);
								micro_B(k - 1, ms / 4, ms % 4, e0, e1, s[(k - 1) & 1], dp[(k - 1) & 1], pbits[(k - 1) & 1], sbits[(k - 1) & 1]);
							}
						} else {
							// several quads share a slot, all in the same phase
							constexpr int QPS = 16 / NSLOT;  // quads per slot
							int grp = j / 4, phase = j % 4;
#pragma unroll
							for (int e = 0; e < QPS; ++e) {
								int q = grp * QPS + e;
								micro_B(k - 1, q, phase, e0, e1, s[(k - 1) & 1], dp[(k - 1) & 1], pbits[(k - 1) & 1], sbits[(k - 1) & 1]);
							}
						}
					}
				};
				// bias of the block whose elementwise stage comes next
				if constexpr (NEXT_B) load_bias_for_slot(k, j);
				if constexpr (HAS_A) mfma_A(k, j, s[k & 1], dp[k & 1]);
				// A matrix product reads its C operand while it runs, and the hardware does not hold back a
				// vector-ALU write to those registers; for the products issued as inline assembly the compiler
				// does not either.  The start values of the two chains (the only C operands that are not also
				// the destination) therefore stay allocated until two further products have been issued.
				if constexpr (HAS_A && KV_AGPR) {
					if (j == 2) asm volatile("; chain start of S still allocated" ::"v"(cstart[0]));
					if (j == 3) asm volatile("; chain start of dP still allocated" ::"v"(cstart[1]));
				}
				// the vector-ALU work below must not move above the product: for the products
				// issued as inline assembly that order is what keeps a read of S / dP at least
				// two matrix products away from the last product of its chain
				if constexpr (HAS_A && HAS_B) __builtin_amdgcn_sched_barrier(0);
				b_half(0, 2);
				if constexpr (HAS_A && HAS_C) __builtin_amdgcn_sched_barrier(0);
				if constexpr (HAS_C || (HALF && k >= 1)) {
					if (has_c) mfma_C(cblk, jc, pbits[HALF ? 0 : (k & 1)], sbits[HALF ? 0 : (k & 1)]);
				}
				b_half(2, 4);
				if constexpr (HAS_B && DROP) {
					if constexpr (NSLOT >= 16) {
						if (j % (NSLOT / 16) == NSLOT / 16 - 1) {
							int ms = j / (NSLOT / 16);
							if (ms + 4 < 16) keep_bit(k - 1, (ms + 4) / 4, ms % 4);
						}
					} else {
						constexpr int QPS = 16 / NSLOT;
						for (int e = 0; e < QPS; ++e) {
							int q = (j / 4) * QPS + e;
							if (q + QPS < 4) keep_bit(k - 1, q + QPS, j % 4, e);
						}
					}
				}
				if constexpr (NEXT_B && DROP) {
					// keep bits of the first quad(s) of the next block, in the last slots of this stage
					if constexpr (NSLOT >= 16) {
						if (j >= NSLOT - 4 * (NSLOT / 16) && (j - (NSLOT - 4 * (NSLOT / 16))) % (NSLOT / 16) == 0)
							keep_bit(k, 0, (j - (NSLOT - 4 * (NSLOT / 16))) / (NSLOT / 16));
					} else {
						if (j >= NSLOT - 4)
							for (int e = 0; e < 16 / NSLOT; ++e) keep_bit(k, e, j - (NSLOT - 4), e);
					}
				}
				__builtin_amdgcn_sched_barrier(0);
			}
		};
		stage(std::integral_constant<int, 0>{});
		stage(std::integral_constant<int, 1>{});
		stage(std::integral_constant<int, 2>{});
		if constexpr (QB + 1 >= 3) stage(std::integral_constant<int, 3>{});
		if constexpr (QB + 1 >= 4) stage(std::integral_constant<int, 4>{});
		if constexpr (QB + 1 >= 5) stage(std::integral_constant<int, 5>{});
		static_assert(QB <= 4, "");
	};

	// (q-head, first row) of the streamed tile the next step computes on: decoded once, when its copies are started
	int cur_hq = 0, cur_m0 = 0;
	if (s_hi > s_lo) {
		decode_step(s_lo, cur_hq, cur_m0);
		issue_tile(s_lo, tile_base(cur_hq, cur_m0), cur_m0, lds, lds + TILE_BYTES);
		store_stat(fetch_stat(cur_hq, cur_m0), 0);
	}

	// One pipeline step: publish streamed tile `step`, start the copies of the next, compute.
	auto run_step = [&](auto masked_tag, int step) {
		const int buf = (step - s_lo) & 1;
		wait_async_loads();
		__syncthreads();
		float next_stat = 0.f;
		int nxt_hq = 0, nxt_m0 = 0;
		const bool has_next = step + 1 < s_hi;
		if (has_next) {
			// statistics first: loads return in order, so waiting for this small load later
			// does not wait for the tile copies issued after it
			decode_step(step + 1, nxt_hq, nxt_m0);
			const TileBase tb = tile_base(nxt_hq, nxt_m0);
			next_stat = fetch_stat(nxt_hq, nxt_m0);
			issue_tile(step + 1, tb, nxt_m0, lds + (buf ^ 1) * (2 * TILE_BYTES), lds + (buf ^ 1) * (2 * TILE_BYTES) + TILE_BYTES);
		}
		{
			const int hq = cur_hq, m0 = cur_m0;
			bool skip = false;
			if constexpr (decltype(masked_tag)::value) {
				// wave-uniform: nothing to do for (rows m0.., keys wn0..)?
				int last_row = m0 + BMQ - 1 < sq_eff - 1 ? m0 + BMQ - 1 : sq_eff - 1;
				skip = wn0 >= sk_eff || (wr >= 0 && wn0 > last_row + off + wr) || (wl >= 0 && wn0 + 31 < m0 + off - wl);
			}
			if (!skip) tile_body(masked_tag, hq, m0);
		}
		// the other buffers next time
#pragma unroll
		for (int ks = 0; ks < KR; ++ks) poff[ks] ^= 2 * TILE_BYTES;
#pragma unroll
		for (int db = 0; db < DR; ++db) {
			toff[db][0] ^= 2 * TILE_BYTES;
			toff[db][1] ^= 2 * TILE_BYTES;
		}
		soff ^= STAT_BYTES;
		if constexpr (BIAS_LDS) {
			boffq[0] ^= BIAS_BYTES;
			boffq[1] ^= BIAS_BYTES;
		}
		if (has_next) store_stat(next_stat, buf ^ 1);
		cur_hq = nxt_hq;
		cur_m0 = nxt_m0;
		// The load of the statistics has completed on every path out of the step.  Without this use the compiler
		// takes the load for possibly still in flight at the top of the next step (it cannot tell that the two
		// `has_next` tests agree) and guards the first reuse of its register there with s_waitcnt vmcnt(0) - which
		// on the hardware waits for the tile copies that were just started.
		asm volatile("; statistics of the next tile present" ::"v"(next_stat));
	};
	// Per q-head the streamed tiles are: tiles crossing this wave's causal diagonal / the window's
	// right edge (masked), tiles entirely inside (no mask), and tiles on the window's left edge or a
	// ragged last tile (masked).
	// The unmasked tiles run in a loop of their own so that the steady state is a
	// single straight-line body.
	int i_diag = 0;  // first tile index (relative to q_lo) with no causal / right-edge masking for this wave
	if (wr >= 0) {
		int first_clear = wn0 + 31 - off - wr;  // rows >= this see all 32 keys of the wave
		int tq = first_clear > 0 ? (first_clear + BMQ - 1) / BMQ : 0;
		i_diag = tq - q_lo;
	}
	int i_full = sq_eff / BMQ - q_lo;  // tiles before this one lie entirely inside the valid rows
	if (wl >= 0) {
		// ... and entirely inside the left edge of the window: rows <= wn0 - off + win_left see even the wave's first key
		int last_clear = wn0 - off + wl;
		int e = last_clear >= 0 ? (last_clear + 1) / BMQ - q_lo : 0;
		i_full = e < i_full ? e : i_full;
	}
	if (wn0 + 32 > sk_eff) i_diag = nq;  // ragged key block: always masked
	i_diag = i_diag < 0 ? 0 : (i_diag > nq ? nq : i_diag);
	i_full = i_full < i_diag ? i_diag : (i_full > nq ? nq : i_full);
	if (order == 0) {
		for (int hi = 0; hi < r && nq > 0; ++hi) {
			// (each of the three runs clipped to this workgroup's share of the steps)
			int base = hi * nq;
			auto clip = [&](int i) { int st = base + i; return st < s_lo ? s_lo : (st > s_hi ? s_hi : st); };
			for (int st = clip(0); st < clip(i_diag); ++st) run_step(std::true_type{}, st);
			for (int st = clip(i_diag); st < clip(i_full); ++st) run_step(std::false_type{}, st);
			for (int st = clip(i_full); st < clip(nq); ++st) run_step(std::true_type{}, st);
		}
	} else {
		// query tiles outermost: the same three runs, r steps per query tile, in the direction of the walk
		const int pa = (order == 2 ? nq - i_full : i_diag) * r, pb = (order == 2 ? nq - i_diag : i_full) * r;
		auto clip = [&](int st) { return st < s_lo ? s_lo : (st > s_hi ? s_hi : st); };
		for (int st = clip(0); st < clip(pa); ++st) run_step(std::true_type{}, st);
		for (int st = clip(pa); st < clip(pb); ++st) run_step(std::false_type{}, st);
		for (int st = clip(pb); st < clip(steps); ++st) run_step(std::true_type{}, st);
	}

	// the last matrix products (issued as inline assembly) must have written dk / dv
	asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
	// epilogue: lane owns key jcol, four consecutive d per store
	if (hsplit > 1) {
		// partial sums over this workgroup's share of the steps, fp32 and unscaled, for the reduce kernel
		if (jcol < a.Sk) {
			float* pp = a.dkv_part + ((((int64_t)hsi * a.B + b) * a.Hkv + hk) * a.Sk + jcol) * (2 * D);
#pragma unroll
			for (int db = 0; db < DB; ++db)
#pragma unroll
				for (int aa = 0; aa < 4; ++aa) {
					int d0 = 32 * db + 8 * aa + 4 * g;
					*(f32x4*)(pp + d0) = f32x4{dk[db][4 * aa], dk[db][4 * aa + 1], dk[db][4 * aa + 2], dk[db][4 * aa + 3]};
					*(f32x4*)(pp + D + d0) = f32x4{dv[db][4 * aa], dv[db][4 * aa + 1], dv[db][4 * aa + 2], dv[db][4 * aa + 3]};
				}
		}
		return;
	}
	if (jcol < a.Sk) {
		char* dkp = a.dk.ptr + (int64_t)b * a.dk.sb + (int64_t)hk * a.dk.sh + (int64_t)jcol * a.dk.ss;
		char* dvp = a.dv.ptr + (int64_t)b * a.dv.sb + (int64_t)hk * a.dv.sh + (int64_t)jcol * a.dv.ss;
		const float ks_ = a.scale;
		const float vs_ = DROP ? a.drop_inv_keep : 1.f;
#pragma unroll
		for (int db = 0; db < DB; ++db)
#pragma unroll
			for (int aa = 0; aa < 4; ++aa) {
				int d0 = 32 * db + 8 * aa + 4 * g;
				u32x2 pk = {pack2<typename T::V2>(dk[db][4 * aa] * ks_, dk[db][4 * aa + 1] * ks_),
				            pack2<typename T::V2>(dk[db][4 * aa + 2] * ks_, dk[db][4 * aa + 3] * ks_)};
				*(u32x2*)(dkp + d0 * 2) = pk;
				u32x2 pv = {pack2<typename T::V2>(dv[db][4 * aa] * vs_, dv[db][4 * aa + 1] * vs_),
				            pack2<typename T::V2>(dv[db][4 * aa + 2] * vs_, dv[db][4 * aa + 3] * vs_)};
				*(u32x2*)(dvp + d0 * 2) = pv;
			}
	}
}

// blockIdx.x -> (key tile or pair of key tiles, kv head, batch); the key tiles of one (b, kv head) stay on one XCD.
// BIAS_T: the bias has the element type of q / k / v (no run-time type dispatch per value)
// CAP: tanh soft-capping of the scores (see the forward kernel); the bias itself may then be absent
// PAIR: the instantiation for launches that give a workgroup two key tiles (a.kv_pair); the launcher picks it only then,
// so that every other launch runs the kernel with the one walk as a compile-time constant.
template <typename T, int D, int NW, int QB, bool BIAS, bool DROP, bool BIAS_T, bool CAP = false, bool PAIR = false>
__global__ __launch_bounds__(NW * 64) void bwd_dkdv_kernel(const KArgs a) {
	// (with the steps of a key tile split over workgroups: the parts of one key tile are adjacent)
	int hk, b, within;
	const int hsplit = a.kv_hsplit > 1 ? a.kv_hsplit : 1;
	const int hsi = hsplit > 1 ? (int)blockIdx.x % hsplit : 0;
	{
		int id = hsplit > 1 ? (int)blockIdx.x / hsplit : (int)blockIdx.x;
		int per_group = a.mtiles;
		int grp;
		if (a.xcd_remap >= 2) {
			// bias shared by the heads: one batch per XCD, the kv-heads of one key tile adjacent
			int xcd = id & 7, j = id >> 3;
			int per_batch = per_group * a.Hkv;
			int rem = j % per_batch;
			grp = ((j / per_batch) * 8 + xcd) * a.Hkv + rem % a.Hkv;
			within = rem / a.Hkv;
			if (a.xcd_remap == 3) {
				// batch rows of different key lengths: the units (batch, key tile) of one batch go round the XCDs
				int u = j / a.Hkv, nb8 = a.B >> 3;
				within = u / nb8;
				grp = (((xcd - within) & 7) + 8 * (u % nb8)) * a.Hkv + j % a.Hkv;
			}
		} else if (a.xcd_remap) {
			int xcd = id & 7, j = id >> 3;
			// a.interleave = e groups of an XCD advance together: e adjacent workgroups are the same key tile (see launch_order())
			int e = a.interleave;
			int sgi = j / (e * per_group), rem = j % (e * per_group);
			grp = (sgi * e + rem % e) * 8 + xcd;
			within = rem / e;
		} else {
			grp = id / per_group;
			within = id % per_group;
		}
		hk = grp % a.Hkv;
		b = grp / a.Hkv;
	}
	const DkdvRow rw = dkdv_row<DROP>(a, b);
	if constexpr (!PAIR) {
		// one key tile, head by head (early key tiles see the most query rows under a causal mask: first)
		bwd_dkdv_tile<T, D, NW, QB, BIAS, DROP, BIAS_T, CAP, false>(a, within, hk, b, hsi, hsplit, 0, 0, rw);
	} else {
		// Causal self-attention: key tile p streams every query tile from p up, so a workgroup takes tile p and tile
		// ntiles - 1 - p one after the other - every workgroup then has the same number of steps (no CU waits for the
		// longest tile, no gaps in the dispatch), and the two walks are arranged so that all workgroups of a KV group
		// stay together: the long tile runs from the last query tile DOWN (all workgroups start at the same tile and
		// drop out one by one), the short tile from its diagonal UP (a workgroup that has finished tile p, one query
		// tile later than the workgroup of p + 1, joins that workgroup's second walk exactly where it is now).  At any
		// time the KV group reads two fronts of Q / dO tiles, not one per workgroup.
		const int r = a.Hq / a.Hkv;
		const int partner = a.kv_ntiles - 1 - within;
		// (an odd number of tiles: the middle one is its own partner)
		const int npass = partner != within ? 2 : 1;
		const int rot = within % r;
		for (int pass = 0; pass < npass; ++pass) {
			bwd_dkdv_tile<T, D, NW, QB, BIAS, DROP, BIAS_T, CAP, true>(a, pass == 0 ? within : partner, hk, b, 0, 1, 2 - pass, rot, rw);
			// (the LDS buffers of the first tile are free once every wave has left its last step)
			if (pass + 1 < npass) __syncthreads();
		}
	}
}

// Sum of the partial dK / dV that a dK/dV launch with split steps left (a.dkv_part, see KArgs), scaled and stored in the
// element type: one thread per (batch, kv-head, key, dK | dV, eight consecutive d).
template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_dkdv_reduce_kernel(const KArgs a, float dk_scale, float dv_scale) {
	constexpr int CH = D / 8;  // chunks of eight per row
	int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	int64_t total = (int64_t)a.B * a.Hkv * a.Sk * 2 * CH;
	if (idx >= total) return;
	int ch = (int)(idx % CH);
	int which = (int)((idx / CH) % 2);
	int64_t row = idx / (2 * CH);  // (b * Hkv + hk) * Sk + key
	int key = (int)(row % a.Sk);
	int hk = (int)((row / a.Sk) % a.Hkv);
	int b = (int)(row / ((int64_t)a.Sk * a.Hkv));
	const int64_t part_stride = (int64_t)a.B * a.Hkv * a.Sk * 2 * D;
	const float* pp = a.dkv_part + row * (2 * D) + which * D + ch * 8;
	float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
	for (int s = 0; s < a.kv_hsplit; ++s) {
		f32x4 x0 = *(const f32x4*)(pp + s * part_stride), x1 = *(const f32x4*)(pp + s * part_stride + 4);
#pragma unroll
		for (int e = 0; e < 4; ++e) {
			acc[e] += x0[e];
			acc[4 + e] += x1[e];
		}
	}
	const float sc = which ? dv_scale : dk_scale;
	const KTensor& out = which ? a.dv : a.dk;
	u32x4 pk = {pack2<typename T::V2>(acc[0] * sc, acc[1] * sc), pack2<typename T::V2>(acc[2] * sc, acc[3] * sc),
	            pack2<typename T::V2>(acc[4] * sc, acc[5] * sc), pack2<typename T::V2>(acc[6] * sc, acc[7] * sc)};
	char* op_ = out.ptr + (int64_t)b * out.sb + (int64_t)hk * out.sh + (int64_t)key * out.ss + ch * 16;
	// (rows of dk / dv need not be 16-byte aligned: two 8-byte stores)
	*(u32x2*)op_ = u32x2{pk[0], pk[1]};
	*(u32x2*)(op_ + 8) = u32x2{pk[2], pk[3]};
}

// ---------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------
// BLDS: the bias goes through LDS as in the forward kernel (conditions checked by the launcher)
// DBIAS: also writes the gradient of the additive term (a.dbias); on the plain path with bias
template <typename T, int D, int NW, int QB, int WPS, bool BIAS, bool DROP, bool BLDS = false, bool CAP = false, bool DBIAS = false>
__global__ __launch_bounds__(NW * 64, WPS) void bwd_dq_kernel(const KArgs a) {
	static_assert(!CAP || (BIAS && !BLDS), "soft-capping runs on the plain path with bias");
	static_assert(!DBIAS || (BIAS && !BLDS), "the bias gradient is written on the plain path with bias");
	typedef typename T::V8 V8;
	constexpr int BM = NW * QB * 32;
	constexpr int BN = kFwdBN;
	constexpr int KB = BN / 32;
	constexpr int KS = D / 16;
	constexpr int DB = D / 32;
	constexpr int NT = NW * 64;
	constexpr int TILE_BYTES = BN * D * 2;

	// bias tiles through LDS as in the forward kernel
	constexpr bool BIAS_LDS = BIAS && BLDS;
	constexpr int BIAS_BYTES = BIAS_LDS ? BM * BN * 2 : 0;
	static_assert(BN == 64, "bias tiles use the 64-element row geometry");
	__shared__ __attribute__((aligned(1024))) char smem[4 * TILE_BYTES + 2 * BIAS_BYTES];
	FA2_LDS char* lds = (FA2_LDS char*)smem;

	int mt, h, b;
	decode_block(a, mt, h, b);
	const int hk = h / (a.Hq / a.Hkv);
	const int tid = threadIdx.x, lane = tid & 63;
	// the wave index as an explicitly scalar value: everything derived from it (tile bounds, loop trip counts,
	// "nothing to do for this wave") then stays in scalar registers and scalar branches
	const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, c = lane & 31;
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
	const int off = sk_eff - sq_eff;
	if (a.kv_lens) {  // key padding only: the causal alignment keeps counting from the full key count
		int len = a.kv_lens[b];
		len = len < 0 ? 0 : len;
		sk_eff = len < sk_eff ? len : sk_eff;
	}
	const int m0 = mt * BM;
	const int wm0 = m0 + w * (QB * 32);

	// row i may look at keys i + off - win_left .. i + off + win_right (each bound only when >= 0; causal is win_right = 0)
	const int wr = a.win_right, wl = a.win_left;
	constexpr int kNoKey = -(1 << 30);
	int kv_end = sk_eff;
	if (wr >= 0) {
		int last_row = (m0 + BM - 1 < sq_eff - 1) ? m0 + BM - 1 : sq_eff - 1;
		int e = last_row + off + wr + 1;
		kv_end = e < kv_end ? e : kv_end;
	}
	if (m0 >= sq_eff) kv_end = 0;
	int t_begin = 0;
	if (wl >= 0) {
		int first_key = m0 + off - wl;  // first key the tile's first row sees
		if (first_key > 0) t_begin = first_key / BN;
	}
	const int ntiles = kv_end > 0 ? (kv_end + BN - 1) / BN : 0;

	int jmax[QB], jmin[QB], qrow[QB];
	float lse_r[QB], del_r[QB];
#pragma unroll
	for (int qb = 0; qb < QB; ++qb) {
		int i = wm0 + 32 * qb + c;
		qrow[qb] = i;
		int jm = sk_eff - 1;
		if (wr >= 0) jm = (i + off + wr < jm) ? i + off + wr : jm;
		if (i >= sq_eff) jm = -1;
		jmax[qb] = jm;
		jmin[qb] = wl >= 0 ? i + off - wl : kNoKey;
		int ic = i < a.Sq ? i : a.Sq - 1;
		int64_t idx = ((int64_t)b * a.Hq + h) * a.Sq + ic;
		float l = a.lse[idx];
		// rows without any allowed key carry lse = -inf; their P is forced to 0 by the mask
		// the addend of the fused multiply-add that forms the exponent, (x - lse) log2(e) = x log2(e) - lse log2(e); kept finite
		// for a row whose keys all carry the finfo.min "mask" bias of the bf16 type (lse = -3.39e38: its P underflows to 0)
		lse_r[qb] = __builtin_fminf(-l * kLog2e, 3.0e38f);
		del_r[qb] = a.delta[idx];
	}
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
	}

	const char* kbase = a.k.ptr + (int64_t)b * a.k.sb + (int64_t)hk * a.k.sh;
	const char* vbase = a.v.ptr + (int64_t)b * a.v.sb + (int64_t)hk * a.v.sh;
	TileLoader<D, BN, NT> kload, vload;
	kload.init(a.k.ss, tid);
	vload.init(a.v.ss, tid);
	if (ntiles > t_begin) {
		int nb = t_begin * BN, bsel = t_begin & 1;
		int rows = sk_eff - nb < BN ? sk_eff - nb : BN;
		kload.load(lds + bsel * TILE_BYTES, kbase + (int64_t)nb * a.k.ss, a.k.ss, rows, tid);
		vload.load(lds + (2 + bsel) * TILE_BYTES, vbase + (int64_t)nb * a.v.ss, a.v.ss, rows, tid);
	}

	V8 qf[QB][KS], dof[QB][KS];
	{
		const char* qbase = a.q.ptr + (int64_t)b * a.q.sb + (int64_t)h * a.q.sh;
		const char* dbase = a.dout.ptr + (int64_t)b * a.dout.sb + (int64_t)h * a.dout.sh;
#pragma unroll
		for (int qb = 0; qb < QB; ++qb) {
			int i = qrow[qb] < a.Sq ? qrow[qb] : a.Sq - 1;
			const char* rp = qbase + (int64_t)i * a.q.ss + g * 16;
			const char* dp_ = dbase + (int64_t)i * a.dout.ss + g * 16;
#pragma unroll
			for (int ks = 0; ks < KS; ++ks) {
				qf[qb][ks] = *(const V8*)(rp + ks * 32);
				dof[qb][ks] = *(const V8*)(dp_ + ks * 32);
			}
		}
	}
	// Whole backward in one call: delta = rowsum(O * dO) of the lane's row is formed here from
	// the dO fragments already in registers (each half-wave holds half of the row) and left
	// in scratch for the dK/dV kernel, which is launched after this one; the separate
	// pre-pass (`_attn_bwd_preprocess`, _backward_triton.py:79-147) is then not launched.
	if (a.dq_makes_delta) {
		const char* obase_ = a.o.ptr + (int64_t)b * a.o.sb + (int64_t)h * a.o.sh;
#pragma unroll
		for (int qb = 0; qb < QB; ++qb) {
			int i = qrow[qb] < a.Sq ? qrow[qb] : a.Sq - 1;
			const char* op_ = obase_ + (int64_t)i * a.o.ss + g * 16;
			float acc4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
			for (int ks = 0; ks < KS; ++ks) {
				V8 ov = *(const V8*)(op_ + ks * 32);
#pragma unroll
				for (int e = 0; e < 8; ++e) acc4[e & 3] += (float)ov[e] * (float)dof[qb][ks][e];
			}
			float d = pair_sum((acc4[0] + acc4[1]) + (acc4[2] + acc4[3]));
			del_r[qb] = d;
			if (g == 0 && qrow[qb] < a.Sq) a.delta[((int64_t)b * a.Hq + h) * a.Sq + qrow[qb]] = d;
		}
	}

	f32x16 dq[QB][DB];
#pragma unroll
	for (int qb = 0; qb < QB; ++qb)
#pragma unroll
		for (int db = 0; db < DB; ++db)
#pragma unroll
			for (int i = 0; i < 16; ++i) dq[qb][db][i] = 0.f;
	// Without dropout the chain of dP starts from -delta of the lane's row (the 16 accumulator
	// registers all belong to that row), so dS = P * (dP accumulator) without a subtraction.
	constexpr bool FOLD_DP = !DROP && D <= 128 && (!BIAS || D == 64);  // (head dim 128 with bias has no registers to spare: bound to 256, its variants spill as it is)
	f32x16 ndel16[QB];
#pragma unroll
	for (int qb = 0; qb < QB; ++qb)
#pragma unroll
		for (int i = 0; i < 16; ++i) ndel16[qb][i] = -del_r[qb];

	const float c1 = BIAS ? a.scale : a.scale * kLog2e;
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
		int row = w * (QB * 32) + c;
		boff_lane = row * 128 + 8 * g + (t_begin & 1) * BIAS_BYTES;
		bkey16 = swz<64>(row) << 4;
		if (bias_lds && ntiles > t_begin)
			bload.load(lds + 4 * TILE_BYTES + (t_begin & 1) * BIAS_BYTES, bias_base + (int64_t)m0 * a.bias_sm + (int64_t)t_begin * BN * 2,
			           a.bias_sm, brows, tid, (a.Sk - t_begin * BN) >> 3);
	}

	// (the offsets carry the buffer - K[1] / V[1] / bias[1] lie a power of two behind K[0] / V[0] / bias[0] -
	// and are flipped after every tile, so that the reads need no address arithmetic in the loop)
	constexpr int KR = KS < 8 ? KS : 8, DR = DB < 4 ? DB : 4;  // (chunks 16 and up: + 256 bytes as an immediate, see the dK/dV kernel)
	int koff[KR];
#pragma unroll
	for (int ks = 0; ks < KR; ++ks) koff[ks] = tile_off<D>(c, 2 * ks + g) + (t_begin & 1) * TILE_BYTES;
	int toff[DR][2];
	{
		int i16 = lane & 15;
		int trow = 4 * g + (i16 >> 2);
		int tcol = 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
#pragma unroll
		for (int db = 0; db < DR; ++db) {
			int col = 32 * db + tcol;
			toff[db][0] = tile_off<D>(trow, col >> 3) + ((col & 4) << 1) + (t_begin & 1) * TILE_BYTES;
			toff[db][1] = tile_off<D>(trow + 8, col >> 3) + ((col & 4) << 1) + (t_begin & 1) * TILE_BYTES;
		}
	}

	auto tile_body = [&](auto masked_tag, int n0) {
		constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
		for (int kb = 0; kb < KB; ++kb) {
			f32x4 bv[BIAS && !BIAS_LDS ? QB : 1][4];
			typename T::V4 bvl[BIAS_LDS ? 4 : 1];  // from LDS, kept in the element type until used (half the registers)
			if constexpr (BIAS_LDS) {
				static_assert(!BIAS_LDS || QB == 1, "");
#pragma unroll
				for (int aa = 0; aa < 4; ++aa)
					bvl[aa] = *(const FA2_LDS typename T::V4*)(lds + 4 * TILE_BYTES + boff_lane + (((kb * 4 + aa) << 4) ^ bkey16));
			} else if constexpr (BIAS) {
#pragma unroll
				for (int qb = 0; qb < QB; ++qb) {
					int i = qrow[qb] < a.Sq ? qrow[qb] : a.Sq - 1;
					const char* rowp = bias_base + (int64_t)i * a.bias_sm;
#pragma unroll
					for (int aa = 0; aa < 4; ++aa) {
						if (CAP && a.bias == nullptr)
							bv[qb][aa] = f32x4{0.f, 0.f, 0.f, 0.f};
						else
							bv[qb][aa] = load_bias4(rowp, n0 + 32 * kb + 8 * aa + 4 * g, a.bias_dtype, a.bias_vec4, a.Sk, a.mask_fill);
					}
				}
			}
			f32x16 s[QB], dp[QB];
#pragma unroll
			for (int qb = 0; qb < QB; ++qb)
#pragma unroll
				for (int i = 0; i < 16; ++i) s[qb][i] = dp[qb][i] = 0.f;
			__builtin_amdgcn_sched_barrier(0);
#if FA2_SETPRIO
			__builtin_amdgcn_s_setprio(FA2_SETPRIO);
#endif
#pragma unroll
			for (int ks = 0; ks < KS; ++ks) {
				V8 ka = *(const FA2_LDS V8*)(lds + koff[ks % KR] + (ks / KR) * 256 + kb * (32 * D * 2));
#pragma unroll
				for (int qb = 0; qb < QB; ++qb) s[qb] = mfma32(ka, qf[qb][ks], s[qb]);
				V8 va = *(const FA2_LDS V8*)(lds + koff[ks % KR] + (ks / KR) * 256 + 2 * TILE_BYTES + kb * (32 * D * 2));
#pragma unroll
				for (int qb = 0; qb < QB; ++qb) dp[qb] = mfma32(va, dof[qb][ks], (FOLD_DP && ks == 0) ? ndel16[qb] : dp[qb]);
			}
			// issue order: a few fragment reads ahead, then one read per product
			{
				constexpr int NR = 2 * KS, PF = NR < 8 ? NR : 8;
				__builtin_amdgcn_sched_group_barrier(0x100, PF, 0);
#pragma unroll
				for (int i = 0; i < NR - PF; ++i) {
					__builtin_amdgcn_sched_group_barrier(0x008, QB, 0);
					__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
				}
				__builtin_amdgcn_sched_group_barrier(0x008, PF * QB, 0);
			}
			__builtin_amdgcn_sched_barrier(0);
#if FA2_SETPRIO
			__builtin_amdgcn_s_setprio(0);
#endif
			// K^T fragments for dQ^T += K^T dS^T, issued ahead of the elementwise math
			constexpr bool BOTH_EARLY = DB <= 4;
			u32x4 kfr[2][DB];
			const FA2_LDS char* kt_a = lds + kb * (32 * D * 2);
			auto issue_k = [&](int hf, u32x4(&dst)[DB]) {
#pragma unroll
				for (int db = 0; db < DB; ++db) dst[db] = lds_tr_issue_rt<D>(kt_a + toff[db % DR][0] + (db / DR) * 256, kt_a + toff[db % DR][1] + (db / DR) * 256, hf);
			};
			issue_k(0, kfr[0]);
			if constexpr (BOTH_EARLY) issue_k(1, kfr[1]);
			V8 dsf[QB][2];
#pragma unroll
			for (int qb = 0; qb < QB; ++qb) {
				uint32_t dw[4][2];
				if constexpr (DROP) dropout_words_rowlane<true>(n0 + 32 * kb + 4 * g, (uint32_t)qrow[qb], (uint32_t)h, (uint32_t)b, drop_k0, drop_k1, dw);
#pragma unroll
				for (int aa = 0; aa < 4; ++aa) {
					float dcap[4];
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						int i = 4 * aa + e;
						float p, th = 0.f;
						if constexpr (CAP) {
							th = tanh_fast(s[qb][i] * a.cap_k1);
							p = exp2_fast(__builtin_fmaf(__builtin_fmaf(th, a.softcap, bv[qb][aa][e]), kLog2e, lse_r[qb]));
						} else if constexpr (BIAS)
							p = exp2_fast(__builtin_fmaf(__builtin_fmaf(s[qb][i], c1, BIAS_LDS ? to_f32x4(bvl[aa])[e] : bv[qb][aa][e]), kLog2e, lse_r[qb]));
						else
							p = exp2_fast(__builtin_fmaf(s[qb][i], c1, lse_r[qb]));
						if constexpr (MASKED) {
							int j = n0 + 32 * kb + 8 * aa + 4 * g + e;
							p = ((j <= jmax[qb]) & (j >= jmin[qb])) ? p : 0.f;
						}
						float dpe = dp[qb][i];
						if constexpr (DROP) dpe = keep16(dw[aa][e >> 1], e & 1, a.drop_thr) ? dpe * a.drop_inv_keep : 0.f;
						s[qb][i] = FOLD_DP ? p * dpe : p * (dpe - del_r[qb]);
						if constexpr (CAP) dcap[e] = __builtin_fmaf(-th, th, 1.f);  // d tanh
					}
					if constexpr (DBIAS) {
						// gradient of the additive term: this lane's row, keys j0 .. j0 + 3
						{
							int j0 = n0 + 32 * kb + 8 * aa + 4 * g;
							if (qrow[qb] < a.Sq && j0 < a.Sk) {
								// (a gradient buffer in the shape of a bias with Hkv heads is indexed like that bias)
								const int hb = a.bias_group ? hk : h;
								char* dp_ = a.dbias + (int64_t)b * a.dbias_sb + (int64_t)hb * a.dbias_sh + (int64_t)qrow[qb] * a.dbias_sm + (int64_t)j0 * 4;
								if (a.dbias_atomic) {
									// several (batch, q-head) pairs share the entry (broadcast axis of the bias): hardware fp32 adds
#pragma unroll
									for (int e = 0; e < 4; ++e)
										if (j0 + e < a.Sk) unsafeAtomicAdd((float*)dp_ + e, s[qb][4 * aa + e]);
								} else if (j0 + 3 < a.Sk) {
									*(f32x4*)dp_ = f32x4{s[qb][4 * aa], s[qb][4 * aa + 1], s[qb][4 * aa + 2], s[qb][4 * aa + 3]};
								} else {
#pragma unroll
									for (int e = 0; e < 4; ++e)
										if (j0 + e < a.Sk) ((float*)dp_)[e] = s[qb][4 * aa + e];
								}
							}
						}
					}
					if constexpr (CAP) {
#pragma unroll
						for (int e = 0; e < 4; ++e) s[qb][4 * aa + e] *= dcap[e];
					}
				}
#pragma unroll
				for (int hf = 0; hf < 2; ++hf) {
					const f32x16& x = s[qb];
					dsf[qb][hf] = pack8<T>(x[8 * hf + 0], x[8 * hf + 1], x[8 * hf + 2], x[8 * hf + 3], x[8 * hf + 4], x[8 * hf + 5],
					                       x[8 * hf + 6], x[8 * hf + 7]);
				}
			}
			// dQ^T += K^T dS^T
#if FA2_SETPRIO
			__builtin_amdgcn_s_setprio(FA2_SETPRIO);
#endif
#pragma unroll
			for (int hf = 0; hf < 2; ++hf) {
				if (hf == 0 && !BOTH_EARLY) issue_k(1, kfr[1]);
#pragma unroll
				for (int db = 0; db < DB; ++db)
#pragma unroll
					for (int qb = 0; qb < QB; ++qb) dq[qb][db] = mfma32(as_frag<T>(kfr[hf][db]), dsf[qb][hf], dq[qb][db]);
			}
#if FA2_SETPRIO
			__builtin_amdgcn_s_setprio(0);
#endif
		}
	};

	// Head dim 256 runs one wave per SIMD, so the elementwise stage overlaps the matrix products only if the wave
	// interleaves them itself (as the forward kernel does at this head dim).  A tile without masking goes as two halves
	// of 32 keys through four phases,
	//   phase 0   S_0 = K_0 Q^T, dP_0 = V_0 dO^T      |  (dropout: the generator calls of half 0)
	//   phase 1   S_1 = K_1 Q^T, dP_1 = V_1 dO^T      |  dS_0 from S_0, dP_0    (dropout: the calls of half 1)
	//   phase 2   dQ^T += K_0^T dS_0^T                |  dS_1 from S_1, dP_1
	//   phase 3   dQ^T += K_1^T dS_1^T
	// with the vector-ALU work in pieces that follow the products one by one and every product preceded by the LDS read
	// of a fragment PA products further on (a scheduling barrier after every slot pins the order).
	constexpr bool PIPE = D == 256 && NW == 4 && QB == 1 && !BIAS && !CAP && !DBIAS;
	auto tile_pipe = [&](int n0) {
		if constexpr (PIPE) {
			constexpr int NA = 2 * KS, NC = 2 * DB;  // products of a phase: S and dP alternating; two 16-key steps x DB
			constexpr int RING = 8, PA = 7;
			static_assert(NA % RING == 0 && NC % RING == 0 && PA < RING, "");
			u32x4 fr[RING];
			f32x16 sc[2], dpc[2];
			u32x4 dsp[2][2];  // [half][16-key step]: dS packed to 16 bits
			float bp[4];
			// fragment f of phase A: k-step f / 2 of K (even f) or V (odd f); of phase C: 16-key step f / DB, d-block f % DB of K^T
			auto read_a = [&](int hf, int f) __attribute__((always_inline)) {
				const int ks = f >> 1;
				fr[f % RING] = __builtin_bit_cast(u32x4, *(const FA2_LDS V8*)(lds + koff[ks % KR] + (ks / KR) * 256 + ((f & 1) ? 2 * TILE_BYTES : 0) + hf * (32 * D * 2)));
			};
			auto read_c = [&](int hf, int f) __attribute__((always_inline)) {
				const int db = f % DB;
				const FA2_LDS char* kt = lds + hf * (32 * D * 2);
				fr[f % RING] = lds_tr_issue_rt<D>(kt + toff[db % DR][0] + (db / DR) * 256, kt + toff[db % DR][1] + (db / DR) * 256, f / DB);
			};
			auto prod_a = [&](int hf, int f) __attribute__((always_inline)) {
				f32x16 zero;
#pragma unroll
				for (int i = 0; i < 16; ++i) zero[i] = 0.f;
				const int ks = f >> 1;
				if (f & 1)
					dpc[hf] = mfma32(as_frag<T>(fr[f % RING]), dof[0][ks], ks == 0 ? zero : dpc[hf]);
				else
					sc[hf] = mfma32(as_frag<T>(fr[f % RING]), qf[0][ks], ks == 0 ? zero : sc[hf]);
			};
			auto prod_c = [&](int hf, int f) __attribute__((always_inline)) {
				dq[0][f % DB] = mfma32(as_frag<T>(fr[f % RING]), as_frag<T>(dsp[hf][f / DB]), dq[0][f % DB]);
			};
			// Dropout: the two generator calls of a half, one after the other, in pieces of two rounds each (see the forward kernel)
			uint32_t cs[4], dwp[2][2][2][2];  // state of the call in flight; words [half][call][group of four keys][word]
			const bool odd = qrow[0] & 1;
			auto gen_piece = [&](int hf, int u, auto pt) __attribute__((always_inline)) {
				if constexpr (DROP) {
					constexpr int pc = decltype(pt)::value;  // 0 .. 4: rounds 2 pc, 2 pc + 1; 5: exchange with the neighbouring row's lane
					if constexpr (pc == 0) {
						cs[0] = (uint32_t)((n0 + 32 * hf + 4 * g + 8 * (2 * u + (odd ? 1 : 0))) >> 2);
						cs[1] = (uint32_t)qrow[0] >> 1;
						cs[2] = (uint32_t)h;
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
			// piece pc (0 .. 7) of the elementwise stage of a half: values 4 aa .. 4 aa + 3 (aa = pc / 2); first P, then dS and the packing
			auto ew_piece = [&](int hf, int pc) __attribute__((always_inline)) {
				const int aa = pc >> 1;
				if ((pc & 1) == 0) {
#pragma unroll
					for (int e = 0; e < 4; ++e) bp[e] = exp2_fast(__builtin_fmaf(sc[hf][4 * aa + e], c1, lse_r[0]));
				} else {
					float ds[4];
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						float dpe = dpc[hf][4 * aa + e];
						if constexpr (DROP) dpe = keep16(dwp[hf][aa >> 1][aa & 1][e >> 1], e & 1, a.drop_thr) ? dpe * a.drop_inv_keep : 0.f;
						ds[e] = bp[e] * (dpe - del_r[0]);
					}
					dsp[hf][aa >> 1][2 * (aa & 1)] = pack2<typename T::V2>(ds[0], ds[1]);
					dsp[hf][aa >> 1][2 * (aa & 1) + 1] = pack2<typename T::V2>(ds[2], ds[3]);
				}
			};
			auto phase = [&](auto n_tag, auto&& read_cur, auto&& prod, auto&& read_next, auto&& valu) __attribute__((always_inline)) {
				constexpr int N = decltype(n_tag)::value;
				__builtin_amdgcn_sched_barrier(0);
				static_for<0, N>([&](auto jt) __attribute__((always_inline)) {
					constexpr int j = decltype(jt)::value;
					if constexpr (j + PA < N)
						read_cur(j + PA);
					else
						read_next(j + PA - N);
					prod(j);
					__builtin_amdgcn_sched_barrier(0);
					valu(jt);
					__builtin_amdgcn_sched_barrier(0);
				});
			};
			auto none = [&](auto) __attribute__((always_inline)) {};
			std::integral_constant<int, NA> na;
			std::integral_constant<int, NC> nc;
			// phase 0: both calls of half 0 (6 pieces each)
			auto v0 = [&](auto jt) __attribute__((always_inline)) {
				constexpr int j = decltype(jt)::value;
				if constexpr (j < 12) gen_piece(0, j / 6, std::integral_constant<int, j % 6>{});
			};
			// phase 1: the pieces of half 0 after the products 2, 4, .. 16; then both calls of half 1
			auto v1 = [&](auto jt) __attribute__((always_inline)) {
				constexpr int j = decltype(jt)::value;
				if constexpr (j >= 2 && j < 18 && j % 2 == 0) ew_piece(0, (j - 2) / 2);
				if constexpr (j >= 18 && j < 30) gen_piece(1, (j - 18) / 6, std::integral_constant<int, (j - 18) % 6>{});
			};
			// phase 2: the pieces of half 1 after the products 2 .. 9
			auto v2 = [&](auto jt) __attribute__((always_inline)) {
				constexpr int j = decltype(jt)::value;
				if constexpr (j >= 2 && j < 10) ew_piece(1, j - 2);
			};
#pragma unroll
			for (int f = 0; f < PA; ++f) read_a(0, f);
			phase(na, [&](int f) __attribute__((always_inline)) { read_a(0, f); }, [&](int f) __attribute__((always_inline)) { prod_a(0, f); },
			      [&](int f) __attribute__((always_inline)) { read_a(1, f); }, v0);
			phase(na, [&](int f) __attribute__((always_inline)) { read_a(1, f); }, [&](int f) __attribute__((always_inline)) { prod_a(1, f); },
			      [&](int f) __attribute__((always_inline)) { read_c(0, f); }, v1);
			phase(nc, [&](int f) __attribute__((always_inline)) { read_c(0, f); }, [&](int f) __attribute__((always_inline)) { prod_c(0, f); },
			      [&](int f) __attribute__((always_inline)) { read_c(1, f); }, v2);
			phase(nc, [&](int f) __attribute__((always_inline)) { read_c(1, f); }, [&](int f) __attribute__((always_inline)) { prod_c(1, f); },
			      [&](int) __attribute__((always_inline)) {}, none);
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
			toff[db][0] ^= TILE_BYTES;
			toff[db][1] ^= TILE_BYTES;
		}
		if constexpr (BIAS_LDS) boff_lane ^= BIAS_BYTES;
	};
	// Tiles that lie entirely inside every row's range of allowed keys need no mask.  They
	// run in a loop of their own, so that the steady-state loop is a single straight-line
	// body; the tiles on the window's left edge come before them, the tiles on the causal
	// diagonal / right edge / ragged end after.
	int t_lo = wave_lmax > 0 ? (wave_lmax + BN - 1) / BN : 0;
	t_lo = t_lo < t_begin ? t_begin : (t_lo > ntiles ? ntiles : t_lo);
	int t_full = (wave_jmin + 1) / BN;
	t_full = t_full < t_lo ? t_lo : (t_full > ntiles ? ntiles : t_full);
	for (int t = t_begin; t < t_lo; ++t) step(std::true_type{}, t);
	for (int t = t_lo; t < t_full; ++t) step(std::false_type{}, t);
	for (int t = t_full; t < ntiles; ++t) step(std::true_type{}, t);

	char* obase = a.dq.ptr + (int64_t)b * a.dq.sb + (int64_t)h * a.dq.sh;
#pragma unroll
	for (int qb = 0; qb < QB; ++qb) {
		int i = qrow[qb];
		if (i < a.Sq) {
			char* rp = obase + (int64_t)i * a.dq.ss;
			const float sc = a.scale;
#pragma unroll
			for (int db = 0; db < DB; ++db)
#pragma unroll
				for (int aa = 0; aa < 4; ++aa) {
					const f32x16& x = dq[qb][db];
					u32x2 pk = {pack2<typename T::V2>(x[4 * aa] * sc, x[4 * aa + 1] * sc),
					            pack2<typename T::V2>(x[4 * aa + 2] * sc, x[4 * aa + 3] * sc)};
					*(u32x2*)(rp + (32 * db + 8 * aa + 4 * g) * 2) = pk;
				}
		}
	}
}

template <typename T, int D>
struct BwdCfg {
	// dK/dV: 4 waves x 32 keys; query rows streamed 64 (32 for D = 256) at a time
	static constexpr int KV_NW = 4;
	static constexpr int KV_QB = D <= 128 ? 4 : 1;
	static constexpr int KV_BN = KV_NW * 32;
	// dQ: 4 waves x QB x 32 rows
	static constexpr int DQ_NW = D <= 128 ? 8 : 4;
	static constexpr int DQ_QB = 1;
	static constexpr int DQ_WPS = 1;
	static constexpr int DQ_BM = DQ_NW * DQ_QB * 32;
};

template <typename T, int D, bool BIAS, bool DROP>
hipError_t launch_bwd_v(KArgs& a, hipStream_t s) {
	typedef BwdCfg<T, D> C;
	int groups = a.B * a.Hkv;
	a.xcd_remap = (groups % 8 == 0) ? 1 : 0;
	if (BIAS && a.bias_sh == 0 && a.B % 8 == 0) a.xcd_remap = a.kv_lens ? 3 : 2;
	// Delta and dQ both requested (the whole backward, or stages 1 + 4): the dQ kernel forms delta
	// itself and runs first, the dK/dV kernel reads the delta it left in scratch.  Otherwise each
	// stage is launched as asked and the dQ / dK/dV kernels read the delta of an earlier pre-pass.
	const bool fused_delta = (a.stages & 5) == 5;
	a.dq_makes_delta = fused_delta ? 1 : 0;
	if ((a.stages & 1) && !fused_delta) {
		int64_t nrows = (int64_t)a.B * a.Sq * a.Hq;
		constexpr int RPB = 256 / (D / 8);
		hipLaunchKernelGGL((bwd_delta_kernel<T, D>), dim3((unsigned)((nrows + RPB - 1) / RPB)), dim3(256), 0, s, a);
	}
	auto launch_dq_cfg = [&](auto nw_tag, auto wps_tag) {
		constexpr int NW = decltype(nw_tag)::value, BM = NW * C::DQ_QB * 32, WPS = decltype(wps_tag)::value;
		a.mtiles = (a.Sq + BM - 1) / BM;
		a.interleave = a.xcd_remap == 1 ? launch_order(a, a.Hq / a.Hkv, groups / 8, (int64_t)a.Sk * D * 4) : 1;
		dim3 grid((unsigned)(a.mtiles * a.B * a.Hq)), block(NW * 64);
		a.fold_half = fold_half_of(a, NW, (int64_t)grid.x, D == 64 || WPS == 2);
		if (BIAS && a.dbias && a.softcap > 0.f)
			hipLaunchKernelGGL((bwd_dq_kernel<T, D, NW, C::DQ_QB, WPS, BIAS, DROP, false, BIAS, BIAS>), grid, block, 0, s, a);
		else if (BIAS && a.dbias)
			hipLaunchKernelGGL((bwd_dq_kernel<T, D, NW, C::DQ_QB, WPS, BIAS, DROP, false, false, BIAS>), grid, block, 0, s, a);
		else if (BIAS && a.softcap > 0.f)
			hipLaunchKernelGGL((bwd_dq_kernel<T, D, NW, C::DQ_QB, WPS, BIAS, DROP, false, BIAS>), grid, block, 0, s, a);
		else if (BIAS && a.bias_lds)
			hipLaunchKernelGGL((bwd_dq_kernel<T, D, NW, C::DQ_QB, WPS, BIAS, DROP, BIAS>), grid, block, 0, s, a);
		else
			hipLaunchKernelGGL((bwd_dq_kernel<T, D, NW, C::DQ_QB, WPS, BIAS, DROP, false>), grid, block, 0, s, a);
	};
	auto launch_dq = [&]() {
		if constexpr (C::DQ_NW == 8) {
			// a grid that leaves at least half of the chip idle: workgroups of 128 rows instead of 256 (see the forward)
			int64_t wgs = (int64_t)((a.Sq + 127) / 128) * a.B * a.Hq;
			if (wgs <= kNumCU) return launch_dq_cfg(std::integral_constant<int, 4>{}, std::integral_constant<int, C::DQ_WPS>{});
			// larger grids: two 128-row workgroups per CU where the K and V of a head fit an XCD's L2 (see the forward;
			// the dQ kernel gains with and without a causal mask: D = 128 B8 S2048 causal 0.460 -> 0.418 ms, non-causal
			// 0.784 -> 0.734 ms, B4 S4096 causal 0.770 -> 0.739 ms; D = 64 B32 S512 0.060 -> 0.051 ms); D = 128 with bias
			// would spill within 256 registers
			if constexpr (D == 64 || !BIAS) {
				if ((int64_t)a.Sk * D * 4 <= (4 << 20))
					return launch_dq_cfg(std::integral_constant<int, 4>{}, std::integral_constant<int, (D == 128 ? 2 : 1)>{});
			}
		}
		launch_dq_cfg(std::integral_constant<int, C::DQ_NW>{}, std::integral_constant<int, C::DQ_WPS>{});
	};
	if (fused_delta) launch_dq();
	if (a.stages & 2) {
		a.mtiles = (a.Sk + C::KV_BN - 1) / C::KV_BN;
		a.interleave = a.xcd_remap == 1 ? launch_order(a, 1, groups / 8, (int64_t)(a.Hq / a.Hkv) * a.Sq * D * 4) : 1;
		const int hs = a.kv_hsplit > 1 ? a.kv_hsplit : 1;
		// Causal self-attention on a grid that fills the chip in whole rounds: every workgroup takes the key tiles p and
		// ntiles - 1 - p one after the other (see bwd_dkdv_kernel).  Measured on the 4096-token workload (B4 Hq32 Hkv8):
		// dK/dV kernel 1.032 -> 1.000 ms and 1318 -> 437 MiB fetched from memory (324 MiB of operands); on the
		// 32768-token one 31.7 -> 30.3 ms and 87 -> 4.8 GiB (1.14 GiB of operands).  Walking the query tiles outermost
		// WITHOUT the pairing (one tile per workgroup, ascending or descending) measured slower than head by head: 1.065 /
		// 1.051 ms, so everything else keeps that order.
		a.kv_pair = 0;
		a.kv_ntiles = a.mtiles;
		// (from 16 key tiles on: B16 H16 S1000, 8 tiles of one q-head each, measured 0.218 ms one tile per workgroup and 0.224 ms paired)
		if (D <= 128 && !BIAS && hs == 1 && a.causal && a.win_left < 0 && a.Sq == a.Sk && !a.seqlens && !a.kv_lens && a.xcd_remap <= 1 && a.mtiles >= 16) {
			const int64_t pairs = (int64_t)((a.mtiles + 1) / 2) * groups;
			if (pairs % kNumCU == 0 || pairs >= 8 * kNumCU) {
				a.kv_pair = 1;
				a.mtiles = (a.mtiles + 1) / 2;
				a.interleave = 1;
			}
		}
		dim3 grid((unsigned)(a.mtiles * a.B * a.Hkv * hs)), block(C::KV_NW * 64);
		// typed variant: bias in the element type of q, staged through LDS: it also needs 16-byte aligned rows of whole 16-byte pieces
		bool typed = BIAS && a.bias_dtype == (std::is_same<T, BF16>::value ? 2 : 1);
		if (!a.bias_lds) typed = false;
		// with bias at D = 128 the streamed tiles are 64 rows, which leaves LDS room for the bias tiles
		constexpr int QBV = (BIAS && D == 128) ? 2 : C::KV_QB;
		if (BIAS && a.softcap > 0.f)
			hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, C::KV_NW, QBV, BIAS, DROP, false, BIAS>), grid, block, 0, s, a);
		else if (typed)
			hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, C::KV_NW, QBV, BIAS, DROP, BIAS>), grid, block, 0, s, a);
		else if (a.kv_pair) {
			// (only instantiated where the launcher can choose it: no bias, head dim up to 128)
			if constexpr (D <= 128 && !BIAS) hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, C::KV_NW, QBV, BIAS, DROP, false, false, true>), grid, block, 0, s, a);
		} else
			hipLaunchKernelGGL((bwd_dkdv_kernel<T, D, C::KV_NW, QBV, BIAS, DROP, false>), grid, block, 0, s, a);
		if (hs > 1) {
			int64_t total = (int64_t)a.B * a.Hkv * a.Sk * 2 * (D / 8);
			hipLaunchKernelGGL((bwd_dkdv_reduce_kernel<T, D>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a, a.scale,
			                   DROP ? a.drop_inv_keep : 1.f);
		}
	}
	if ((a.stages & 4) && !fused_delta) launch_dq();
	return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_bwd_t(bool bias, bool drop, KArgs& a, hipStream_t s) {
	if (bias && drop) return launch_bwd_v<T, D, true, true>(a, s);
	if (bias) return launch_bwd_v<T, D, true, false>(a, s);
	if (drop) return launch_bwd_v<T, D, false, true>(a, s);
	return launch_bwd_v<T, D, false, false>(a, s);
}

}  // namespace fa2
