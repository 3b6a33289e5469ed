// Device-side building blocks shared by the forward and backward kernels:
// element types, MFMA wrappers, swizzled LDS tiles (plain and transposed
// fragment reads), direct global->LDS tile copies, Philox dropout.
// gfx950 (CDNA4) only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fa2 {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define FA2_DEV __device__ __forceinline__
#define FA2_LDS __attribute__((address_space(3)))
#define FA2_GLB __attribute__((address_space(1)))

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// f(integral_constant<int, I>) for I = FROM .. TO - 1, unrolled at compile time
template <int FROM, int TO, typename F>
FA2_DEV void static_for(F&& f) {
	if constexpr (FROM < TO) {
		f(std::integral_constant<int, FROM>{});
		static_for<FROM + 1, TO>(f);
	}
}

// Element traits: E = storage element, V8/V4/V2 = vectors of it.
struct BF16 {
	typedef __bf16 E;
	typedef bf16x8 V8;
	typedef bf16x4 V4;
	typedef bf16x2 V2;
};
struct FP16 {
	typedef _Float16 E;
	typedef f16x8 V8;
	typedef f16x4 V4;
	typedef f16x2 V2;
};

// D[32x32] += A[32x16] * B[16x32].  Lane l supplies A[row l%32][k 8*(l/32)..+7]
// and B[k 8*(l/32)..+7][col l%32]; it receives D[row 8*(i/4)+4*(l/32)+i%4][col l%32]
// in element i of the accumulator.
FA2_DEV f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
	return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
FA2_DEV f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
	return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// The same product issued through inline assembly so that the register file of
// every operand is fixed by the constraint: accumulators that only matrix
// products touch (and operands that stay for the whole kernel) live in AGPRs,
// accumulators that the vector ALU consumes live in VGPRs.  Left to itself the
// register allocator puts those into AGPRs as well and copies each value out
// with v_accvgpr_read before the vector ALU can use it.
// The compiler does not know these statements are matrix products, so it adds
// no wait states for them: the caller keeps a vector-ALU read of a result at
// least two further matrix products away from the product that wrote it.
//   mfma32_va: C(VGPR) += A(VGPR) * B(AGPR)
//   mfma32_vc: C(VGPR) = A(VGPR) * B(AGPR) + C0(VGPR)   first product of a chain, from a start value
//   mfma32_vz: C(VGPR) = A(VGPR) * B(VGPR)              first product of a chain, from zero
//   mfma32_aa: C(AGPR) += A(VGPR) * B(VGPR)
// BA: the B operand lives in an AGPR (else in a VGPR)
template <bool BA>
FA2_DEV void mfma32_va(f32x16& c, bf16x8 a, bf16x8 b) {
	if constexpr (BA)
		asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
	else
		asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
template <bool BA>
FA2_DEV void mfma32_va(f32x16& c, f16x8 a, f16x8 b) {
	if constexpr (BA)
		asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
	else
		asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
// first product of a chain that starts from zero: C(VGPR) = A(VGPR) * B(VGPR)
FA2_DEV void mfma32_vz(f32x16& c, bf16x8 a, bf16x8 b) { asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b)); }
FA2_DEV void mfma32_vz(f32x16& c, f16x8 a, f16x8 b) { asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b)); }
FA2_DEV void mfma32_vc(f32x16& c, bf16x8 a, bf16x8 b, f32x16 c0) {
	asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(c) : "v"(a), "a"(b), "v"(c0));
}
FA2_DEV void mfma32_vc(f32x16& c, f16x8 a, f16x8 b, f32x16 c0) {
	asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(c) : "v"(a), "a"(b), "v"(c0));
}
FA2_DEV void mfma32_aa(f32x16& c, bf16x8 a, bf16x8 b) {
	asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
FA2_DEV void mfma32_aa(f32x16& c, f16x8 a, f16x8 b) {
	asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

template <typename V2>
FA2_DEV uint32_t pack2(float a, float b) {
	f32x2 f = {a, b};
	V2 h = __builtin_convertvector(f, V2);
	return __builtin_bit_cast(uint32_t, h);
}

// Eight fp32 -> one 8-element MFMA operand.
template <typename T>
FA2_DEV typename T::V8 pack8(float x0, float x1, float x2, float x3, float x4, float x5, float x6, float x7) {
	u32x4 u = {pack2<typename T::V2>(x0, x1), pack2<typename T::V2>(x2, x3), pack2<typename T::V2>(x4, x5),
	           pack2<typename T::V2>(x6, x7)};
	return __builtin_bit_cast(typename T::V8, u);
}

// 16-bit element -> fp32.  A bf16 value is the upper half of the fp32 with the same value; written as the shift itself
// because the compiler's extension adds a multiply by 1.0 (it quiets signalling NaNs), one more vector-ALU instruction per
// bias value in loops that are bound by exactly those.
FA2_DEV float to_f32(__bf16 x) { return __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(uint16_t, x) << 16); }
FA2_DEV float to_f32(_Float16 x) { return (float)x; }
FA2_DEV f32x4 to_f32x4(bf16x4 x) {
	u32x2 u = __builtin_bit_cast(u32x2, x);
	f32x4 r = {__builtin_bit_cast(float, u[0] << 16), __builtin_bit_cast(float, u[0] & 0xffff0000u), __builtin_bit_cast(float, u[1] << 16),
	           __builtin_bit_cast(float, u[1] & 0xffff0000u)};
	return r;
}
FA2_DEV f32x4 to_f32x4(f16x4 x) { return __builtin_convertvector(x, f32x4); }

FA2_DEV float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
FA2_DEV float log2_fast(float x) { return __builtin_amdgcn_logf(x); }
// tanh(x) = 1 - 2 / (1 + e^(2x)): one exp2, one reciprocal; exactly +-1 at the ends of the range
FA2_DEV float tanh_fast(float x) {
	float t = exp2_fast(x * (2.f * kLog2e));
	return __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(t + 1.f), 1.f);
}

// max of the values held by lane l and lane l^32
FA2_DEV float pair_max(float x) {
	auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), false, false);
	return __builtin_fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
}
FA2_DEV float pair_sum(float x) {
	auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), false, false);
	return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}

// ---------------------------------------------------------------------------
// LDS tiles.  A tile is ROWS x D elements, row-major, 16-byte chunks XOR
// swizzled inside each row so that (a) sixteen lanes reading the same chunk of
// sixteen consecutive rows and (b) the four-row groups of a transposed read
// fall on distinct banks.
// ---------------------------------------------------------------------------
template <int D>
FA2_DEV int swz(int row) {
	if constexpr (D >= 128)
		return ((row & 3) << 2) | ((row >> 2) & 3);
	else
		return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
}

// byte offset of 16-byte chunk `chunk` of row `row`
template <int D>
FA2_DEV int tile_off(int row, int chunk) {
	return row * (D * 2) + ((chunk ^ swz<D>(row)) << 4);
}

// Fragments.  Operand whose 32 rows/cols are tile rows and whose MFMA k runs along D:
// lane l holds tile[row0 + l%32][16*ks + 8*(l/32) .. +7], one 16-byte read at tile_off().
// Transposed operand (its 32 rows/cols run along D, its MFMA k along tile rows):
// k-slot (g = l/32, j) is tile row row0 + 4g + j for j < 4 and row0 + 8 + 4g + (j-4) for
// j >= 4, which is the order in which a 32x32 accumulator holds its rows - so an
// accumulator packed to 16 bits is directly the other operand.  It is built from two
// ds_read_b64_tr_b16: inside a block of 16 lanes, lane i receives element i%4 of the
// 8-byte rows fetched by lanes 4j + i/4, j = 0..3; the lane's own piece is rows
// row0 + 4g + (l%16)/4 (+ 8), columns col0 + 16 ((l/16)%2) + 4 (l%4) .. +3.

// Transposed fragment from two per-lane byte addresses (rows r and r + 8) plus a
// compile-time byte offset.  Returned as raw bits; as_frag<T>() views them as the
// MFMA operand.
template <int IMM>
FA2_DEV u32x4 lds_tr_issue(const FA2_LDS char* p_lo, const FA2_LDS char* p_hi) {
	typedef __attribute__((__vector_size__(4 * sizeof(short)))) short v4s;
	v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA2_LDS v4s*)(p_lo + IMM));
	v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA2_LDS v4s*)(p_hi + IMM));
	typedef __attribute__((__vector_size__(8 * sizeof(short)))) short v8s;
	v8s both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
	return __builtin_bit_cast(u32x4, both);
}

// Same with the offset chosen among the 16-row steps 0..3 of a tile with row
// length D (the step is a compile-time constant after unrolling, so the switch
// folds away).
template <int D>
FA2_DEV u32x4 lds_tr_issue_rt(const FA2_LDS char* p_lo, const FA2_LDS char* p_hi, int step16) {
	switch (step16) {
		case 0: return lds_tr_issue<0>(p_lo, p_hi);
		case 1: return lds_tr_issue<16 * D * 2>(p_lo, p_hi);
		case 2: return lds_tr_issue<32 * D * 2>(p_lo, p_hi);
		default: return lds_tr_issue<48 * D * 2>(p_lo, p_hi);
	}
}

// One step of a double-buffered LDS pipeline.  `issue(next0, next1)` starts the
// direct global->LDS copies of the next tile, `body(cur0, cur1)` computes on the
// current one.  The four regions are distinct; declaring them __restrict__ here
// is what lets the compiler see that the LDS reads of `body` never touch the
// regions the copies are filling - without it every transposed read would be
// preceded by a wait for ALL outstanding copies (s_waitcnt vmcnt(0)), which
// would serialise the double buffer.
template <typename Issue, typename Body>
FA2_DEV void lds_pipeline_step(const FA2_LDS char* __restrict__ cur0, const FA2_LDS char* __restrict__ cur1,
                               FA2_LDS char* __restrict__ next0, FA2_LDS char* __restrict__ next1, Issue&& issue,
                               Body&& body) {
	issue(next0, next1);
	body(cur0, cur1);
}

template <typename T>
FA2_DEV typename T::V8 as_frag(u32x4 x) {
	return __builtin_bit_cast(typename T::V8, x);
}

// Copy of a ROWS x D tile from global memory (row stride in bytes) into a swizzled LDS
// tile without passing through registers.  Each wave-level instruction moves 64 x 16
// bytes; lane i lands at LDS slot base + i, so the swizzle is applied by choosing which
// global chunk each lane fetches.  Rows at or beyond the valid ones are fetched from the
// last valid row instead (the caller masks their scores), so no lane reads out of bounds.
// The copies are issued through inline assembly on purpose: the compiler then does not
// model them as LDS accesses in flight.  If it did, every wait for an LDS read
// (s_waitcnt lgkmcnt) issued while a copy is outstanding would drain ALL outstanding LDS
// reads instead of only those older than the one needed, which defeats reading fragments
// several products ahead.  Completion is awaited explicitly with wait_async_loads()
// before the workgroup barrier that publishes the tile.
// The addressing is hoisted out of the loop that streams tiles: init() computes, once,
// this lane's byte offsets inside a tile; load() then issues one instruction per
// 64 x 16 bytes from a wave-uniform tile base (SGPR pair) plus that 32-bit lane offset
// (row stride x ROWS must fit 31 bits; the launcher checks).
// One such instruction: lane i fetches 16 bytes at uniform_base + lane_off, they land at
// LDS byte address wave_dst + 16 i (wave_dst is wave-uniform).
FA2_DEV void lds_dma16_so(uint32_t lane_off, const char* uniform_base, FA2_LDS char* wave_dst) {
	uint32_t m = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)wave_dst);
	// s_nop 3: with s_mov that makes 5 wait states between a v_readfirstlane that produced the
	// base and the memory instruction reading it as an SGPR operand; the compiler pads such
	// hazards for its own instructions but does not look inside inline assembly
	asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(uniform_base), "s"(m)
	             : "m0");
}

template <int D, int ROWS, int NTHREADS>
struct TileLoader {
	static constexpr int CPR = D / 8;
	static constexpr int TOTAL = ROWS * CPR;
	static constexpr int NIT = TOTAL / NTHREADS;  // 64 x 16 byte pieces per wave and tile
	static_assert(TOTAL % NTHREADS == 0, "tile must divide over the workgroup");
	// Rows of 512 bytes (head dim 256) make eight pieces per tile and registers are short there.  Piece `it`
	// covers rows it * RPI + tid / CPR, and the swizzle repeats every 16 rows: pieces P apart differ by a
	// whole number of 16-row blocks, which goes into the wave-uniform base address.  Only the first NP offsets
	// are kept; a tile that needs clamping (ragged end) computes its offsets as it goes.
	static constexpr bool COMPACT = D >= 256 && NTHREADS % CPR == 0;
	static constexpr int RPI = NTHREADS / CPR;
	static constexpr int P = RPI >= 16 ? 1 : 16 / RPI;
	static constexpr int NP = COMPACT ? (NIT < P ? NIT : P) : NIT;
	uint32_t off[NP];
	int rows_state;  // the offsets clamp rows to [0, rows_state)
	int cols_state;  // ... and 16-byte chunks of a row to [0, cols_state)
	int wave_slot;   // byte offset of this wave's 64 x 16 bytes inside a piece (scalar)

	static FA2_DEV uint32_t offset_of(int it, int64_t stride_bytes, int tid, int rows_valid, int chunks_valid) {
		int slot = it * NTHREADS + tid;
		int row = slot / CPR;
		int chunk = (slot % CPR) ^ swz<D>(row);
		int grow = row < rows_valid ? row : rows_valid - 1;
		int gchunk = chunk < chunks_valid ? chunk : chunks_valid - 1;
		return (uint32_t)grow * (uint32_t)stride_bytes + (uint32_t)(gchunk << 4);
	}
	// stride_bytes * ROWS must fit 31 bits (the launcher checks)
	FA2_DEV void init(int64_t stride_bytes, int tid, int rows_valid = ROWS, int chunks_valid = CPR) {
		rows_state = rows_valid;
		cols_state = chunks_valid;
		wave_slot = __builtin_amdgcn_readfirstlane((tid >> 6) << 10);
#pragma unroll
		for (int it = 0; it < NP; ++it)
			off[it] = COMPACT ? offset_of(it, stride_bytes, tid, ROWS, CPR) : offset_of(it, stride_bytes, tid, rows_valid, chunks_valid);
	}
	// make the offsets fit a tile with rows_valid rows of chunks_valid chunks (wave-uniform; recomputes only on change)
	FA2_DEV void fit(int64_t stride_bytes, int tid, int rows_valid, int chunks_valid = CPR) {
		rows_valid = rows_valid < ROWS ? rows_valid : ROWS;
		chunks_valid = chunks_valid < CPR ? chunks_valid : CPR;
		if constexpr (COMPACT) {
			rows_state = rows_valid;
			cols_state = chunks_valid;
		} else {
			if (rows_valid != rows_state || chunks_valid != cols_state) init(stride_bytes, tid, rows_valid, chunks_valid);
		}
	}
	// a wave-uniform pointer as an explicitly scalar value
	static FA2_DEV const char* uniform(const char* p) {
		uint64_t gb = (uint64_t)p;
		uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)gb), hi = __builtin_amdgcn_readfirstlane((uint32_t)(gb >> 32));
		return (const char*)(((uint64_t)hi << 32) | lo);
	}
	// piece `it` (0 .. NIT-1) of the tile whose first row is at ub = uniform(address)
	FA2_DEV void load_one(FA2_LDS char* tile, const char* ub, int it, int tid) const {
		lds_dma16_so(off[it], ub, tile + it * NTHREADS * 16 + wave_slot);
	}
	// whole tile; rows at or beyond rows_valid are fetched from the last valid row, 16-byte chunks at or
	// beyond chunks_valid from the last valid chunk of their row
	FA2_DEV void load(FA2_LDS char* tile, const char* gbase, int64_t stride_bytes, int rows_valid, int tid, int chunks_valid = CPR) {
		fit(stride_bytes, tid, rows_valid, chunks_valid);
		const char* ub = uniform(gbase);
		if constexpr (COMPACT) {
			if (rows_state == ROWS && cols_state == CPR) {
#pragma unroll
				for (int it = 0; it < NIT; ++it)
					lds_dma16_so(off[it % NP], ub + (int64_t)((it / NP) * NP * RPI) * stride_bytes, tile + it * NTHREADS * 16 + wave_slot);
			} else {
#pragma unroll
				for (int it = 0; it < NIT; ++it)
					lds_dma16_so(offset_of(it, stride_bytes, tid, rows_state, cols_state), ub, tile + it * NTHREADS * 16 + wave_slot);
			}
		} else {
#pragma unroll
			for (int it = 0; it < NIT; ++it) load_one(tile, ub, it, tid);
		}
	}
};

FA2_DEV void wait_async_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---------------------------------------------------------------------------
// Dropout: Philox-4x32-10, key = (seed lo, seed hi).  One call serves two adjacent rows x four adjacent
// keys: counter = (j >> 2, i >> 1, h, b); its four words are eight 16-bit values (word w = values 2w in
// the low half, 2w + 1 in the high half), value (i & 1) * 4 + (j & 3) belongs to element (i, j), which is
// kept iff value >= floor(p * 65536).  The generator dominates the cost of dropout (20 64-bit multiplies
// per call), and both register layouts of the scores let the lanes that share a call exchange its words
// with DPP moves inside a quad, so every lane evaluates half the calls it has values for.
// ---------------------------------------------------------------------------
FA2_DEV u32x4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
	for (int r = 0; r < 10; ++r) {
		// written as one 32 x 32 -> 64 bit product each (one v_mad_u64_u32 instead of a high and a low multiply)
		uint64_t p0 = (uint64_t)0xD2511F53u * (uint64_t)c0;
		uint64_t p1 = (uint64_t)0xCD9E8D57u * (uint64_t)c2;
		uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
		uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
		uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
		c0 = n0;
		c1 = lo1;
		c2 = n2;
		c3 = lo0;
		k0 += 0x9E3779B9u;
		k1 += 0xBB67AE85u;
	}
	u32x4 out = {c0, c1, c2, c3};
	return out;
}

// Rounds [R0, R1) of the same generator on a counter kept by the caller, for callers that
// spread one evaluation over several places of their instruction stream.
template <int R0, int R1>
FA2_DEV void philox4x32_rounds(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
#pragma unroll
	for (int r = R0; r < R1; ++r) {
		uint32_t kr0 = k0 + (uint32_t)r * 0x9E3779B9u, kr1 = k1 + (uint32_t)r * 0xBB67AE85u;
		// written as one 32 x 32 -> 64 bit product each
		uint64_t p0 = (uint64_t)0xD2511F53u * (uint64_t)c[0];
		uint64_t p1 = (uint64_t)0xCD9E8D57u * (uint64_t)c[2];
		uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
		uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
		uint32_t n0 = hi1 ^ c[1] ^ kr0, n2 = hi0 ^ c[3] ^ kr1;
		c[0] = n0;
		c[1] = lo1;
		c[2] = n2;
		c[3] = lo0;
	}
}

// value `half` (0 / 1) of a word against the threshold
FA2_DEV bool keep16(uint32_t word, int half, uint32_t thr16) { return (half ? (word >> 16) : (word & 0xffffu)) >= thr16; }

// Two packed 16-bit elements `x` against the two 16-bit values of `word` (low half with low half): an element whose value is
// below the threshold becomes +0.  thr2 = the threshold in both halves.  Three packed 16-bit integer operations:
// d = thr -sat value is non-zero exactly for a dropped element, 1 -sat d is the factor 1 / 0.
FA2_DEV uint32_t keep_pair16(uint32_t x, uint32_t word, uint32_t thr2) {
	typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
	const u16x2 one = {1, 1};
	u16x2 d = __builtin_elementwise_sub_sat(__builtin_bit_cast(u16x2, thr2), __builtin_bit_cast(u16x2, word));
	u16x2 k = __builtin_elementwise_sub_sat(one, d);
	return __builtin_bit_cast(uint32_t, (u16x2)(__builtin_bit_cast(u16x2, x) * k));
}

// the neighbouring lane's value (lanes 0 <-> 1, 2 <-> 3 of every quad)
FA2_DEV uint32_t quad_swap1(uint32_t x) { return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, 0xB1, 0xf, 0xf, false); }

// Layout "lane = query row" (forward and dQ kernels: a lane holds keys jb + 8 aa + e, aa = 0..3, e = 0..3, of its row,
// and the lane next to it holds the same keys of the other row of the pair): w[aa][0..1] receive the two words with
// the row's four values for keys jb + 8 aa .. + 3.  SHARE: the lane of the even row evaluates the calls of aa = 0, 2,
// the lane of the odd row those of aa = 1, 3, and they exchange (needs lane ^ 1 = row ^ 1 in the same (b, h));
// otherwise every lane evaluates its four calls itself.
// This function yields one half of that - w[0], w[1] = the words of aa = 2 pr and 2 pr + 1 (with SHARE one generator call per lane).
template <bool SHARE>
FA2_DEV void dropout_words_rowlane_half(int jb, uint32_t row, uint32_t h, uint32_t b, uint32_t k0, uint32_t k1, int pr, uint32_t (&w)[2][2]) {
	const bool odd = row & 1u;
	if constexpr (SHARE) {
		int aa_mine = 2 * pr + (odd ? 1 : 0);
		u32x4 r = philox4x32_10((uint32_t)((jb + 8 * aa_mine) >> 2), row >> 1, h, b, k0, k1);
		uint32_t own0 = odd ? r[2] : r[0], own1 = odd ? r[3] : r[1];
		uint32_t got0 = quad_swap1(odd ? r[0] : r[2]), got1 = quad_swap1(odd ? r[1] : r[3]);
		w[0][0] = odd ? got0 : own0;
		w[0][1] = odd ? got1 : own1;
		w[1][0] = odd ? own0 : got0;
		w[1][1] = odd ? own1 : got1;
	} else {
#pragma unroll
		for (int u = 0; u < 2; ++u) {
			u32x4 r = philox4x32_10((uint32_t)((jb + 8 * (2 * pr + u)) >> 2), row >> 1, h, b, k0, k1);
			w[u][0] = odd ? r[2] : r[0];
			w[u][1] = odd ? r[3] : r[1];
		}
	}
}
// both halves: w[aa] for aa = 0 .. 3
template <bool SHARE>
FA2_DEV void dropout_words_rowlane(int jb, uint32_t row, uint32_t h, uint32_t b, uint32_t k0, uint32_t k1, uint32_t (&w)[4][2]) {
#pragma unroll
	for (int pr = 0; pr < 2; ++pr) {
		uint32_t half[2][2];
		dropout_words_rowlane_half<SHARE>(jb, row, h, b, k0, k1, pr, half);
		w[2 * pr][0] = half[0][0];
		w[2 * pr][1] = half[0][1];
		w[2 * pr + 1][0] = half[1][0];
		w[2 * pr + 1][1] = half[1][1];
	}
}

}  // namespace fa2
