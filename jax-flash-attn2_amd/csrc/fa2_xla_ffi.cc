// XLA FFI handlers: the JAX-side entry into libfa2_hip.so.
//
// Each handler only translates XLA buffers and attributes into an fa2_params
// block and calls the plain C ABI (fa2_fwd / fa2_bwd / fa2_dropout_mask,
// include/fa2.h) on the stream XLA hands over.  They take the place of the
// custom calls the reference emits through eformer.callib.triton_call
// (jax_flash_attn2/flash_attention_triton/_forward_triton.py:547-588,
//  _backward_triton.py:1049-1154).
//
// This file needs the XLA FFI headers that ship inside jaxlib
// (`jax.ffi.include_dir()`); it is compiled into libfa2_xla_ffi.so by
// `make ffi XLA_FFI_INCLUDE=<dir>` and is not part of the default build.
//
// Operand convention (absent optional operands are passed as 0-element buffers); the same lists, in the same
// order, are in jax_flash_attn2/_ffi_spec.py, from which the Python side builds its calls:
//   fa2_fwd_ffi : args q, k, v, bias, seqlens, kv_lens, seed                    rets o, lse, scratch
//   fa2_bwd_ffi : args q, k, v, bias, seqlens, kv_lens, seed, o, lse, dout      rets dq, dk, dv, dbias, scratch
//   attrs (both): scale f32, dropout_p f32, causal bool, bias_group bool,
//                 has_window bool, window_left i32, window_right i32, softcap f32
// Every field of fa2_params is reachable: a `bias` buffer of element type PRED / U8 / S8 is a boolean mask, one
// byte per position (bias_dtype = FA2_MASK_U8); `kv_lens` int32 [B]; the window and soft-capping are attributes;
// `dbias`, fp32 in the shape of the bias, is a result (0 elements = not wanted), cleared here by a fill kernel because
// the dQ kernel leaves skipped key tiles unwritten and adds into entries that several (batch, head) pairs share.
// The dropout seed is an OPERAND (8 bytes on the device: u32[2] low word first, or one 64-bit
// integer), as in the reference, whose custom call takes dropout_seed as an operand
// (_forward_triton.py:553): a new seed then needs no new executable and the seed may be traced.
// All tensors are dense row-major as XLA lays them out: q/o/dout/dq [B,Sq,Hq,D],
// k/v/dk/dv [B,Sk,Hkv,D], bias [B|1, H|1, Sq, Sk], lse [B,Hq,Sq] f32,
// scratch u8: fa2_bwd_scratch_bytes (or the larger fa2_bwd_split_scratch_bytes) for the backward, fa2_fwd_scratch_bytes (or any smaller size: no split) for the forward.
#include <hip/hip_runtime.h>

#include <cstring>

#include "../../include/fa2.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

int elem_type(ffi::DataType t) {
	switch (t) {
		case ffi::DataType::F16: return FA2_FP16;
		case ffi::DataType::BF16: return FA2_BF16;
		case ffi::DataType::F32: return FA2_FP32;
		// a boolean mask, one byte per position (XLA stores PRED as bytes)
		case ffi::DataType::PRED:
		case ffi::DataType::U8:
		case ffi::DataType::S8: return FA2_MASK_U8;
		default: return 0;
	}
}

fa2_tensor dense4(void* ptr, ffi::Span<const int64_t> d) {
	fa2_tensor t;
	t.ptr = ptr;
	t.stride_b = d[1] * d[2] * d[3];
	t.stride_s = d[2] * d[3];
	t.stride_h = d[3];
	return t;
}

// Clears a result buffer on the stream.  A kernel, not hipMemsetAsync: XLA may record the custom call into a
// command buffer (a HIP graph), where memset nodes are not dependable.
__global__ void fill_zero_kernel(uint4* p, size_t n16) {
	size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
	const size_t step = (size_t)gridDim.x * blockDim.x;
	for (; i < n16; i += step) p[i] = uint4{0u, 0u, 0u, 0u};
}

struct Attrs {
	float scale, dropout_p;
	bool causal, bias_group, has_window;
	int32_t window_left, window_right;
	float softcap;
};

ffi::Error fill_common(fa2_params& p, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer bias,
                       ffi::AnyBuffer seqlens, ffi::AnyBuffer kv_lens, ffi::AnyBuffer seed, const Attrs& at) {
	std::memset(&p, 0, sizeof(p));
	p.struct_size = sizeof(p);
	auto qd = q.dimensions(), kd = k.dimensions();
	if (qd.size() != 4 || kd.size() != 4 || v.dimensions().size() != 4)
		return ffi::Error(ffi::ErrorCode::kInvalidArgument, "q, k, v must be [B, S, H, D]");
	p.dtype = elem_type(q.element_type());
	p.B = (int32_t)qd[0];
	p.Sq = (int32_t)qd[1];
	p.Hq = (int32_t)qd[2];
	p.D = (int32_t)qd[3];
	p.Sk = (int32_t)kd[1];
	p.Hkv = (int32_t)kd[2];
	p.causal = at.causal ? 1 : 0;
	p.scale = at.scale;
	p.p_drop = at.dropout_p;
	p.has_window = at.has_window ? 1 : 0;
	p.window_left = at.window_left;
	p.window_right = at.window_right;
	p.softcap = at.softcap;
	if (seed.size_bytes() != 8) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "seed must hold 8 bytes (u32[2] or one 64-bit integer)");
	p.seed_dev = (const uint64_t*)seed.untyped_data();
	p.q = dense4(q.untyped_data(), qd);
	p.k = dense4(k.untyped_data(), kd);
	p.v = dense4(v.untyped_data(), v.dimensions());
	if (bias.element_count() > 0) {
		auto bd = bias.dimensions();
		if (bd.size() != 4) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "bias must be 4-D");
		p.bias = bias.untyped_data();
		p.bias_dtype = elem_type(bias.element_type());
		if (!p.bias_dtype) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "bias must be f16, bf16, f32 or a boolean / byte mask");
		p.bias_stride_m = bd[3];
		p.bias_stride_h = bd[1] == 1 ? 0 : bd[2] * bd[3];
		p.bias_stride_b = bd[0] == 1 ? 0 : bd[1] * bd[2] * bd[3];
		p.bias_group = at.bias_group ? 1 : 0;
	}
	if (seqlens.element_count() > 0) {
		if (seqlens.element_type() != ffi::DataType::S32 || (int64_t)seqlens.element_count() != qd[0])
			return ffi::Error(ffi::ErrorCode::kInvalidArgument, "seqlens must be int32 [B]");
		p.seqlens = (const int32_t*)seqlens.untyped_data();
	}
	if (kv_lens.element_count() > 0) {
		if (kv_lens.element_type() != ffi::DataType::S32 || (int64_t)kv_lens.element_count() != qd[0])
			return ffi::Error(ffi::ErrorCode::kInvalidArgument, "kv_lens must be int32 [B]");
		p.kv_lens = (const int32_t*)kv_lens.untyped_data();
	}
	return ffi::Error::Success();
}

ffi::Error to_error(int rc) {
	if (rc == FA2_OK) return ffi::Error::Success();
	return ffi::Error(rc == FA2_EHIP ? ffi::ErrorCode::kInternal : ffi::ErrorCode::kInvalidArgument, fa2_strerror(rc));
}

ffi::Error FwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer bias,
                   ffi::AnyBuffer seqlens, ffi::AnyBuffer kv_lens, ffi::AnyBuffer seed, ffi::Result<ffi::AnyBuffer> o,
                   ffi::Result<ffi::AnyBuffer> lse, ffi::Result<ffi::AnyBuffer> scratch, float scale, float dropout_p, bool causal,
                   bool bias_group, bool has_window, int32_t window_left, int32_t window_right, float softcap) {
	fa2_params p;
	Attrs at{scale, dropout_p, causal, bias_group, has_window, window_left, window_right, softcap};
	if (auto e = fill_common(p, q, k, v, bias, seqlens, kv_lens, seed, at); e.failure()) return e;
	p.o = dense4(o->untyped_data(), q.dimensions());
	p.lse = (float*)lse->untyped_data();
	// optional: with fa2_fwd_scratch_bytes() of scratch a short query is split over key ranges
	p.scratch = scratch->untyped_data();
	p.scratch_bytes = scratch->size_bytes();
	return to_error(fa2_fwd(&p, stream));
}

ffi::Error BwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer bias,
                   ffi::AnyBuffer seqlens, ffi::AnyBuffer kv_lens, ffi::AnyBuffer seed, ffi::AnyBuffer o, ffi::AnyBuffer lse,
                   ffi::AnyBuffer dout, ffi::Result<ffi::AnyBuffer> dq, ffi::Result<ffi::AnyBuffer> dk, ffi::Result<ffi::AnyBuffer> dv,
                   ffi::Result<ffi::AnyBuffer> dbias, ffi::Result<ffi::AnyBuffer> scratch, float scale, float dropout_p, bool causal,
                   bool bias_group, bool has_window, int32_t window_left, int32_t window_right, float softcap) {
	fa2_params p;
	Attrs at{scale, dropout_p, causal, bias_group, has_window, window_left, window_right, softcap};
	if (auto e = fill_common(p, q, k, v, bias, seqlens, kv_lens, seed, at); e.failure()) return e;
	p.o = dense4(o.untyped_data(), q.dimensions());
	p.lse = (float*)lse.untyped_data();
	p.dout = dense4(dout.untyped_data(), q.dimensions());
	p.dq = dense4(dq->untyped_data(), q.dimensions());
	p.dk = dense4(dk->untyped_data(), k.dimensions());
	p.dv = dense4(dv->untyped_data(), v.dimensions());
	p.scratch = scratch->untyped_data();
	p.scratch_bytes = scratch->size_bytes();
	if (dbias->element_count() > 0) {
		// fp32, dense, in the shape of the bias ([B|1, Hq|Hkv|1, Sq, Sk]): stride 0 on its size-1 axes, where the dQ
		// kernel accumulates over batch rows / heads itself; it leaves key tiles it skips unwritten: cleared first
		auto dd = dbias->dimensions();
		auto bd = bias.dimensions();
		if (dd.size() != 4 || bd.size() != 4 || dbias->element_type() != ffi::DataType::F32 || dd[0] != bd[0] || dd[1] != bd[1] ||
		    dd[2] != p.Sq || dd[3] != p.Sk || dd[3] % 4)
			return ffi::Error(ffi::ErrorCode::kInvalidArgument, "dbias must be f32 in the shape of the bias, Sk a multiple of 4");
		p.dbias = (float*)dbias->untyped_data();
		p.dbias_stride_m = dd[3];
		p.dbias_stride_h = dd[1] == 1 ? 0 : dd[2] * dd[3];
		p.dbias_stride_b = dd[0] == 1 ? 0 : dd[1] * dd[2] * dd[3];
		size_t n16 = dbias->size_bytes() / 16;
		size_t blocks = (n16 + 255) / 256;
		hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)(blocks < 65535 ? blocks : 65535)), dim3(256), 0, stream, (uint4*)p.dbias, n16);
	}
	return to_error(fa2_bwd(&p, stream));
}

ffi::Error DropoutMaskImpl(hipStream_t stream, ffi::AnyBuffer seed, ffi::Result<ffi::AnyBuffer> keep, float dropout_p) {
	auto d = keep->dimensions();  // [B, H, Sq, Sk] u8
	if (d.size() != 4) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "keep must be [B, H, Sq, Sk]");
	fa2_params p;
	std::memset(&p, 0, sizeof(p));
	p.struct_size = sizeof(p);
	p.B = (int32_t)d[0];
	p.Hq = p.Hkv = (int32_t)d[1];
	p.Sq = (int32_t)d[2];
	p.Sk = (int32_t)d[3];
	p.p_drop = dropout_p;
	if (seed.size_bytes() != 8) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "seed must hold 8 bytes (u32[2] or one 64-bit integer)");
	p.seed_dev = (const uint64_t*)seed.untyped_data();
	return to_error(fa2_dropout_mask(&p, (uint8_t*)keep->untyped_data(), stream));
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(fa2_fwd_ffi, FwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // q
                                  .Arg<ffi::AnyBuffer>()  // k
                                  .Arg<ffi::AnyBuffer>()  // v
                                  .Arg<ffi::AnyBuffer>()  // bias
                                  .Arg<ffi::AnyBuffer>()  // seqlens
                                  .Arg<ffi::AnyBuffer>()  // kv_lens
                                  .Arg<ffi::AnyBuffer>()  // seed
                                  .Ret<ffi::AnyBuffer>()  // o
                                  .Ret<ffi::AnyBuffer>()  // lse
                                  .Ret<ffi::AnyBuffer>()  // scratch
                                  .Attr<float>("scale")
                                  .Attr<float>("dropout_p")
                                  .Attr<bool>("causal")
                                  .Attr<bool>("bias_group")
                                  .Attr<bool>("has_window")
                                  .Attr<int32_t>("window_left")
                                  .Attr<int32_t>("window_right")
                                  .Attr<float>("softcap"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(fa2_bwd_ffi, BwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // q
                                  .Arg<ffi::AnyBuffer>()  // k
                                  .Arg<ffi::AnyBuffer>()  // v
                                  .Arg<ffi::AnyBuffer>()  // bias
                                  .Arg<ffi::AnyBuffer>()  // seqlens
                                  .Arg<ffi::AnyBuffer>()  // kv_lens
                                  .Arg<ffi::AnyBuffer>()  // seed
                                  .Arg<ffi::AnyBuffer>()  // o
                                  .Arg<ffi::AnyBuffer>()  // lse
                                  .Arg<ffi::AnyBuffer>()  // dout
                                  .Ret<ffi::AnyBuffer>()  // dq
                                  .Ret<ffi::AnyBuffer>()  // dk
                                  .Ret<ffi::AnyBuffer>()  // dv
                                  .Ret<ffi::AnyBuffer>()  // dbias
                                  .Ret<ffi::AnyBuffer>()  // scratch
                                  .Attr<float>("scale")
                                  .Attr<float>("dropout_p")
                                  .Attr<bool>("causal")
                                  .Attr<bool>("bias_group")
                                  .Attr<bool>("has_window")
                                  .Attr<int32_t>("window_left")
                                  .Attr<int32_t>("window_right")
                                  .Attr<float>("softcap"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(fa2_dropout_mask_ffi, DropoutMaskImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // seed
                                  .Ret<ffi::AnyBuffer>()  // keep
                                  .Attr<float>("dropout_p"));
