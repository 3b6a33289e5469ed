"""ctypes binding of libfa2_hip.so (the C ABI declared in include/fa2.h).

This is the only place the shared library is opened.  There is no fallback:
if the library is missing every call raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

FA2_FP16, FA2_BF16, FA2_FP32, FA2_MASK_U8 = 1, 2, 3, 4

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libfa2_hip.so")


class Fa2Tensor(ctypes.Structure):
	_fields_ = [
		("ptr", ctypes.c_void_p),
		("stride_b", ctypes.c_int64),
		("stride_s", ctypes.c_int64),
		("stride_h", ctypes.c_int64),
	]


class Fa2Params(ctypes.Structure):
	_fields_ = [
		("struct_size", ctypes.c_uint32),
		("dtype", ctypes.c_int32),
		("B", ctypes.c_int32),
		("Sq", ctypes.c_int32),
		("Sk", ctypes.c_int32),
		("Hq", ctypes.c_int32),
		("Hkv", ctypes.c_int32),
		("D", ctypes.c_int32),
		("causal", ctypes.c_int32),
		("scale", ctypes.c_float),
		("p_drop", ctypes.c_float),
		("seed", ctypes.c_uint64),
		("q", Fa2Tensor),
		("k", Fa2Tensor),
		("v", Fa2Tensor),
		("o", Fa2Tensor),
		("lse", ctypes.c_void_p),
		("bias", ctypes.c_void_p),
		("bias_dtype", ctypes.c_int32),
		("bias_group", ctypes.c_int32),
		("bias_stride_b", ctypes.c_int64),
		("bias_stride_h", ctypes.c_int64),
		("bias_stride_m", ctypes.c_int64),
		("seqlens", ctypes.c_void_p),
		("dout", Fa2Tensor),
		("dq", Fa2Tensor),
		("dk", Fa2Tensor),
		("dv", Fa2Tensor),
		("scratch", ctypes.c_void_p),
		("scratch_bytes", ctypes.c_uint64),
		("seed_dev", ctypes.c_void_p),
		("kv_lens", ctypes.c_void_p),
		("has_window", ctypes.c_int32),
		("window_left", ctypes.c_int32),
		("window_right", ctypes.c_int32),
		("softcap", ctypes.c_float),
		("dbias", ctypes.c_void_p),
		("dbias_stride_b", ctypes.c_int64),
		("dbias_stride_h", ctypes.c_int64),
		("dbias_stride_m", ctypes.c_int64),
	]


EXPORTS = (
	"fa2_fwd",
	"fa2_bwd",
	"fa2_bwd_stages",
	"fa2_bwd_static",
	"fa2_bwd_scratch_bytes",
	"fa2_bwd_split_scratch_bytes",
	"fa2_fwd_scratch_bytes",
	"fa2_dropout_mask",
	"fa2_validate",
	"fa2_strerror",
	"fa2_version",
)

_lib = None
_lock = threading.Lock()


class Fa2Error(RuntimeError):
	def __init__(self, code: int, message: str):
		super().__init__(f"libfa2_hip: {message} (code {code})")
		self.code = code


def load() -> ctypes.CDLL:
	"""Open libfa2_hip.so once and declare the prototypes of include/fa2.h."""
	global _lib
	if _lib is not None:
		return _lib
	with _lock:
		if _lib is not None:
			return _lib
		if not os.path.exists(LIB_PATH):
			raise ImportError(
				f"{LIB_PATH} is missing: build it with `make -C {os.path.join(os.path.dirname(_HERE), 'csrc')}` "
				"(there is no non-HIP fallback for this path)"
			)
		lib = ctypes.CDLL(LIB_PATH)
		pp = ctypes.POINTER(Fa2Params)
		lib.fa2_fwd.argtypes = [pp, ctypes.c_void_p]
		lib.fa2_fwd.restype = ctypes.c_int
		lib.fa2_bwd.argtypes = [pp, ctypes.c_void_p]
		lib.fa2_bwd.restype = ctypes.c_int
		lib.fa2_bwd_stages.argtypes = [pp, ctypes.c_void_p, ctypes.c_int]
		lib.fa2_bwd_stages.restype = ctypes.c_int
		lib.fa2_bwd_static.argtypes = [pp, ctypes.c_void_p]
		lib.fa2_bwd_static.restype = ctypes.c_int
		lib.fa2_bwd_scratch_bytes.argtypes = [pp]
		lib.fa2_bwd_scratch_bytes.restype = ctypes.c_size_t
		lib.fa2_bwd_split_scratch_bytes.argtypes = [pp]
		lib.fa2_bwd_split_scratch_bytes.restype = ctypes.c_size_t
		lib.fa2_fwd_scratch_bytes.argtypes = [pp]
		lib.fa2_fwd_scratch_bytes.restype = ctypes.c_size_t
		lib.fa2_dropout_mask.argtypes = [pp, ctypes.c_void_p, ctypes.c_void_p]
		lib.fa2_dropout_mask.restype = ctypes.c_int
		lib.fa2_validate.argtypes = [pp, ctypes.c_int]
		lib.fa2_validate.restype = ctypes.c_int
		lib.fa2_strerror.argtypes = [ctypes.c_int]
		lib.fa2_strerror.restype = ctypes.c_char_p
		lib.fa2_version.argtypes = []
		lib.fa2_version.restype = ctypes.c_int
		_lib = lib
	return _lib


def strerror(code: int) -> str:
	return load().fa2_strerror(code).decode()


def check(code: int) -> None:
	if code != 0:
		raise Fa2Error(code, strerror(code))


def new_params() -> Fa2Params:
	p = Fa2Params()
	p.struct_size = ctypes.sizeof(Fa2Params)
	return p
