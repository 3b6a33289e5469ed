"""The C ABI without a GPU: the library loads, exports every symbol that
include/fa2.h declares, the ctypes mirror of fa2_params has the C layout, and
argument validation returns the documented codes.  No kernel is launched."""

import ctypes
import os
import re
import subprocess
import sys
import tempfile

import pytest

from jax_flash_attn2 import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fa2.h")


def _declared_functions():
	src = open(HEADER).read()
	src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
	return sorted(set(re.findall(r"\b(fa2_[a-z_0-9]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
	lib = _lib.load()
	names = _declared_functions()
	assert set(names) == set(_lib.EXPORTS)
	for n in names:
		assert hasattr(lib, n), n
	assert lib.fa2_version() >= 100


def test_struct_layout_matches_c():
	prog = r"""
#include <stdio.h>
#include <stddef.h>
#include "fa2.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(fa2_params), offsetof(fa2_params, seed), offsetof(fa2_params, q),
         offsetof(fa2_params, lse), offsetof(fa2_params, bias), offsetof(fa2_params, bias_stride_b),
         offsetof(fa2_params, seqlens), offsetof(fa2_params, dout), offsetof(fa2_params, scratch),
         offsetof(fa2_params, softcap), offsetof(fa2_params, dbias), offsetof(fa2_params, dbias_stride_m));
  return 0;
}"""
	with tempfile.TemporaryDirectory() as d:
		c = os.path.join(d, "t.c")
		open(c, "w").write(prog)
		exe = os.path.join(d, "t")
		subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe])
		got = [int(x) for x in subprocess.check_output([exe]).split()]
	P = _lib.Fa2Params
	want = [ctypes.sizeof(P)] + [getattr(P, f).offset for f in ("seed", "q", "lse", "bias", "bias_stride_b", "seqlens", "dout", "scratch", "softcap", "dbias", "dbias_stride_m")]
	assert got == want


def _good_params():
	p = _lib.new_params()
	p.dtype = _lib.FA2_BF16
	p.B, p.Sq, p.Sk, p.Hq, p.Hkv, p.D = 2, 128, 128, 8, 2, 128
	p.scale = 0.088
	for name in ("q", "k", "v", "o", "dout", "dq", "dk", "dv"):
		t = getattr(p, name)
		t.ptr = 0x10000
		t.stride_b, t.stride_s, t.stride_h = 128 * 8 * 128, 8 * 128, 128
	p.lse = 0x20000
	p.scratch = 0x30000
	p.scratch_bytes = 1 << 20
	return p


def _rc(p, which=0):
	return _lib.load().fa2_validate(ctypes.byref(p), which)


def test_validate_accepts_good_params():
	p = _good_params()
	assert _rc(p, 0) == 0 and _rc(p, 1) == 0
	assert _lib.load().fa2_bwd_scratch_bytes(ctypes.byref(p)) == 2 * 8 * 128 * 4


def test_parameter_block_of_the_first_header_version_is_accepted():
	"""struct_size of the block without the fields added later (seed_dev): the library fills them with zeros;
	anything shorter is refused."""
	P = _lib.Fa2Params
	v1 = P.seed_dev.offset
	p = _good_params()
	p.seed_dev = 0xdead0008  # beyond struct_size: must not be looked at
	p.struct_size = v1
	assert _rc(p, 0) == 0 and _rc(p, 1) == 0
	assert _lib.load().fa2_bwd_scratch_bytes(ctypes.byref(p)) == 2 * 8 * 128 * 4
	p.struct_size = v1 - 8
	assert _rc(p, 0) == -1
	# a misaligned device seed pointer is refused
	p = _good_params()
	p.seed_dev = 0x60004
	assert _rc(p, 0) == -5


@pytest.mark.parametrize(
	"mutate,code",
	[
		(lambda p: setattr(p, "struct_size", 8), -1),
		(lambda p: setattr(p, "dtype", 3), -2),  # fp32 q/k/v: "Only support fp16 and bf16"
		(lambda p: setattr(p, "Sq", 0), -3),
		(lambda p: setattr(p, "Hkv", 3), -4),
		(lambda p: setattr(p.q, "ptr", 0), -5),
		(lambda p: setattr(p.k, "ptr", 0x10008), -5),
		(lambda p: setattr(p.v, "stride_s", 1028), -6),
		(lambda p: setattr(p.k, "stride_s", 1 << 24), -6),  # rows of a tile no longer within 32-bit byte offsets
		(lambda p: setattr(p.q, "stride_s", -1024), -6),
		(lambda p: setattr(p, "p_drop", 1.0), -7),
		(lambda p: setattr(p, "p_drop", -0.1), -7),
		(lambda p: (setattr(p, "bias", 0x40000), setattr(p, "bias_dtype", 7)), -8),
		(lambda p: (setattr(p, "bias", 0x40000), setattr(p, "bias_dtype", 2), setattr(p, "bias_stride_m", 64)), -8),
		(lambda p: (setattr(p, "seqlens", 0x50000), setattr(p, "Sk", 256)), -9),
		(lambda p: (setattr(p, "seqlens", 0x50000), setattr(p, "bias", 0x40000), setattr(p, "bias_dtype", 2),
		            setattr(p, "bias_stride_m", 128)), -9),
		(lambda p: setattr(p, "D", 96), -10),
	],
)
def test_validate_error_codes(mutate, code):
	p = _good_params()
	mutate(p)
	assert _rc(p, 0) == code
	assert _lib.strerror(code) != "unknown error"


def test_validate_backward_scratch():
	p = _good_params()
	p.scratch_bytes = 16
	assert _rc(p, 1) == -11 and _rc(p, 0) == 0
	p = _good_params()
	p.scratch = 0
	assert _rc(p, 1) == -11
	p = _good_params()
	p.dq.ptr = 0
	assert _rc(p, 1) == -5
	lib = _lib.load()
	# errors never reach a launch: NULL stream and bogus pointers are fine here
	assert lib.fa2_bwd(ctypes.byref(p), None) == -5
	assert lib.fa2_fwd(None, None) == -1
	assert lib.fa2_dropout_mask(ctypes.byref(p), None, None) == -5


def test_validate_bias_gradient_buffer():
	def with_dbias(**kw):
		p = _good_params()
		p.bias, p.bias_dtype, p.bias_stride_m = 0x40000, 2, 128
		p.dbias = 0x50000
		p.dbias_stride_b, p.dbias_stride_h, p.dbias_stride_m = 8 * 128 * 128, 128 * 128, 128
		for k, v in kw.items():
			setattr(p, k, v)
		return p

	assert _rc(with_dbias(), 1) == 0
	assert _rc(with_dbias(), 0) == 0                       # the forward does not look at it
	assert _rc(with_dbias(bias=0), 1) == -8                # no additive term in the kernels: nothing to differentiate
	assert _rc(with_dbias(bias=0, softcap=2.0), 1) == 0    # ... unless soft-capping selects the variants that carry one
	assert _rc(with_dbias(dbias=0x50004), 1) == -8         # rows are stored 16 bytes at a time
	assert _rc(with_dbias(dbias_stride_m=126), 1) == -8
	assert _rc(with_dbias(dbias_stride_m=64), 1) == -8     # shorter than a row
	assert _rc(with_dbias(dbias_stride_h=-4), 1) == -8


def test_missing_library_fails_loudly(monkeypatch):
	monkeypatch.setattr(_lib, "_lib", None)
	monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libfa2_hip.so")
	with pytest.raises(ImportError):
		_lib.load()


def test_forward_scratch_only_for_small_grids_over_many_keys():
	"""fa2_fwd_scratch_bytes: non-zero exactly where the split forward applies (too few row tiles to fill the chip, many keys)."""
	lib = _lib.load()

	def need(B, Sq, Sk, Hq, D=128):
		p = _lib.new_params()
		p.B, p.Sq, p.Sk, p.Hq, p.Hkv, p.D = B, Sq, Sk, Hq, Hq, D
		return lib.fa2_fwd_scratch_bytes(ctypes.byref(p))

	assert need(4, 4096, 4096, 32) == 0          # training shape: one pass
	assert need(1, 1, 256, 8) == 0               # too few keys to split
	assert need(64, 1, 8192, 32) == 0            # enough (batch, head) pairs already
	n = need(1, 1, 8192, 8)
	assert n > 0 and n % 256 == 0
	# ranges x rows x (D values + logsumexp) floats, rounded up to 256 bytes
	assert n >= 2 * 8 * (128 + 1) * 4 and n <= 64 * 8 * (128 + 1) * 4 + 256
	n2 = need(1, 65, 8192, 8)                    # two row tiles of 64: still far from filling the chip
	assert n2 > 0 and n2 % 256 == 0
	assert need(1, 4096, 4096, 8) == 0           # 512 row tiles of 64: enough already
	assert need(2, 512, 512, 16, 64) == 0        # 256 row tiles over 8 key tiles: too short a kernel for a second launch
	assert need(1, 1024, 1024, 16, 64) == 0      # 256 row tiles over 16 key tiles: the same
	assert need(1, 2048, 2048, 8, 64) > 0        # 256 row tiles over 32 key tiles: split
	assert need(1, 1024, 1024, 8, 64) > 0        # 128 row tiles over 16 key tiles: split


def test_backward_split_scratch_only_on_small_grids():
	"""fa2_bwd_split_scratch_bytes: non-zero exactly where the dK/dV kernel may split the steps of a key tile over
	workgroups - delta plus one fp32 [B, Hkv, Sk, 2, D] partial per part (at most 8; enough to fill the chip and, for causal
	launches, to even out key tiles of different length)."""
	lib = _lib.load()

	def need(B, S, Hq, Hkv, D=128, causal=0):
		p = _lib.new_params()
		p.B, p.Sq, p.Sk, p.Hq, p.Hkv, p.D, p.causal = B, S, S, Hq, Hkv, D, causal
		return lib.fa2_bwd_split_scratch_bytes(ctypes.byref(p)), lib.fa2_bwd_scratch_bytes(ctypes.byref(p))

	assert need(4, 4096, 32, 8)[0] == 0        # 4 x 8 x 32 workgroups fill the chip
	assert need(1, 4096, 32, 8)[0] == 0        # 256 workgroups: one per CU already
	n, base = need(1, 2048, 16, 4)             # 1 x 4 x 16 = 64 workgroups: 4 parts
	assert n == base + 4 * (1 * 4 * 2048 * 2 * 128 * 4)
	n, base = need(1, 2048, 8, 8)              # 128 workgroups: 2 parts, also with one q-head per kv-head
	assert n == base + 2 * (1 * 8 * 2048 * 2 * 128 * 4)
	n, base = need(1, 1024, 12, 2, 64)         # 16 workgroups: the limit of 8 parts
	assert n == base + 8 * (1 * 2 * 1024 * 2 * 64 * 4)
	n, base = need(1, 512, 6, 2, 64)           # 12 steps of 128 rows per key tile: at most 6 parts
	assert n == base + 6 * (1 * 2 * 512 * 2 * 64 * 4)
	assert need(2, 512, 8, 8)[0] == 0          # only 4 steps per key tile: the split would cost more than it saves
	assert need(1, 100, 2, 2)[0] == 0
	# causal key tiles differ in length: fewer than 512 workgroups are split further - up to 128 into 8 parts of at least
	# 16 steps, more towards 1024 parts of at least 64 steps (but at least 2 parts)
	n, base = need(1, 4096, 32, 8, causal=1)   # 256 workgroups, 128 steps: 2 parts
	assert n == base + 2 * (1 * 8 * 4096 * 2 * 128 * 4)
	n, base = need(4, 4096, 32, 2, causal=1)   # 256 workgroups, 512 steps: 4 parts
	assert n == base + 4 * (4 * 2 * 4096 * 2 * 128 * 4)
	n, base = need(4, 4096, 32, 1, causal=1)   # 128 workgroups, 1024 steps: 8 parts
	assert n == base + 8 * (4 * 1 * 4096 * 2 * 128 * 4)
	n, base = need(3, 4096, 32, 4, causal=1)   # 384 workgroups: 3 parts
	assert n == base + 3 * (3 * 4 * 4096 * 2 * 128 * 4)
	n, base = need(2, 4096, 8, 2, causal=1)    # 128 workgroups, 128 steps: 8 parts of 16 steps
	assert n == base + 8 * (2 * 2 * 4096 * 2 * 128 * 4)
	n, base = need(1, 4096, 8, 8, causal=1)    # 256 workgroups, 32 steps: 2 parts
	assert n == base + 2 * (1 * 8 * 4096 * 2 * 128 * 4)
	assert need(2, 4096, 32, 8, causal=1)[0] == 0   # 512 workgroups pack well unsplit
	assert need(4, 4096, 32, 8, causal=1)[0] == 0
	n, base = need(1, 2048, 8, 8, causal=1)    # 16 steps: the 2 parts that fill the chip, no more
	assert n == base + 2 * (1 * 8 * 2048 * 2 * 128 * 4)
