"""Runs the host logic of jax_flash_attn2/_jax_op.py without jax.

jax is not installed in this image, so the module cannot meet the real library here.  What CAN be executed is
everything in it that is plain Python: operand preparation, the seed split, the attribute dictionary, result
shapes, the order in which operands reach the custom call, the differentiation rule's plumbing and the head-dim
padding.  The test installs a minimal stand-in for the few jax entry points the module touches (arrays are NumPy
arrays, `ffi_call` records its call and returns zero-filled results, `custom_vjp` runs the forward rule and keeps
the residuals) and checks every recorded call against jax_flash_attn2/_ffi_spec.py.  It proves nothing about jax
itself - only that this module's own code runs and hands over what the handlers in csrc/fa2_xla_ffi.cc bind.
"""

import importlib
import os
import sys
import types

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "jax-flash-attn2_amd"))


class _CustomVjp:
	def __init__(self, fun, nondiff_argnums=()):
		self.fun, self.nondiff = fun, tuple(nondiff_argnums)

	def defvjp(self, fwd, bwd):
		self.fwd, self.bwd = fwd, bwd

	def __call__(self, *args):
		out, self.residual = self.fwd(*args)
		self.static = tuple(args[i] for i in self.nondiff)
		return out

	def pullback(self, dout):
		return self.bwd(*self.static, self.residual, dout)


def _install_fake_jax(monkeypatch, calls):
	jnp = types.ModuleType("jax.numpy")
	for name in ("zeros", "asarray", "stack", "pad", "float16", "float32", "uint8", "int8", "int32", "uint32", "uint64", "bool_",
	             "issubdtype", "floating"):
		setattr(jnp, name, getattr(np, name))
	jnp.bfloat16 = np.dtype("V2")  # no bfloat16 in NumPy: a placeholder that no array here has

	class ShapeDtypeStruct:
		def __init__(self, shape, dtype):
			self.shape, self.dtype = tuple(shape), dtype

	def ffi_call(name, out_types, vmap_method=None):
		def run(*operands, **attrs):
			calls.append((name, operands, attrs, out_types, vmap_method))
			outs = tuple(np.zeros(t.shape, t.dtype) for t in (out_types if isinstance(out_types, tuple) else (out_types,)))
			return outs if isinstance(out_types, tuple) else outs[0]

		return run

	ffi = types.ModuleType("jax.ffi")
	ffi.ffi_call = ffi_call
	ffi.register_ffi_target = lambda *a, **k: None
	ffi.pycapsule = lambda f: f
	jax = types.ModuleType("jax")
	jax.numpy, jax.ffi = jnp, ffi
	jax.ShapeDtypeStruct = ShapeDtypeStruct
	jax.custom_vjp = _CustomVjp
	for name, mod in (("jax", jax), ("jax.numpy", jnp), ("jax.ffi", ffi)):
		monkeypatch.setitem(sys.modules, name, mod)


@pytest.fixture
def jop(monkeypatch):
	calls = []
	_install_fake_jax(monkeypatch, calls)
	monkeypatch.delitem(sys.modules, "jax_flash_attn2._jax_op", raising=False)
	mod = importlib.import_module("jax_flash_attn2._jax_op")
	monkeypatch.setattr(mod, "_registered", True)  # no libfa2_xla_ffi.so here
	yield mod, calls
	sys.modules.pop("jax_flash_attn2._jax_op", None)


def _qkv(B=2, Sq=128, Sk=128, Hq=4, Hkv=2, D=64):
	rng = np.random.default_rng(0)
	f = lambda *s: rng.standard_normal(s).astype(np.float16)
	return f(B, Sq, Hq, D), f(B, Sk, Hkv, D), f(B, Sk, Hkv, D)


def test_forward_and_backward_calls_follow_the_binding_order(jop):
	from jax_flash_attn2 import _ffi_spec as spec

	mod, calls = jop
	q, k, v = _qkv()
	bias = np.zeros((2, 2, 128, 128), np.float32)  # Hkv heads -> bias_group
	out = mod.flash_attention(q, k, v, bias=bias, causal=True, dropout_prob=0.1, dropout_seed=(5 << 32) | 7, kv_lens=[100, 128],
	                          window_size=(64, 0), softcap=30.0, bias_grad=True)
	assert out.shape == q.shape and out.dtype == q.dtype
	name, operands, attrs, out_types, vmap_method = calls[-1]
	assert name == "fa2_fwd_ffi" and vmap_method == "sequential"
	assert len(operands) == len(spec.FWD_OPERANDS) and len(out_types) == len(spec.FWD_RESULTS)
	ops = dict(zip(spec.FWD_OPERANDS, operands))
	assert ops["q"] is q and ops["k"] is k and ops["v"] is v and ops["bias"] is bias
	assert ops["seqlens"].size == 0 and ops["seqlens"].dtype == np.int32
	assert ops["kv_lens"].dtype == np.int32 and ops["kv_lens"].tolist() == [100, 128]
	assert ops["seed"].dtype == np.uint32 and ops["seed"].tolist() == [7, 5]  # low word first, all 64 bits
	assert list(attrs) == [n for n, _ in spec.ATTRS]
	assert attrs["causal"] is True and attrs["bias_group"] is True and attrs["has_window"] is True
	assert (int(attrs["window_left"]), int(attrs["window_right"])) == (64, 0)
	assert isinstance(attrs["scale"], np.float32) and abs(float(attrs["scale"]) - 0.125) < 1e-7
	assert abs(float(attrs["softcap"]) - 30.0) < 1e-6 and abs(float(attrs["dropout_p"]) - 0.1) < 1e-6
	res = dict(zip(spec.FWD_RESULTS, out_types))
	assert res["o"].shape == q.shape and res["lse"].shape == (2, 4, 128) and res["scratch"].dtype == np.uint8
	# the differentiation rule: same operands plus o, lse, dout; dbias as a result in the shape of the bias
	grads = mod._attention.pullback(np.ones_like(q))
	name, operands, attrs, out_types, _ = calls[-1]
	assert name == "fa2_bwd_ffi" and len(operands) == len(spec.BWD_OPERANDS)
	ops = dict(zip(spec.BWD_OPERANDS, operands))
	assert ops["o"].shape == q.shape and ops["lse"].shape == (2, 4, 128) and ops["dout"].shape == q.shape
	assert ops["seed"].tolist() == [7, 5] and ops["kv_lens"].tolist() == [100, 128]
	res = dict(zip(spec.BWD_RESULTS, out_types))
	assert res["dbias"].shape == bias.shape and res["dbias"].dtype == np.float32  # not one entry per (batch, q-head)
	assert res["dk"].shape == k.shape and res["dv"].shape == v.shape
	dq, dk, dv, dbias, *rest = grads
	assert dq.shape == q.shape and dk.shape == k.shape and dbias.shape == bias.shape and rest == [None, None, None]


def test_boolean_mask_goes_to_the_kernels_as_bytes(jop):
	mod, calls = jop
	q, k, v = _qkv()
	mask = np.ones((2, 1, 128, 128), np.int32)
	mod.flash_attention(q, k, v, attention_mask=mask)
	ops = dict(zip(("q", "k", "v", "bias"), calls[-1][1]))
	assert ops["bias"].dtype == np.bool_ and ops["bias"].shape == mask.shape  # one byte per position, no 16-bit bias
	assert calls[-1][2]["bias_group"] is False
	grads = mod._attention.pullback(np.ones_like(q))
	assert calls[-1][3][3].shape == (0,)  # no dbias wanted
	assert grads[3] is None
	# 2-D right-padded mask -> lengths
	m2 = np.zeros((2, 128), np.int32)
	m2[0, :50] = 1
	m2[1, :128] = 1
	mod.flash_attention(q, k, v, attention_mask=m2)
	assert calls[-1][1][4].tolist() == [50, 128] and calls[-1][1][3].size == 0
	with pytest.raises(AssertionError):
		mod.flash_attention(q, k, v, attention_mask=mask, bias=np.zeros((2, 1, 128, 128), np.float32))
	with pytest.raises(ValueError):
		mod.flash_attention(q, k, v, attention_mask=mask, bias_grad=True)


@pytest.mark.parametrize("seed,expect", [(None, [0, 0]), (42, [42, 0]), (2 ** 31, [2 ** 31, 0]), (2 ** 63 + 5, [5, 2 ** 31]),
                                         (np.int64(2 ** 40 + 3), [3, 256]), (np.array(7, np.int32), [7, 0]),
                                         (np.array([9, 1], np.uint32), [9, 1])])
def test_seed_operand(jop, seed, expect):
	mod, _ = jop
	x = mod._seed_operand(seed)
	assert x.dtype == np.uint32 and x.tolist() == expect


def test_other_head_dims_are_padded_and_cut(jop):
	mod, calls = jop
	q, k, v = _qkv(D=80)
	out = mod.flash_attention(q, k, v)
	assert out.shape == q.shape
	assert calls[-1][1][0].shape[-1] == 128 and np.array_equal(calls[-1][1][0][..., :80], q) and not calls[-1][1][0][..., 80:].any()
	assert abs(float(calls[-1][2]["scale"]) - 80 ** -0.5) < 1e-7  # the scale keeps the true head dim
	with pytest.raises(ValueError):
		mod.flash_attention(*_qkv(D=320))
