"""Host-only checks of the JAX side of the boundary (no jax, no GPU needed):

* the `Bind()` chains of csrc/fa2_xla_ffi.cc list exactly the operands, results and attributes of
  jax_flash_attn2/_ffi_spec.py, in the same order - the table `_jax_op.py` builds its `ffi_call`s from,
  the counterpart of the positional operand lists of the reference's `triton_call`s
  (_forward_triton.py:547-588, _backward_triton.py:1049-1154);
* the C++ signature of every handler takes what its chain binds;
* every field of `fa2_params` (include/fa2.h) is reachable from those operands and attributes;
* `_jax_op.py` spells no operand list of its own.
"""

import ast
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "jax-flash-attn2_amd"))

from jax_flash_attn2 import _ffi_spec as spec  # noqa: E402
from jax_flash_attn2 import _lib  # noqa: E402

CC = os.path.join(ROOT, "jax-flash-attn2_amd", "csrc", "fa2_xla_ffi.cc")
JAX_OP = os.path.join(ROOT, "jax-flash-attn2_amd", "jax_flash_attn2", "_jax_op.py")


def _chains():
	"""{handler symbol: (impl function, [operand names], [result names], [(attr name, C++ type)])} from the source text."""
	src = open(CC).read()
	out = {}
	for m in re.finditer(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(\w+)\s*,\s*(\w+)\s*,(.*?)\);\n", src, re.S):
		sym, impl, chain = m.group(1), m.group(2), m.group(3)
		assert ".Ctx<ffi::PlatformStream<hipStream_t>>()" in chain, sym
		args, rets, attrs = [], [], []
		order = []
		for line in chain.splitlines():
			a = re.search(r"\.Arg<ffi::AnyBuffer>\(\)\s*//\s*(\w+)", line)
			r = re.search(r"\.Ret<ffi::AnyBuffer>\(\)\s*//\s*(\w+)", line)
			t = re.search(r"\.Attr<(\w+)>\(\"(\w+)\"\)", line)
			if a:
				args.append(a.group(1))
				order.append("arg")
			elif r:
				rets.append(r.group(1))
				order.append("ret")
			elif t:
				attrs.append((t.group(2), t.group(1)))
				order.append("attr")
			else:
				assert ".Arg<" not in line and ".Ret<" not in line and ".Attr<" not in line, f"unparsed binding line: {line!r}"
		# XLA hands a handler its operands first, then its results, then its attributes
		assert order == sorted(order, key=["arg", "ret", "attr"].index), sym
		out[sym] = (impl, args, rets, attrs)
	return out


def test_bind_chains_match_the_spec_table():
	chains = _chains()
	assert set(chains) == set(spec.HANDLERS)
	for sym, (operands, results, attrs) in spec.HANDLERS.items():
		_, args, rets, cattrs = chains[sym]
		assert tuple(args) == tuple(operands), sym
		assert tuple(rets) == tuple(results), sym
		assert tuple(cattrs) == tuple(attrs), sym


def test_handler_signatures_take_what_the_chains_bind():
	src = open(CC).read()
	for sym, (impl, args, rets, attrs) in _chains().items():
		m = re.search(r"ffi::Error\s+" + impl + r"\((.*?)\)\s*\{", src, re.S)
		assert m, impl
		params = [p.strip() for p in re.sub(r"\s+", " ", m.group(1)).split(",")]
		assert params[0] == "hipStream_t stream"
		expect = [f"ffi::AnyBuffer {a}" for a in args] + [f"ffi::Result<ffi::AnyBuffer> {r}" for r in rets] + [f"{t} {n}" for n, t in attrs]
		assert params[1:] == expect, impl


def test_every_field_of_the_parameter_block_is_reachable():
	"""The fields of fa2_params, minus the ones the handler derives from buffer shapes, are each named by an operand,
	result or attribute of the forward or backward handler."""
	fields = {n for n, _ in _lib.Fa2Params._fields_}
	derived = {"struct_size", "dtype", "B", "Sq", "Sk", "Hq", "Hkv", "D", "seed"}  # seed: the host copy; the handlers use seed_dev
	covered = set()
	for sym in ("fa2_fwd_ffi", "fa2_bwd_ffi"):
		operands, results, attrs = spec.HANDLERS[sym]
		for n in list(operands) + list(results) + [a for a, _ in attrs]:
			for f in re.split(r"[,\s]+", re.sub(r"\(.*?\)", "", spec.PARAM_FIELDS[n])):
				if f.endswith("_*"):
					covered |= {x for x in fields if x.startswith(f[:-1])}
				elif f:
					covered.add(f)
	assert fields - derived <= covered, sorted(fields - derived - covered)
	# ... and the handler source assigns each of them
	src = open(CC).read()
	for f in sorted(fields - derived):
		assert re.search(r"\bp\." + f + r"\b\s*=", src), f"fa2_xla_ffi.cc never sets fa2_params.{f}"


def test_jax_operator_builds_its_calls_from_the_spec_table():
	"""_jax_op.py cannot be imported here (no jax): read as text.  Every ffi call goes through the lists of _ffi_spec."""
	src = open(JAX_OP).read()
	tree = ast.parse(src)
	names = {n.attr for n in ast.walk(tree) if isinstance(n, ast.Attribute) and isinstance(n.value, ast.Name) and n.value.id == "spec"}
	assert {"FWD_OPERANDS", "FWD_RESULTS", "BWD_OPERANDS", "BWD_RESULTS", "ATTRS", "HANDLERS"} <= names
	# the only literal handler names are the three targets
	called = set(re.findall(r"_ffi_call\(\"(\w+)\"", src))
	assert called == set(spec.HANDLERS)
	# a 4-D boolean mask is passed as bytes, never turned into a 16-bit bias on the host
	assert "finfo" not in re.sub(r'""".*?"""', "", src, flags=re.S)
	# the keyword-only operands of the torch operator exist on the jax operator as well
	fn = next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == "flash_attention")
	assert [a.arg for a in fn.args.kwonlyargs] == ["kv_lens", "window_size", "softcap", "bias_grad"]
	assert [a.arg for a in fn.args.args] == ["q", "k", "v", "attention_mask", "bias", "softmax_scale", "dropout_prob", "causal",
	                                         "dropout_seed", "varlen_mode"]  # _flash_attention.py:125-136
