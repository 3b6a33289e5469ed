#!/usr/bin/env python3
"""Build-time check of the register hazards around matrix products issued as inline assembly.

The kernels issue some v_mfma instructions through inline assembly (so that the register file
of every operand can be pinned).  The compiler treats such a statement as opaque: it neither
pads the wait states a matrix product needs nor keeps its source registers untouched while
the product runs.  The sources keep those distances by construction; this script reads the
assembly text the compiler emits for the same translation unit (`hipcc -S`, no binary is
taken apart) and fails the build when a later compiler version, or an edit, breaks one.

Rules, per kernel, in program-text order along fall-through paths (the scan follows the text and
forgets what is pending at an unconditional branch; a v_mfma between `;;#ASMSTART` and `;;#ASMEND`):
  R1  the product's C operand, when it is not also its destination, is not written by any
      instruction before one further v_mfma has been issued (or 7 wait states have passed):
      an 8-pass product reads C while it runs, and the hardware does not hold back a
      vector-ALU write to those registers;
  R2  the product's destination is not read by anything but a v_mfma C operand before two
      further v_mfma have been issued (or 11 wait states have passed).
  R3  (over the kernel's control-flow graph, not the text order; every v_mfma, also the compiler's own)
      no register of a matrix product's operands is read at a point that some path from the kernel's
      entry reaches without writing it.  Seen with this compiler: a four-register operand spilled as
      three registers to scratch memory plus one kept in a spare accumulation register, and reloaded
      as three registers only - the product then read a stale fourth.  The build switches that kind of
      spill off (-mllvm -amdgpu-spill-vgpr-to-agpr=0); this rule is the check that no operand is left
      partly unwritten.  (Other instructions are not checked: under a divergent branch the compiler
      legitimately reads registers that are only written for the lanes that use them.)
  R4  (loops that stream tiles: blocks the compiler marks `Depth=2` or deeper) no access to scratch memory, and no
      `s_waitcnt vmcnt` that a matrix product follows in the same block - unless the block itself loads values from
      global memory into registers (the variants that read bias or mask values one by one).  The counter behind
      vmcnt also counts the direct-to-LDS copies of the next tile, which are issued at the start of a step: a spill
      reload or a late wait for a value loaded before the loop makes every step wait for those copies.
      A violation fails the build for the kernel variants without bias and without dropout (the first two boolean
      template arguments); for the other variants, whose register budget is tighter, it is printed as a note.
A wait state is one instruction; `s_nop N` counts N + 1.

Usage: asm_lint.py FILE.s [FILE.s ...]   (exit status 1 and one line per violation)
"""

from __future__ import annotations

import re
import sys

R1_WAIT = 7
R2_WAIT = 11

_LABEL = re.compile(r"^([A-Za-z_][\w$]*):\s*(;.*)?$")  # a function label (local labels start with a dot)
_REG = re.compile(r"\b([va])(?:\[(\d+):(\d+)\]|(\d+))")


def _regs(operand: str):
	"""Set of (file, index) named by one operand."""
	out = set()
	for m in _REG.finditer(operand):
		f = m.group(1)
		if m.group(4) is not None:
			out.add((f, int(m.group(4))))
		else:
			out.update((f, i) for i in range(int(m.group(2)), int(m.group(3)) + 1))
	return out


def _split(line: str):
	line = line.split(";")[0].strip()
	if not line or line.endswith(":") or line.startswith("."):
		return None, []
	parts = line.split(None, 1)
	ops = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
	return parts[0], ops


def _writes(mn: str, ops):
	"""Registers an instruction writes (vector files only)."""
	if not ops:
		return set()
	if mn.startswith(("v_cmp", "v_readfirstlane", "v_readlane", "s_", "ds_write", "ds_store", "global_store", "buffer_store",
	                  "flat_store", "global_atomic", "global_load_lds", "buffer_wbl2", "buffer_inv")):
		return set()
	if mn.startswith(("v_swap", "v_permlane")):
		return _regs(ops[0]) | (_regs(ops[1]) if len(ops) > 1 else set())
	if mn.startswith(("v_", "ds_read", "ds_load", "ds_bpermute", "ds_permute", "ds_swizzle", "global_load", "buffer_load", "flat_load",
	                  "scratch_load")):
		return _regs(ops[0])
	return set()


def _reads(mn: str, ops):
	if not ops:
		return set()
	if mn.startswith(("ds_write", "ds_store", "global_store", "buffer_store", "flat_store", "global_atomic", "global_load_lds")):
		src = ops
	else:
		src = ops[1:]
	out = set()
	for o in src:
		out |= _regs(o)
	return out


def lint(path: str):
	problems = []
	kernel = "?"
	in_asm = False
	pending = []  # dicts: line, c (set or None), dst (set), mfma_since, wait_since
	with open(path) as f:
		for ln, raw in enumerate(f, 1):
			s = raw.strip()
			if s.startswith(";;#ASMSTART"):
				in_asm = True
				continue
			if s.startswith(";;#ASMEND"):
				in_asm = False
				continue
			m = _LABEL.match(s)
			if m:
				kernel = m.group(1)
				pending = []
				continue
			mn, ops = _split(raw)
			if mn is None:
				continue
			is_mfma = mn.startswith("v_mfma")
			w, r = _writes(mn, ops), _reads(mn, ops)
			if is_mfma and len(ops) >= 4:
				r_nonc = _regs(ops[1]) | _regs(ops[2])
			else:
				r_nonc = r
			for p in pending:
				if p["c"] and p["mfma"] < 1 and p["wait"] < R1_WAIT and (w & p["c"]):
					problems.append(f"{path}:{ln}: {kernel}: R1: `{s}` writes the C operand of the product at line {p['line']}")
				if p["mfma"] < 2 and p["wait"] < R2_WAIT and (r_nonc & p["dst"]):
					problems.append(f"{path}:{ln}: {kernel}: R2: `{s}` reads the result of the product at line {p['line']}")
			# advance the clocks
			step = 1
			if mn == "s_nop" and ops:
				try:
					step = int(ops[0], 0) + 1
				except ValueError:
					pass
			for p in pending:
				p["wait"] += step
				if is_mfma:
					p["mfma"] += 1
			pending = [p for p in pending if p["mfma"] < 2 and p["wait"] < max(R1_WAIT, R2_WAIT)]
			if mn in ("s_branch", "s_endpgm", "s_setpc_b64"):
				pending = []  # the next line of text is not reached from here
			if is_mfma and in_asm and len(ops) >= 4:
				dst, c = _regs(ops[0]), _regs(ops[3])
				pending.append({"line": ln, "c": (c if c and c != dst else None), "dst": dst, "mfma": 0, "wait": 0})
	return problems


_DEPTH = re.compile(r"^(\.L[\w$]+):.*Depth=(\d+)")


def lint_loops(path: str):
	"""Rule R4: nothing in a tile loop waits on the memory counter that the tile copies share."""
	problems, notes = [], []
	kernel = "?"
	blocks = []  # (label, depth, [(ln, text)])
	cur = None

	def flush():
		flags = re.findall(r"Lb([01])E", kernel)[:2]
		strict = flags == ["0", "0"]
		out = problems if strict else notes
		# variants that read bias or mask values one by one load into registers inside the loops: their waits are their own
		loads = any(t.startswith(("global_load_", "buffer_load_", "flat_load_")) and not t.startswith("global_load_lds")
		            for _, depth, insts in blocks if depth >= 2 for _, t in insts)
		for label, depth, insts in blocks:
			if depth < 2 or loads:
				continue
			for i, (ln, t) in enumerate(insts):
				if t.startswith(("scratch_load", "scratch_store")):
					out.append(f"{path}:{ln}: {kernel}: R4: scratch access `{t.split(';')[0].strip()}` inside a tile loop ({label})")
				elif t.startswith("s_waitcnt") and "vmcnt" in t:
					if any(u.startswith("v_mfma") for _, u in insts[i + 1:]):
						out.append(f"{path}:{ln}: {kernel}: R4: `{t}` ahead of matrix products inside a tile loop ({label})")

	with open(path) as f:
		for ln, raw in enumerate(f, 1):
			s = raw.strip()
			m = _LABEL.match(s)
			if m:
				flush()
				kernel, blocks, cur = m.group(1), [], None
				continue
			if s.startswith(".Lfunc_end"):
				flush()
				blocks, cur = [], None
				continue
			md = _DEPTH.match(s)
			if md:
				cur = (md.group(1), int(md.group(2)), [])
				blocks.append(cur)
				continue
			if _BLOCK.match(s):
				cur = None  # a block outside any loop
				continue
			if cur is not None and s and not s.startswith((";", ".")):
				cur[2].append((ln, s))
	flush()
	return problems, notes


_TARGET = re.compile(r"^(s_cbranch_\w+|s_branch)\s+(\S+)")
_BLOCK = re.compile(r"^(\.L[\w$]+):")


def _bit(reg):
	return 1 << (reg[1] + (512 if reg[0] == "a" else 0))


def _mask(regs):
	m = 0
	for r in regs:
		m |= _bit(r)
	return m


def lint_defined(path: str):
	"""Rule R3: definite assignment of vector registers over each kernel's control-flow graph."""
	problems = []
	kernels = []  # (name, [(ln, text)])
	cur = None
	with open(path) as f:
		for ln, raw in enumerate(f, 1):
			s = raw.strip()
			m = _LABEL.match(s)
			if m:
				cur = (m.group(1), [])
				kernels.append(cur)
				continue
			if cur is None:
				continue
			if s.startswith(".Lfunc_end"):
				cur = None
				continue
			cur[1].append((ln, s))
	for name, lines in kernels:
		# basic blocks: a label starts one, a branch or the end of the program ends one
		blocks = []  # dict: label, insts [(ln, text, reads, writes)], succ labels, falls
		blk = {"label": None, "insts": [], "succ": [], "falls": True}
		for ln, s in lines:
			mb = _BLOCK.match(s)
			if mb:
				if blk["insts"] or blk["label"] is not None:
					blocks.append(blk)
				blk = {"label": mb.group(1), "insts": [], "succ": [], "falls": True}
				continue
			mn, ops = _split(s)
			if mn is None:
				continue
			blk["insts"].append((ln, s, _mask(_reads(mn, ops)) if mn.startswith("v_mfma") else 0, _mask(_writes(mn, ops))))
			mt = _TARGET.match(s)
			if mt or mn in ("s_endpgm", "s_setpc_b64"):
				if mt:
					blk["succ"].append(mt.group(2))
				blk["falls"] = bool(mt) and mt.group(1) != "s_branch"
				blocks.append(blk)
				blk = {"label": None, "insts": [], "succ": [], "falls": True}
		if blk["insts"] or blk["label"] is not None:
			blocks.append(blk)
		if not blocks:
			continue
		index = {b["label"]: i for i, b in enumerate(blocks) if b["label"] is not None}
		preds = [[] for _ in blocks]
		for i, b in enumerate(blocks):
			for t in b["succ"]:
				if t in index:
					preds[index[t]].append(i)
			if b["falls"] and i + 1 < len(blocks):
				preds[i + 1].append(i)
		full = (1 << 1024) - 1
		gen = []
		for b in blocks:
			g = 0
			for _, _, _, w in b["insts"]:
				g |= w
			gen.append(g)
		out = [full] * len(blocks)
		entry = _bit(("v", 0))
		changed = True
		while changed:
			changed = False
			for i in range(len(blocks)):
				if i == 0:
					inn = entry
				else:
					inn = full
					for p in preds[i]:
						inn &= out[p]
					if not preds[i]:
						inn = full  # unreachable
				o = inn | gen[i]
				if o != out[i]:
					out[i] = o
					changed = True
		reported = 0
		for i, b in enumerate(blocks):
			if i == 0:
				have = entry
			else:
				have = full
				for p in preds[i]:
					have &= out[p]
			for ln, s, r, w in b["insts"]:
				miss = r & ~have & ~reported
				if miss:
					reported |= miss
					names = [("a%d" % (k - 512)) if k >= 512 else ("v%d" % k) for k in range(1024) if (miss >> k) & 1]
					problems.append(f"{path}:{ln}: {name}: R3: `{s}` reads {', '.join(names)}, unwritten on some path from the entry")
				have |= w
	return problems


def main(argv):
	if len(argv) < 2:
		print(__doc__)
		return 2
	bad = []
	for path in argv[1:]:
		bad += lint(path)
		bad += lint_defined(path)
		p4, n4 = lint_loops(path)
		bad += p4
		for n in n4:
			print("note: " + n)
	for b in bad:
		print(b)
	if bad:
		print(f"asm_lint: {len(bad)} hazard(s)")
		return 1
	return 0


if __name__ == "__main__":
	sys.exit(main(sys.argv))
