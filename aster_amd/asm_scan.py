"""Checks of the generated gfx950 device assembly that the build runs on every source.

Some kernels write MFMAs, global->LDS transfers and register loads as inline assembly (to tie the
accumulators to the accumulation registers, to count `vmcnt` by hand).  The compiler's hazard
recogniser and its wait-count insertion do not look inside inline assembly, so two kinds of
mistakes can only be found in the assembly text:

* a VALU write into a source register of an inline-asm MFMA, or into a scalar operand of an
  inline-asm vector-memory instruction, too few wait states in front of it (`scan_mfma_hazards`);
* a register that an inline-asm load is still filling being copied elsewhere by the register
  allocator, to scratch memory or into an accumulation register (`scan_spills_beside_asm_loads`).

The scans follow branches: at a local label the instruction history is the set of histories of
every path that reaches the label (the fall-through and every branch to it, the back-edge of a loop
included), so a write at the bottom of a loop followed by an MFMA at its head is seen.
"""

from __future__ import annotations

import re

MFMA_WAIT_STATES = 2
# An SGPR written by a VALU instruction (v_readlane restoring a spilled SGPR, v_readfirstlane, a
# compare into an SGPR pair) must not be read by a vector-memory instruction for five wait states.
VMEM_SGPR_WAIT_STATES = 5

_HIST = 8            # entries of history kept per path (>= the largest wait-state requirement)
_MAX_PATHS = 16      # distinct histories kept at one point

_REG_RANGE = re.compile(r"([va])\[(\d+):(\d+)\]$")
_REG_ONE = re.compile(r"([va])(\d+)$")
_SREG_RANGE = re.compile(r"s\[(\d+):(\d+)\]$")
_SREG_ONE = re.compile(r"s(\d+)$")


def _sregs(tok: str) -> frozenset:
    tok = tok.strip().rstrip(",")
    m = _SREG_RANGE.match(tok)
    if m:
        return frozenset(("s", i) for i in range(int(m.group(1)), int(m.group(2)) + 1))
    m = _SREG_ONE.match(tok)
    return frozenset({("s", int(m.group(1)))}) if m else frozenset()


def _regs(tok: str) -> frozenset:
    tok = tok.strip().rstrip(",")
    m = _REG_RANGE.match(tok)
    if m:
        return frozenset((m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1))
    m = _REG_ONE.match(tok)
    return frozenset({(m.group(1), int(m.group(2)))}) if m else frozenset()


def parse(asm_text: str):
    """[(line number, kind, payload)] with kind in 'func' (payload = name), 'label' (name),
    'asm' (True at ;;#ASMSTART, False at ;;#ASMEND) and 'inst' (opcode, [operand tokens], text).
    Directives and comments are dropped; a label may carry a trailing comment."""
    out = []
    for no, raw in enumerate(asm_text.split("\n"), 1):
        l = raw.strip()
        if l.startswith(";;#ASMSTART"):
            out.append((no, "asm", True))
            continue
        if l.startswith(";;#ASMEND"):
            out.append((no, "asm", False))
            continue
        code = l.split(";")[0].strip()
        if not code:
            continue
        if code.endswith(":") and " " not in code and "\t" not in code:
            name = code[:-1]
            out.append((no, "label" if name.startswith(".L") else "func", name))
            continue
        if code[0] == ".":
            continue
        op = code.split()[0]
        toks = [t for t in re.split(r",\s*", code[len(op):].strip()) if t]
        out.append((no, "inst", (op, toks, code)))
    return out


def _written_by_valu(op: str, toks):
    """Registers whose write by this instruction an inline-asm consumer has to wait for."""
    if not toks:
        return frozenset()
    if op.startswith(("v_readlane", "v_readfirstlane")) or (op.startswith("v_cmp") and toks[0].startswith("s")):
        return _sregs(toks[0])
    if op.startswith("v_") and not op.startswith("v_cmp"):
        return _regs(toks[0])
    return frozenset()


def _branch_target(op: str, toks):
    if op in ("s_branch",) or op.startswith("s_cbranch"):
        for t in toks:
            if t.startswith(".L"):
                return t.split()[0]
    return None


def _dedupe(paths):
    seen, out = set(), []
    for p in paths:
        key = tuple(e[3] for e in p)
        if key not in seen:
            seen.add(key)
            out.append(p)
        if len(out) >= _MAX_PATHS:
            break
    return out


def scan_mfma_hazards(asm_text: str, wait_states: int = MFMA_WAIT_STATES):
    """[(line, instruction text, writer line, writer text)] for every MFMA inside an inline-asm block
    of gfx9 assembly text whose A, B, C or scale registers were written by a VALU instruction fewer
    than `wait_states` wait states earlier (an instruction is one wait state, `s_nop n` is n + 1) on
    any path that reaches it, and for every vector-memory instruction inside an inline-asm block
    whose SGPR operands were written by a VALU instruction fewer than VMEM_SGPR_WAIT_STATES wait
    states earlier."""
    items = parse(asm_text)
    snapshots = {}          # label -> histories at the branches that jump to it
    found = {}
    for _ in range(3):      # histories at back-edges are known one pass later; they settle at once
        new_snap = {}
        found = {}
        paths = [()]        # each history: tuple of (wait states, registers written, text, line)
        in_asm = False
        for no, kind, pay in items:
            if kind == "asm":
                in_asm = pay
                continue
            if kind == "func":
                paths = [()]
                continue
            if kind == "label":
                paths = _dedupe(list(paths) + snapshots.get(pay, []))
                if not paths:
                    paths = [()]
                continue
            op, toks, text = pay
            w, written = 1, frozenset()
            is_mfma = op.startswith(("v_mfma", "v_smfmac"))
            is_vmem = op.startswith(("global_load", "global_store", "buffer_load", "buffer_store"))
            if is_mfma:
                if in_asm:
                    srcs = set()
                    for t in toks[1:]:
                        if t.split():
                            srcs |= _regs(t.split()[0])
                    _check(paths, srcs, wait_states, no, text, found)
            else:
                if op == "s_nop":
                    w = int(toks[0], 0) + 1 if toks else 1
                else:
                    written = _written_by_valu(op, toks)
                if in_asm and is_vmem:
                    srcs = set()
                    for t in toks:
                        if t.split():
                            srcs |= _sregs(t.split()[0])
                    _check(paths, srcs, VMEM_SGPR_WAIT_STATES, no, text, found)
            entry = (w, written, text, no)
            paths = [(p + (entry,))[-_HIST:] for p in paths]
            if len(paths) > 1:
                paths = _dedupe(paths)
            tgt = _branch_target(op, toks)
            if tgt is not None:
                new_snap.setdefault(tgt, [])
                new_snap[tgt] = _dedupe(new_snap[tgt] + list(paths))
            if op in ("s_branch", "s_endpgm") or op.startswith("s_setpc"):
                paths = []          # nothing falls through
        if new_snap == snapshots:
            break
        snapshots = new_snap
    return sorted(found.values())


def _check(paths, srcs, need, no, text, found):
    for p in paths:
        ws = 0
        for (w, written, wtext, wno) in reversed(p):
            if ws >= need:
                break
            if written & srcs:
                found[(no, wno)] = (no, text[:110], wno, wtext[:90])
            ws += w


_ASM_REG_LOAD = ("buffer_load_dword", "global_load_dword", "buffer_load_b", "global_load_b")
_META_KEY = re.compile(r"^(?:  - | {4})\.(\w+):\s*(.*)$")


def kernel_spill_counts(asm_text: str) -> dict:
    """{kernel name: .vgpr_spill_count + .sgpr_spill_count} from the `.amdgpu_metadata` block of
    gfx9 assembly text (the kernel-level keys sit at the first level of each `amdhsa.kernels`
    list item; argument entries, one level deeper, have names of their own and are skipped)."""
    out, in_meta, cur = {}, False, None
    for raw in asm_text.split("\n"):
        s = raw.strip()
        if s.startswith(".amdgpu_metadata"):
            in_meta = True
            continue
        if s.startswith(".end_amdgpu_metadata"):
            in_meta = False
        if not in_meta:
            continue
        line = raw.replace("\t", "    ") if raw.startswith("\t") else raw
        if line.startswith("  - ."):
            cur = {"name": None, "spills": 0}
            out[id(cur)] = cur
        m = _META_KEY.match(line)
        if m and cur is not None:
            if m.group(1) == "name":
                cur["name"] = m.group(2).strip()
            elif m.group(1) in ("vgpr_spill_count", "sgpr_spill_count"):
                cur["spills"] += int(m.group(2))
    return {c["name"]: c["spills"] for c in out.values() if c["name"]}


def scan_spills_beside_asm_loads(asm_text: str):
    """[(function, count)] for every function of gfx9 assembly text that loads registers inside
    inline-asm blocks (loads the kernel counts by hand: the compiler inserts no wait for them) and
    in which the register allocator moved registers on its own: scratch stores / loads, copies of
    a register that such a load writes into an accumulation register (`v_accvgpr_write_b32 aN, vM`
    outside inline assembly: gfx950 spills vector registers there first), or a non-zero
    `.vgpr_spill_count` / `.sgpr_spill_count` in the kernel's metadata.  A copy of such a register
    between the load and the kernel's own wait would keep the bytes the register held before."""
    items = parse(asm_text)
    funcs = {}       # name -> dict(loads, dests, spills, agpr)
    order = []
    cur, in_asm = None, False
    for no, kind, pay in items:
        if kind == "asm":
            in_asm = pay
        elif kind == "func":
            cur = {"loads": 0, "dests": set(), "spills": 0, "agpr": []}
            funcs[pay] = cur
            order.append(pay)
        elif kind == "inst" and cur is not None:
            op, toks, text = pay
            if in_asm and op.startswith(_ASM_REG_LOAD) and "_lds_" not in op:
                cur["loads"] += 1
                if toks:
                    cur["dests"] |= {r for (f, r) in _regs(toks[0]) if f == "v"}
            elif op.startswith(("scratch_store", "scratch_load")):
                cur["spills"] += 1
            elif not in_asm and op.startswith("v_accvgpr_write") and len(toks) >= 2:
                cur["agpr"].append({r for (f, r) in _regs(toks[1]) if f == "v"})
    meta = kernel_spill_counts(asm_text)
    found = []
    for name in order:
        f = funcs[name]
        if not f["loads"]:
            continue
        count = f["spills"] + sum(1 for srcs in f["agpr"] if srcs & f["dests"]) + meta.get(name, 0)
        if count:
            found.append((name, count))
    return found
