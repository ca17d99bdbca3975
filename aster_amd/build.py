"""Ahead-of-time build of libastergemm.so for gfx950 with hipcc.

The reference JIT-compiles every GEMM through its MLIR pipeline
(`compile_mlir_module_to_asm` + `assemble_to_hsaco`,
python/aster/compiler/core.py:100-345); here the kernels are hand-written HIP
and are compiled once, in-tree, so the shared library travels with the source
tree.  `python -m aster_amd.build` rebuilds it.
"""

from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libastergemm.so")
OBJ_DIR = os.path.join(ROOT, "build", "obj")

SOURCES = ["gemm_tile.hip", "gemm_stream.hip", "gemm_skinny.hip", "astergemm_api.hip", "quantize.hip",
           "weight_artifact.hip", "diag_mfma_rate.hip"]
HSACO_SOURCE = "hsaco_kernels.hip"
HSACO_PATH = os.path.join(LIB_DIR, "astergemm_kernels.hsaco")
REPLAY_PATH = os.path.join(LIB_DIR, "astergemm_replay")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops off: hipcc must not form v_pk_{add,mul,fma}_f32 from the
# epilogue float math.
COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"),
    "-I" + CSRC,
]


def _compile(src: str) -> str:
    """Compile one source; the device assembly is kept beside the object and checked for the
    hazard `scan_mfma_hazards` describes."""
    stem = os.path.splitext(src)[0]
    obj = os.path.join(OBJ_DIR, stem + ".o")
    cmd = [HIPCC, *COMMON_FLAGS, "-save-temps=obj", "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    asm = os.path.join(OBJ_DIR, stem + "-hip-amdgcn-amd-amdhsa-gfx950.s")
    if not os.path.exists(asm):
        raise RuntimeError(f"hipcc left no device assembly for {src} (expected {asm})")
    with open(asm) as f:
        text = f.read()
    found = scan_mfma_hazards(text)
    spilled = scan_spills_beside_asm_loads(text)
    if spilled:
        raise RuntimeError(f"{src}: register spills in kernels whose register loads are inline assembly "
                           f"(the compiler does not wait for those loads): {spilled}")
    for name in os.listdir(OBJ_DIR):  # the other intermediates are large and of no use
        if name.startswith(stem + "-") and name.endswith((".hipi", ".bc", ".out", ".resolution.txt")):
            os.remove(os.path.join(OBJ_DIR, name))
    if found:
        lines = "\n".join(f"  {asm}:{no}: {mfma}\n      written at line {wno}: {writer}"
                          for (no, mfma, wno, writer) in found[:20])
        raise RuntimeError(f"{src}: {len(found)} inline-asm instruction(s) read a register a VALU instruction "
                           f"wrote too few wait states earlier (MFMA sources: {MFMA_WAIT_STATES}, scalar "
                           f"bases of vector-memory instructions: {VMEM_SGPR_WAIT_STATES}):\n{lines}")
    return obj


# ---- a hazard the compiler cannot see -----------------------------------------------------
#
# The stream kernels write some MFMAs as inline asm (to tie the accumulator to the accumulation
# registers).  The compiler's hazard recogniser does not look inside inline asm: where register
# allocation places a copy (v_mov, v_accvgpr_mov, v_and ...) into a source register right in front
# of such an MFMA, it inserts no wait states and the MFMA reads the register before the copy has
# landed: wrong sums, no error (seen on gfx950 with one v_mov_b64 directly in front of a
# v_mfma_scale_f32_16x16x128_f8f6f4).  The kernels keep such copies out of their K loops and put
# `s_nop 1` in front of the MFMAs elsewhere; this scan of the generated assembly is the proof.

MFMA_WAIT_STATES = 2
# The same blind spot for the transfers (global_load_lds_* / buffer_load_* written as inline asm with
# a scalar base): an SGPR written by a VALU instruction (v_readlane restoring a spilled SGPR,
# v_readfirstlane, a compare into an SGPR pair) must not be read by a vector-memory instruction
# for five wait states.
VMEM_SGPR_WAIT_STATES = 5

_REG_RANGE = re.compile(r"([va])\[(\d+):(\d+)\]$")
_REG_ONE = re.compile(r"([va])(\d+)$")


_SREG_RANGE = re.compile(r"s\[(\d+):(\d+)\]$")
_SREG_ONE = re.compile(r"s(\d+)$")


def _sregs(tok: str) -> set:
    tok = tok.strip().rstrip(",")
    m = _SREG_RANGE.match(tok)
    if m:
        return {("s", i) for i in range(int(m.group(1)), int(m.group(2)) + 1)}
    m = _SREG_ONE.match(tok)
    return {("s", int(m.group(1)))} if m else set()


def _regs(tok: str) -> set:
    tok = tok.strip().rstrip(",")
    m = _REG_RANGE.match(tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = _REG_ONE.match(tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


def scan_mfma_hazards(asm_text: str, wait_states: int = MFMA_WAIT_STATES):
    """[(line, instruction text, writer line, writer text)] for every MFMA inside an inline-asm block
    of gfx9 assembly text whose A, B, C or scale registers were written by a VALU instruction fewer
    than `wait_states` wait states earlier (an instruction is one wait state, `s_nop n` is n + 1),
    and for every vector-memory instruction inside an inline-asm block whose SGPR operands were
    written by a VALU instruction fewer than VMEM_SGPR_WAIT_STATES wait states earlier."""
    found = []
    hist = []      # (wait states, registers written by a VALU instruction, text, line)
    in_asm = False
    for no, raw in enumerate(asm_text.split("\n"), 1):
        l = raw.strip()
        if l.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if l.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not l or l[0] in ";." :
            continue
        if l.endswith(":"):
            if not l.startswith(".L"):
                hist = []          # a new function
            continue
        op = l.split()[0]
        args = l[len(op):].split(";")[0]
        toks = [t for t in re.split(r",\s*", args.strip()) if t]
        if op.startswith("v_mfma") or op.startswith("v_smfmac"):
            if in_asm:
                srcs = set()
                for t in toks[1:]:
                    if t.split():
                        srcs |= _regs(t.split()[0])
                ws = 0
                for (w, written, text, wno) in reversed(hist):
                    if ws >= wait_states:
                        break
                    if written & srcs:
                        found.append((no, l[:110], wno, text[:90]))
                    ws += w
            hist.append((1, set(), l, no))
        else:
            w, written = 1, set()
            if op == "s_nop":
                w = int(toks[0], 0) + 1 if toks else 1
            elif op.startswith(("v_readlane", "v_readfirstlane")) or \
                    (op.startswith("v_cmp") and toks and toks[0].startswith("s")):
                written = _sregs(toks[0]) if toks else set()
            elif op.startswith("v_") and not op.startswith("v_cmp"):
                written = _regs(toks[0]) if toks else set()
            if in_asm and op.startswith(("global_load", "global_store", "buffer_load", "buffer_store")):
                srcs = set()
                for t in toks:
                    if t.split():
                        srcs |= _sregs(t.split()[0])
                ws = 0
                for (w2, written2, text, wno) in reversed(hist):
                    if ws >= VMEM_SGPR_WAIT_STATES:
                        break
                    if written2 & srcs:
                        found.append((no, l[:110], wno, text[:90]))
                    ws += w2
            hist.append((w, written, l, no))
        if len(hist) > 12:
            hist.pop(0)
    return found


def scan_spills_beside_asm_loads(asm_text: str):
    """[(function, spill instructions)] for every function of gfx9 assembly text that loads
    registers inside inline-asm blocks (loads the kernel counts by hand: the compiler inserts no
    wait for them) and also holds register spills: a spill of such a register between the load and
    the kernel's own wait would store the bytes the register held before."""
    found = []
    name, asm_loads, spills, in_asm = None, 0, 0, False

    def close():
        if name and asm_loads and spills:
            found.append((name, spills))

    for raw in asm_text.split("\n"):
        l = raw.strip()
        if l.startswith(";;#ASMSTART"):
            in_asm = True
        elif l.startswith(";;#ASMEND"):
            in_asm = False
        elif l.endswith(":") and not l.startswith((".L", ";")):
            close()
            name, asm_loads, spills = l[:-1], 0, 0
        elif l and l[0] not in ";.":
            op = l.split()[0]
            if in_asm and op.startswith(("buffer_load_dword", "global_load_dword")) and "_lds_" not in op:
                asm_loads += 1
            elif op.startswith(("scratch_store", "scratch_load")):
                spills += 1
    close()
    return found


def _genco(src: str) -> str:
    """Device-only code object for module launchers (hipModuleLoadData)."""
    flags = [f for f in COMMON_FLAGS if f != "-fPIC"]
    cmd = [HIPCC, "--genco", *flags, os.path.join(CSRC, src), "-o", HSACO_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc --genco failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    return HSACO_PATH


def build_library(verbose: bool = False) -> str:
    """Compile every HIP source, link libastergemm.so and build the code object
    astergemm_kernels.hsaco; returns the library path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as pool:
        hsaco = pool.submit(_genco, HSACO_SOURCE)
        objs = list(pool.map(_compile, SOURCES))
        hsaco.result()
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC",
           "-Wno-unused-command-line-argument", *objs, "-o", LIB_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    # astergemm_replay: host-only program on top of the C-ABI, for profilers.
    cmd = ["g++", "-O2", "-std=c++17", "-I" + os.path.join(ROOT, "include"),
           os.path.join(CSRC, "astergemm_replay.cpp"), "-o", REPLAY_PATH,
           "-L" + LIB_DIR, "-lastergemm", "-Wl,-rpath,$ORIGIN"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"replay tool build failed:\n{proc.stdout}\n{proc.stderr}")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build_library(verbose=True)
    sys.exit(0)
