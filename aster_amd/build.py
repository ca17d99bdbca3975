"""Ahead-of-time build of libastergemm.so for gfx950 with hipcc.

The reference JIT-compiles every GEMM through its MLIR pipeline
(`compile_mlir_module_to_asm` + `assemble_to_hsaco`,
python/aster/compiler/core.py:100-345); here the kernels are hand-written HIP
and are compiled once, in-tree, so the shared library travels with the source
tree.  `python -m aster_amd.build` rebuilds it.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

from .asm_scan import (MFMA_WAIT_STATES, VMEM_SGPR_WAIT_STATES, scan_mfma_hazards,  # noqa: F401
                       scan_spills_beside_asm_loads)

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libastergemm.so")
OBJ_DIR = os.path.join(ROOT, "build", "obj")

# (object stem, source file, extra flags).  gemm_stream.hip holds the variant table of the stream
# kernels in four parts (bf16, fp8, MXFP4, f16 operands) and is compiled once per part.
UNITS = [("gemm_stream_p0", "gemm_stream.hip", ["-DAG_STREAM_PART=0"]),
         ("gemm_stream_p3", "gemm_stream.hip", ["-DAG_STREAM_PART=3"]),
         ("gemm_stream_p2", "gemm_stream.hip", ["-DAG_STREAM_PART=2"]),
         ("gemm_stream_p1", "gemm_stream.hip", ["-DAG_STREAM_PART=1"]),
         ("gemm_skinny", "gemm_skinny.hip", []),
         ("gemm_tile", "gemm_tile.hip", []),
         ("astergemm_api", "astergemm_api.hip", []),
         ("quantize", "quantize.hip", []),
         ("weight_artifact", "weight_artifact.hip", []),
         ("diag_mfma_rate", "diag_mfma_rate.hip", [])]
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


def _compile(unit) -> str:
    """Compile one unit; the device assembly is kept beside the object and checked for the
    hazard `scan_mfma_hazards` describes."""
    stem, src, extra = unit
    # a directory per unit: the intermediates kept by -save-temps are named after the source file
    udir = os.path.join(OBJ_DIR, stem)
    os.makedirs(udir, exist_ok=True)
    obj = os.path.join(udir, stem + ".o")
    cmd = [HIPCC, *COMMON_FLAGS, *extra, "-save-temps=obj", "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    sstem = os.path.splitext(src)[0]
    asm = os.path.join(udir, sstem + "-hip-amdgcn-amd-amdhsa-gfx950.s")
    if not os.path.exists(asm):
        raise RuntimeError(f"hipcc left no device assembly for {src} (expected {asm})")
    with open(asm) as f:
        text = f.read()
    found = scan_mfma_hazards(text)
    spilled = scan_spills_beside_asm_loads(text)
    if spilled:
        raise RuntimeError(f"{src}: register spills (scratch, accumulation registers or the metadata's "
                           f"spill counts) in kernels whose register loads are inline assembly "
                           f"(the compiler does not wait for those loads): {spilled}")
    for name in os.listdir(udir):  # the other intermediates are large and of no use
        if name.startswith(sstem + "-") and name.endswith((".hipi", ".bc", ".out", ".resolution.txt")):
            os.remove(os.path.join(udir, name))
    if found:
        lines = "\n".join(f"  {asm}:{no}: {mfma}\n      written at line {wno}: {writer}"
                          for (no, mfma, wno, writer) in found[:20])
        raise RuntimeError(f"{src}: {len(found)} inline-asm instruction(s) read a register a VALU instruction "
                           f"wrote too few wait states earlier (MFMA sources: {MFMA_WAIT_STATES}, scalar "
                           f"bases of vector-memory instructions: {VMEM_SGPR_WAIT_STATES}):\n{lines}")
    return obj


PLAN_HEADER = os.path.join(CSRC, "stream_load_plan.inc")


def write_generated_sources() -> None:
    """The stream kernels' staging constants come from the cooperative load plan of
    `aster_amd.coop` (the host-side mirror of the reference's make_coop_load_plan): the header the
    kernels include is written from it, so a change of the plan changes the kernels."""
    from .coop import stream_load_plan_header

    text = stream_load_plan_header()
    old = None
    if os.path.exists(PLAN_HEADER):
        with open(PLAN_HEADER) as f:
            old = f.read()
    if old != text:
        with open(PLAN_HEADER, "w") as f:
            f.write(text)


def _genco(src: str) -> str:
    """Device-only code object for module launchers (hipModuleLoadData)."""
    flags = [f for f in COMMON_FLAGS if f != "-fPIC"]
    cmd = [HIPCC, "--genco", *flags, os.path.join(CSRC, src), "-o", HSACO_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc --genco failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    return HSACO_PATH


def build_library(verbose: bool = False, only=None) -> str:
    """Compile every HIP source, link libastergemm.so and build the code object
    astergemm_kernels.hsaco; returns the library path.  `only` (a list of unit names, for work
    on one kernel file) recompiles just those and links them with the objects already there."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    write_generated_sources()
    with ThreadPoolExecutor(max_workers=8) as pool:
        if only:
            todo = [u for u in UNITS if u[0] in only]
            list(pool.map(_compile, todo))
            objs = [os.path.join(OBJ_DIR, u[0], u[0] + ".o") for u in UNITS]
            missing = [o for o in objs if not os.path.exists(o)]
            if missing:
                raise RuntimeError(f"objects missing for a partial build: {missing}")
        else:
            hsaco = pool.submit(_genco, HSACO_SOURCE)
            objs = list(pool.map(_compile, UNITS))
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
    build_library(verbose=True, only=sys.argv[1:] or None)
    sys.exit(0)
