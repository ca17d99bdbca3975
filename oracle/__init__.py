"""CPU oracle for the GEMM hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the product: only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import
it, and only as the checker.  The product (package `aster_amd`) never imports
it and has no CPU fallback.

What it restates, and from where in the reference:

* `gemm.py`     -- the reference's numerical check of every GEMM,
                   `A.astype(np.float32) @ B.astype(np.float32).T`
                   (contrib/kittens/test/bench/bench_harness.py:821, 1837;
                   contrib/kittens/test/test_102_gemm_python_multitile_g2s_directb_cdna4.py:481-483),
                   extended by the epilogue (scale, bias, cast) that the
                   reference does not have.
* `formats.py`  -- bf16, OCP e4m3 (the reference's converter,
                   test/integration/test_conversion_pack_e2e.py:91-167, gfx950 = OCP),
                   e2m1 / e8m0 and the OCP-MX block quantiser (published
                   closed form; the reference only defines the instruction,
                   include/aster/Dialect/AMDGCN/IR/MMA.td:765-803).
* `layouts.py`  -- `shuffle_weight` (contrib/kittens/test/kittens_helpers.py:90-119),
                   the LDS swizzles (python/aster/layout/algebra.py:153-171,
                   mlir_kernels/library/common/indexing.mlir:584-592) and the
                   MFMA fragment index maps (indexing.mlir:182-227).
* `cgemm.c`     -- the same GEMM formula as plain C (fp32 accumulate), used to
                   cross-check the numpy oracle and as a CPU baseline.

Pinning status (what fixes each function independently of its own formula):

* GEMM value: brute-force triple loop on tiny shapes, float64 BLAS, and the C
  restatement; the reference's closed-form known answers 32.0 / 16.0 (all-ones
  bf16 MFMA), 2240.0 and 186.0 (scaled fp8 MFMA,
  test/integration/test_mfma_f8f6f4_e2e.py:39-95).
* e4m3: the code points the reference's tests hold (0x38=1.0, 0x3E=1.75,
  0x3A=1.25, 0x3C=1.5, 0x40=2.0, 0x30=0.5, 0x7E=448; mfma-f8f6f4-e2e.mlir),
  exhaustive 256-code decode->encode round trip, `torch.float8_e4m3fn`.
* e8m0: 0x7F=1, 0x80=2, 0x81=4 from the same reference test.
* bf16: `torch.bfloat16` round trip on random and boundary values.
* e2m1 / MX quantiser: brute force over all 16 codes x scale bytes and the
  OCP-MX closed form; NOT pinned by any reference test or fixture (the
  reference has no MXFP4 data path) -- **parity unpinned** for
  `formats.quantize_mxfp4` and `gemm.gemm_mxfp4` against the reference.
* per-tensor fp8 scaling (`formats.quantize_fp8_tensor`, `gemm.gemm_fp8`):
  defined here by closed form; the reference has no such path --
  **parity unpinned** against the reference.
* `shuffle_weight`: its docstring's lane property checked by brute force, plus
  permutation / inverse invariants.
* swizzles: involution + bijection on a 1 KiB tile and the reference's bank
  tables' defining property (conflict-free 16-lane groups).
"""
