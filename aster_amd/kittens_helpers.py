"""Host helpers of the GEMM family: B pre-shuffle and pipeline-strategy table.

Mirrors contrib/kittens/test/kittens_helpers.py:90-169 of the reference.  The
MLIR-template plumbing of that file (library paths, `run_kittens_kernel`,
`{{...}}` substitutions) belongs to the compiler path that this build does not
have.
"""

from __future__ import annotations

import numpy as np

_STAGE_KEYS = ("A_LOAD", "A_LDS_WRITE", "A_LDS_READ", "B_LOAD", "B_LDS_WRITE", "B_LDS_READ",
               "COMPUTE")

# Stage index of every op class, one row per strategy, columns as _STAGE_KEYS
# (reference: PIPELINE_STRATEGIES, kittens_helpers.py:137-157).  The reference
# feeds these to its SCF pipeliner; here they only describe prefetch distance
# for the resource estimators and for labels.
_STAGE_ROWS = (
    (0, 0, 0, 0, 0, 0, 0),
    (0, 1, 1, 1, 1, 1, 1),
    (0, 0, 1, 0, 1, 1, 1),
    (0, 1, 2, 0, 1, 2, 2),
    (0, 2, 2, 0, 1, 2, 2),
    (0, 1, 2, 2, 2, 2, 3),
    (0, 2, 2, 1, 1, 2, 3),
    (0, 2, 3, 0, 2, 3, 4),
    (0, 1, 3, 0, 2, 3, 4),
    (0, 3, 4, 0, 3, 4, 5),
    (0, 2, 4, 0, 3, 4, 5),
    (0, 1, 3, 0, 1, 4, 4),
    (0, 1, 3, 1, 2, 4, 4),
    (0, 1, 3, 0, 2, 4, 4),
)
PIPELINE_STRATEGIES = {i: dict(zip(_STAGE_KEYS, row)) for i, row in enumerate(_STAGE_ROWS)}


def pipeline_strategy_stages(strategy: int):
    """(a_stages, b_stages): deepest stage index + 1 on each operand's chain
    (reference: kittens_helpers.py:161-169)."""
    s = PIPELINE_STRATEGIES[strategy]
    a = max(s["A_LOAD"], s["A_LDS_WRITE"], s["A_LDS_READ"], s["COMPUTE"]) + 1
    b = max(s["B_LOAD"], s["B_LDS_WRITE"], s["B_LDS_READ"], s["COMPUTE"]) + 1
    return a, b


def shuffle_weight(B: np.ndarray) -> np.ndarray:
    """Pre-shuffle B[N, K] (2-byte elements) so that each lane's 16-byte load is
    its MFMA operand for two 16x16x16 K-steps.

    Same result as the reference's `shuffle_weight` (kittens_helpers.py:90-119):
    view B as (n_block, n_lane=16, k_block, k_half=2, lane_group=4, k_within=4)
    and store it in the order (n_block, k_block, lane_group, n_lane, k_half,
    k_within).  Lane d of block (nb, kb) then finds
    B[nb*16 + d%16, kb*32 + kh*16 + (d//16)*4 + 0..3] for kh = 0, 1 contiguous.
    """
    N, K = B.shape
    if N % 16 != 0:
        raise AssertionError(f"N={N} must be multiple of 16")
    if K % 32 != 0:
        raise AssertionError(f"K={K} must be multiple of 32")
    view = B.reshape(N // 16, 16, K // 32, 2, 4, 4)
    return np.ascontiguousarray(np.moveaxis(view, (0, 2, 4, 1, 3, 5), (0, 1, 2, 3, 4, 5))).reshape(N, K)


def unshuffle_weight(Bs: np.ndarray) -> np.ndarray:
    """Inverse of `shuffle_weight`."""
    N, K = Bs.shape
    view = Bs.reshape(N // 16, K // 32, 4, 16, 2, 4)
    return np.ascontiguousarray(view.transpose(0, 3, 1, 4, 2, 5)).reshape(N, K)


def shuffle_weight_k8(B: np.ndarray) -> np.ndarray:
    """Pre-shuffle B[N, K] (2-byte elements) for the 16x16x32 MFMA read with 16-byte operand
    loads: view B as (n_block, n_lane=16, k_block, lane_group=4, k_within=8) and store it in
    the order (n_block, k_block, lane_group, n_lane, k_within).  Lane d of block (nb, kb) then
    finds B[nb*16 + d%16, kb*32 + (d//16)*8 + 0..7] contiguous.  The reference's
    `shuffle_weight` (kittens_helpers.py:90-119) is the same idea for A fragments read with
    two ds_read_b64 (K elements {4g..4g+3} and {16+4g..16+4g+3} per lane); this is the order
    for ds_read_b128, which the HIP stream kernel with operand_path direct_b_k8 uses."""
    N, K = B.shape
    if N % 16 != 0:
        raise AssertionError(f"N={N} must be multiple of 16")
    if K % 32 != 0:
        raise AssertionError(f"K={K} must be multiple of 32")
    view = B.reshape(N // 16, 16, K // 32, 4, 8)
    return np.ascontiguousarray(view.transpose(0, 2, 3, 1, 4)).reshape(N, K)


def unshuffle_weight_k8(Bs: np.ndarray) -> np.ndarray:
    """Inverse of `shuffle_weight_k8`."""
    N, K = Bs.shape
    view = Bs.reshape(N // 16, K // 32, 4, 16, 8)
    return np.ascontiguousarray(view.transpose(0, 3, 1, 2, 4)).reshape(N, K)


def shuffle_weight_bytes(B: np.ndarray) -> np.ndarray:
    """Pre-shuffle the byte rows of an fp8 (B[N, K] uint8) or MXFP4 (B[N, K/2] uint8 nibble
    pairs) weight matrix into STEP ORDER, the operand order of the 16x16x128 MFMA, which takes
    the 16-byte pieces q and 4 + q of a 128-byte step of a row: view B as (n_block, n_lane=16,
    step, half=2, lane_group=4, 16 bytes) and store it in the order (n_block, step, half,
    lane_group, n_lane, 16 bytes).  Lane d of the KiB (nb, step, half) then finds bytes
    [(4 half + d // 16) * 16, + 16) of row 16 nb + d % 16 at byte 16 d.  The reference's
    `shuffle_weight` (kittens_helpers.py:90-119) is the same idea for 2-byte elements and the
    16x16x16 MFMA; it has no byte-type form."""
    B = np.ascontiguousarray(B)
    if B.dtype.itemsize != 1 or B.ndim != 2:
        raise AssertionError("shuffle_weight_bytes takes a 2-D array of one-byte elements")
    N, rb = B.shape
    if N % 16 != 0:
        raise AssertionError(f"N={N} must be multiple of 16")
    if rb % 128 != 0:
        raise AssertionError(f"rows of {rb} bytes are not whole 128-byte steps")
    view = B.reshape(N // 16, 16, rb // 128, 2, 4, 16)
    return np.ascontiguousarray(view.transpose(0, 2, 3, 4, 1, 5)).reshape(N, rb)


def unshuffle_weight_bytes(Bs: np.ndarray) -> np.ndarray:
    """Inverse of `shuffle_weight_bytes`."""
    N, rb = Bs.shape
    view = np.ascontiguousarray(Bs).reshape(N // 16, rb // 128, 2, 4, 16, 16)
    return np.ascontiguousarray(view.transpose(0, 4, 1, 2, 3, 5)).reshape(N, rb)


def shuffle_scales_e8m0(S: np.ndarray) -> np.ndarray:
    """The e8m0 plane S[N, K/32] of pre-shuffled MXFP4 weights in the matching order: view it as
    (n_block, n_lane=16, step, 8 bytes) and store (n_block, step, n_lane, 8 bytes), so that the
    scales of a row block and 256-element step are one 128-byte line."""
    S = np.ascontiguousarray(S, dtype=np.uint8)
    N, nb = S.shape
    if N % 16 != 0:
        raise AssertionError(f"N={N} must be multiple of 16")
    if nb % 8 != 0:
        raise AssertionError(f"{nb} scale bytes per row are not whole 256-element steps")
    view = S.reshape(N // 16, 16, nb // 8, 8)
    return np.ascontiguousarray(view.transpose(0, 2, 1, 3)).reshape(N, nb)


def unshuffle_scales_e8m0(Ss: np.ndarray) -> np.ndarray:
    """Inverse of `shuffle_scales_e8m0`."""
    N, nb = Ss.shape
    view = np.ascontiguousarray(Ss).reshape(N // 16, nb // 8, 16, 8)
    return np.ascontiguousarray(view.transpose(0, 2, 1, 3)).reshape(N, nb)


def shuffle_scales_e8m0_lanes(S: np.ndarray) -> np.ndarray:
    """The e8m0 plane S[N, K/32] of pre-shuffled MXFP4 weights in LANE ORDER, for the stream
    kernel that loads B straight into MFMA operands: view it as (group of 64 rows, tile t=4,
    row i=16, step, half h=2, lane group q=4) and store (group, step, q, i, t, h), so that lane
    16 q + i of a wave finds, in the 8 bytes at 8 (16 q + i) of the 512 bytes of (group, step),
    the scales of blocks q (h = 0) and 4 + q (h = 1) of its row in each of the wave's four
    16-row tiles: the byte pairs the two MFMAs of a 256-element step select with op_sel."""
    S = np.ascontiguousarray(S, dtype=np.uint8)
    N, nb = S.shape
    if N % 64 != 0:
        raise AssertionError(f"N={N} must be multiple of 64")
    if nb % 8 != 0:
        raise AssertionError(f"{nb} scale bytes per row are not whole 256-element steps")
    view = S.reshape(N // 64, 4, 16, nb // 8, 2, 4)
    return np.ascontiguousarray(view.transpose(0, 3, 5, 2, 1, 4)).reshape(N, nb)


def unshuffle_scales_e8m0_lanes(Ss: np.ndarray) -> np.ndarray:
    """Inverse of `shuffle_scales_e8m0_lanes`."""
    N, nb = Ss.shape
    view = np.ascontiguousarray(Ss).reshape(N // 64, nb // 8, 4, 16, 4, 2)
    return np.ascontiguousarray(view.transpose(0, 4, 3, 1, 5, 2)).reshape(N, nb)


def mx_lanes128_bytes(M: int, K: int) -> int:
    """Bytes of an activation e8m0 plane in lane order: whole groups of 128 rows."""
    return ((M + 127) // 128) * (K // 256) * 1024


def shuffle_scales_e8m0_lanes128(S: np.ndarray) -> np.ndarray:
    """The e8m0 plane S[M, K/32] of MXFP4 ACTIVATIONS in lane order, for the stream kernel whose
    waves multiply eight 16-row tiles of A each: rows padded to whole groups of 128 with the byte
    127 (scale 1), viewed as (group, tile t=8, row i=16, step, half h=2, lane group q=4) and
    stored (group, step, q, i, t, h): lane 16 q + i finds in its 16 bytes of the KiB (group,
    step) the scales of blocks q (h = 0) and 4 + q (h = 1) of its row in each of the eight
    tiles.  Returns a flat array of `mx_lanes128_bytes(M, K)` bytes."""
    S = np.ascontiguousarray(S, dtype=np.uint8)
    M, nb = S.shape
    if nb % 8 != 0:
        raise AssertionError(f"{nb} scale bytes per row are not whole 256-element steps")
    G = (M + 127) // 128
    pad = np.full((G * 128, nb), 127, np.uint8)
    pad[:M] = S
    view = pad.reshape(G, 8, 16, nb // 8, 2, 4)
    return np.ascontiguousarray(view.transpose(0, 3, 5, 2, 1, 4)).reshape(-1)


def unshuffle_scales_e8m0_lanes128(flat: np.ndarray, M: int, K: int) -> np.ndarray:
    """Inverse of `shuffle_scales_e8m0_lanes128`: the row-major plane [M, K/32]."""
    nb = K // 32
    G = (M + 127) // 128
    view = np.ascontiguousarray(flat, dtype=np.uint8).reshape(G, nb // 8, 4, 16, 8, 2)
    return np.ascontiguousarray(view.transpose(0, 4, 3, 1, 5, 2)).reshape(G * 128, nb)[:M]
