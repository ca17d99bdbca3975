"""Data-layout maps of the GEMM path as explicit index formulas.  Test infrastructure."""

from __future__ import annotations

import numpy as np


def shuffle_weight_index(N: int, K: int) -> np.ndarray:
    """Flat source index for every flat destination index of the B pre-shuffle.

    Restates `shuffle_weight` (contrib/kittens/test/kittens_helpers.py:90-119):
    destination order (n_block, k_block, lane_group, n_lane, k_half, k_within),
    source element B[n_block*16 + n_lane, k_block*32 + k_half*16 + lane_group*4 + k_within].
    """
    assert N % 16 == 0 and K % 32 == 0
    src = np.empty(N * K, dtype=np.int64)
    o = 0
    for nb in range(N // 16):
        for kb in range(K // 32):
            for g in range(4):
                for nl in range(16):
                    for kh in range(2):
                        for kw in range(4):
                            src[o] = (nb * 16 + nl) * K + kb * 32 + kh * 16 + g * 4 + kw
                            o += 1
    return src


def shuffle_weight(B: np.ndarray) -> np.ndarray:
    N, K = B.shape
    return B.reshape(-1)[shuffle_weight_index(N, K)].reshape(N, K)


def swizzle(offset: int, bits: int, base: int, shift: int) -> int:
    """`Swizzle.__call__` (python/aster/layout/algebra.py:166-168)."""
    mask = ((1 << bits) - 1) << base
    return offset ^ ((offset >> shift) & mask)


def lds_swizzled_addr_16x64_b(base: int, row: int, byte_in_row: int) -> int:
    """mlir_kernels/library/common/indexing.mlir:584-592."""
    return base + row * 64 + (byte_in_row ^ (((row // 2) % 8) * 8))


def mfma_index_a_16x16_f16(lane: int):
    """(row, col) of a lane's first A element, 16x16x16 f16 (indexing.mlir:182-188)."""
    return lane % 16, (lane // 16) * 4


def mfma_index_a_16x16_fp8(lane: int):
    """indexing.mlir:202-208."""
    return lane % 16, (lane // 16) * 8


def mfma_index_c_16x16_f32(lane: int):
    """(col, row_base): lane holds C[row_base + 0..3, col] (indexing.mlir:221-227, 355-363)."""
    return lane % 16, (lane // 16) * 4


# --- layout of the build's own LDS tile (128-byte rows, 16-byte granules) --------


def tile_granule_slot(row: int, granule: int) -> int:
    """Slot (0..7) of a 128-byte LDS row that holds K-granule `granule` of that row."""
    return granule ^ ((row >> 1) & 7)


def tile_lds_offset(row: int, granule: int) -> int:
    return row * 128 + tile_granule_slot(row, granule) * 16


def bank_groups_16B(offsets) -> list:
    """16-byte bank-group index (0..15) of each byte offset, for 64 banks x 4 B."""
    return [(o // 16) % 16 for o in offsets]
