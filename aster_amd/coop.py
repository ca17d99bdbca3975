"""Cooperative global->LDS load split.

`coop_2d_split` mirrors contrib/kittens/test/coop.py:12-27 of the reference: how
a workgroup's (tiles x k_tiles) staging work is divided over its waves with the
least clamping waste; `make_coop_load_plan` (coop.py:50-94) turns the split into
what one wave moves.  The HIP stream kernels use the degenerate split of that rule
(every wave moves whole 8-row, 1 KiB slabs, waves_k = 1), interleaved over the
waves: `stream_kernel_load_plan` is that staging written as a plan.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

from .layout import Layout


def coop_2d_split(num_tiles: int, num_waves: int, kt: int):
    """(waves_s, waves_k, coop_s, coop_k): split `num_waves` into a spatial x K
    grid; each wave then moves coop_s x coop_k tiles.  Among the divisor pairs of
    num_waves, least redundant tiles wins, then fewest idle waves, then the most
    spatial waves."""
    ranked = []
    for ws in (d for d in range(1, num_waves + 1) if num_waves % d == 0):
        wk = num_waves // ws
        cs, ck = math.ceil(num_tiles / ws), math.ceil(kt / wk)
        redundant = ws * wk * cs * ck - num_tiles * kt
        idle = max(0, ws - num_tiles) + max(0, wk - kt)
        ranked.append(((redundant, idle, -ws), (ws, wk, cs, ck)))
    return min(ranked, key=lambda r: r[0])[1]


def coop_wave_start(wave_index: int, coop: int, total: int) -> int:
    """First tile of a wave along one axis, clamped so surplus waves redo the last
    block instead of running past the end (coop.py:62-79)."""
    return min(wave_index * coop, max(0, total - coop))


# ---- per-wave load plan ----------------------------------------------------------------------


@dataclass(frozen=True)
class CoopLoadPlan:
    """What one wave moves of a workgroup's (tiles x k_tiles) global -> LDS staging work
    (reference: CoopLoadPlan, contrib/kittens/test/coop.py:30-48).

    `global_layout` / `lds_layout`: rank-2 layouts of sizes (coop_s, coop_k) over the wave's own
    transfers, offsets in bytes; `global_wave_off` / `lds_wave_off`: the wave's clamped start,
    added to every offset of the layouts; `unroll_axes`: (spatial_axis, k_axis).  The reference
    builds the two offsets as IR values of a kernel under construction; here nothing is
    compiled, so they are the integers for the wave id that was asked for."""

    global_layout: Layout
    global_wave_off: int
    lds_layout: Layout
    lds_wave_off: int
    unroll_axes: tuple

    def transfers(self):
        """[(global byte offset, LDS byte offset)] of this wave's transfers, spatial-major."""
        (cs, ck) = self.global_layout.sizes
        (gs, gk), (ls, lk) = self.global_layout.strides, self.lds_layout.strides
        return [(self.global_wave_off + s * gs + k * gk, self.lds_wave_off + s * ls + k * lk)
                for s in range(cs) for k in range(ck)]


def make_coop_load_plan(wid: int, *, num_waves: int, wg_tile_global: Layout, wg_tile_lds: Layout,
                        spatial_axis="s", k_axis="k", interleave: bool = False) -> CoopLoadPlan:
    """Plan of wave `wid` from the workgroup-level layouts of one operand: both have sizes
    (num_tiles, k_tiles) and give the byte offset of a transfer tile in global memory and in
    LDS (reference: make_coop_load_plan, contrib/kittens/test/coop.py:50-94; `b` and the IR
    values are gone, the arithmetic is the same).

    The waves form a (waves_s, waves_k) grid chosen by `coop_2d_split`; a wave's start along
    each axis is clamped in tile units so that surplus waves redo the last block.  With
    `interleave` a wave's spatial tiles are waves_s apart instead of adjacent (wave w takes
    tiles w, w + waves_s, ...), which is the order the HIP stream kernels issue their
    transfers in: neighbouring waves then touch neighbouring rows at the same time.  It needs a
    spatial split without remainder."""
    num_tiles, kt = wg_tile_global.sizes
    if tuple(wg_tile_lds.sizes) != (num_tiles, kt):
        raise AssertionError(f"wg_tile_lds sizes {wg_tile_lds.sizes} != wg_tile_global "
                             f"{wg_tile_global.sizes}")
    s_g, k_g = wg_tile_global.strides
    s_l, k_l = wg_tile_lds.strides
    waves_s, waves_k, coop_s, coop_k = coop_2d_split(num_tiles, num_waves, kt)
    if not 0 <= wid < num_waves:
        raise ValueError(f"wave id {wid} outside the {num_waves} waves of the workgroup")
    ws_idx, wk_idx = divmod(wid, waves_k)
    k_start = coop_wave_start(wk_idx, coop_k, kt)
    if interleave:
        if num_tiles != waves_s * coop_s:
            raise AssertionError("interleaved plans need num_tiles == waves_s * coop_s")
        s_start, step = ws_idx, waves_s
    else:
        s_start, step = coop_wave_start(ws_idx, coop_s, num_tiles), 1
    axes = (spatial_axis, k_axis)
    return CoopLoadPlan(
        global_layout=Layout((coop_s, coop_k), (step * s_g, k_g), axes=axes),
        global_wave_off=s_start * s_g + k_start * k_g,
        lds_layout=Layout((coop_s, coop_k), (step * s_l, k_l), axes=axes),
        lds_wave_off=s_start * s_l + k_start * k_l,
        unroll_axes=axes,
    )


# Transfer tile of the HIP stream kernels: 8 operand rows x 128 bytes = one 1 KiB wave
# instruction (global_load_lds_dwordx4, 64 lanes x 16 bytes).
STREAM_TILE_ROWS = 8
STREAM_ROW_BYTES = 128


def stream_kernel_load_plan(wid: int, *, tile_rows: int, num_waves: int,
                            ld_bytes: int) -> CoopLoadPlan:
    """The staging of one operand half of one K-step in the stream kernels
    (gemm_stream_kernel.hpp and its fp8 / MXFP4 siblings) as a CoopLoadPlan: `tile_rows` rows
    (256 or 128) of 128 bytes, cut into transfer tiles of 8 rows, one K tile, interleaved over
    the waves.  The kernels' `LH` (transfers per wave and slot) is this plan's coop_s, and
    transfer j of wave w covers operand rows (j * num_waves + w) * 8 .. + 7 and lands at LDS
    offset (j * num_waves + w) * 1 KiB of the slot."""
    tiles = tile_rows // STREAM_TILE_ROWS
    g = Layout((tiles, 1), (STREAM_TILE_ROWS * ld_bytes, STREAM_ROW_BYTES))
    l = Layout((tiles, 1), (STREAM_TILE_ROWS * STREAM_ROW_BYTES, STREAM_TILE_ROWS * STREAM_ROW_BYTES * tiles))
    return make_coop_load_plan(wid, num_waves=num_waves, wg_tile_global=g, wg_tile_lds=l,
                               interleave=True)


# (tile rows, waves) of every instantiation of the stream kernels' staging.
STREAM_PLAN_CONFIGS = [(256, 8), (256, 4), (128, 4)]


def stream_load_plan_header() -> str:
    """Text of `aster_amd/csrc/stream_load_plan.inc`: for every (tile rows, waves) the stream
    kernels are built with, the constants of `stream_kernel_load_plan` as a C++ struct the
    kernels take their transfer count, operand rows and LDS offsets from.  The plan of wave w is
    affine in (w, transfer j) - checked here - so four numbers describe it: transfers per wave,
    tiles between the first tiles of neighbouring waves, tiles between a wave's consecutive
    transfers, and the tile (rows, LDS bytes)."""
    out = ["// Generated by aster_amd.coop.stream_load_plan_header() (python -m aster_amd.build writes it);",
           "// do not edit.  The staging of one operand half of one K-step in the stream kernels as the",
           "// cooperative load plan of the reference (make_coop_load_plan,",
           "// contrib/kittens/test/coop.py:50-94): transfer j of wave w covers operand rows",
           "// first_row(w, j) .. + TILE_ROWS - 1 and lands at lds_offset(w, j) of the ring slot.",
           "#pragma once",
           "",
           "namespace astergemm {",
           "",
           "template <int TILE_ROWS_OF_SLOT, int NUM_WAVES>",
           "struct StreamLoadPlan;",
           ""]
    ld = 1 << 20      # any pitch: the plan is linear in it
    for rows, nw in STREAM_PLAN_CONFIGS:
        plans = [stream_kernel_load_plan(w, tile_rows=rows, num_waves=nw, ld_bytes=ld) for w in range(nw)]
        lh = plans[0].global_layout.sizes[0]
        t = [p_.transfers() for p_ in plans]
        row = lambda w, j: t[w][j][0] // ld
        assert all(t[w][j][0] % ld == 0 for w in range(nw) for j in range(lh))
        wave_step_rows = row(1, 0) - row(0, 0)
        xfer_step_rows = row(0, 1) - row(0, 0) if lh > 1 else nw * STREAM_TILE_ROWS
        tile_lds = STREAM_TILE_ROWS * STREAM_ROW_BYTES
        for w in range(nw):
            for j in range(lh):
                assert row(w, j) == w * wave_step_rows + j * xfer_step_rows
                assert t[w][j][1] * STREAM_TILE_ROWS == row(w, j) * tile_lds   # LDS follows the rows
        assert wave_step_rows % STREAM_TILE_ROWS == 0 and xfer_step_rows % STREAM_TILE_ROWS == 0
        out += [f"template <>",
                f"struct StreamLoadPlan<{rows}, {nw}> {{",
                f"  static constexpr int LH = {lh};                 // transfers per wave and slot",
                f"  static constexpr int TILE_ROWS = {STREAM_TILE_ROWS};          // operand rows of one transfer",
                f"  static constexpr int TILE_LDS_BYTES = {tile_lds};  // its bytes in the slot",
                f"  static constexpr int WAVE_STEP_TILES = {wave_step_rows // STREAM_TILE_ROWS};    // from wave w to w + 1",
                f"  static constexpr int XFER_STEP_TILES = {xfer_step_rows // STREAM_TILE_ROWS};    // from transfer j to j + 1",
                "  __host__ __device__ static constexpr int tile(int w, int j) {",
                "    return w * WAVE_STEP_TILES + j * XFER_STEP_TILES;",
                "  }",
                "  __host__ __device__ static constexpr int first_row(int w, int j) { return tile(w, j) * TILE_ROWS; }",
                "  __host__ __device__ static constexpr int lds_offset(int w, int j) { return tile(w, j) * TILE_LDS_BYTES; }",
                "};",
                ""]
    out += ["}  // namespace astergemm", ""]
    return "\n".join(out)
