"""Cooperative global->LDS load split.

`coop_2d_split` mirrors contrib/kittens/test/coop.py:12-27 of the reference: how
a workgroup's (tiles x k_tiles) staging work is divided over its waves with the
least clamping waste.  The HIP tile kernel uses the degenerate split of that
rule: every wave moves whole 8-row (1 KiB) slabs, waves_k = 1.
"""

from __future__ import annotations

import math


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
