"""Strided layouts and XOR swizzles used by the GEMM problem description.

Mirrors the part of the reference's `aster.layout` that the GEMM config surface
and the LDS swizzle specification need: `Layout`, `Swizzle`, `tile`, and the
integer-tuple helpers (reference: python/aster/layout/algebra.py:52-171,
255-309; python/aster/layout/int_tuple.py:22-89).  The MLIR-emitting methods
(`Layout.lower`, `SwizzledLayout.lower`) have no role here: nothing is lowered
through a compiler, the swizzles are evaluated by the HIP kernels directly.
"""

from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple, Union

IntTuple = Union[int, Tuple[int, ...]]


def flatten_nested(t) -> tuple:
    """Flatten nested tuples/lists (or a scalar) into one flat tuple."""
    if not isinstance(t, (tuple, list)):
        return (t,)
    out: list = []
    stack = [iter(t)]
    while stack:
        try:
            x = next(stack[-1])
        except StopIteration:
            stack.pop()
            continue
        if isinstance(x, (tuple, list)):
            stack.append(iter(x))
        else:
            out.append(x)
    return tuple(out)


def product(a: IntTuple) -> int:
    return math.prod(a) if isinstance(a, tuple) else a


def suffix_product(a: IntTuple) -> IntTuple:
    """Compact row-major strides: (s0, s1, s2) -> (s1*s2, s2, 1); scalar -> 1."""
    if not isinstance(a, tuple):
        return 1
    strides = [1] * len(a)
    for i in range(len(a) - 2, -1, -1):
        strides[i] = strides[i + 1] * a[i + 1]
    return tuple(strides)


def delinearize(idx: int, sizes: Sequence[int]) -> tuple:
    """Row-major (first mode slowest) coordinates of a flat index."""
    coords = [0] * len(sizes)
    for i in range(len(sizes) - 1, -1, -1):
        idx, coords[i] = divmod(idx, sizes[i])
    return tuple(coords)


def linearize(coords: Sequence[int], strides: Sequence[int]) -> int:
    if len(coords) != len(strides):
        raise AssertionError("coords and strides differ in rank")
    return sum(c * s for c, s in zip(coords, strides))


class Layout:
    """Function from logical coordinates to an offset: phi(x) = sum_i x_i * stride_i.

    `Layout((4, 16), (16, 64))` has explicit strides; `Layout((4, 16))` is the
    compact row-major layout.  `axes` is an optional tuple of labels parallel to
    `flat_sizes` (set by `tile`).
    """

    __slots__ = ("sizes", "strides", "axes")

    def __init__(self, sizes: IntTuple, strides: Optional[IntTuple] = None, *,
                 axes: Optional[tuple] = None) -> None:
        self.sizes = sizes
        self.strides = suffix_product(sizes) if strides is None else strides
        self.axes = axes

    def __call__(self, idx: int) -> int:
        if isinstance(self.sizes, int):
            return idx * self.strides
        fs, fd = flatten_nested(self.sizes), flatten_nested(self.strides)
        return linearize(delinearize(idx, fs), fd)

    def size(self) -> int:
        return product(flatten_nested(self.sizes)) if isinstance(self.sizes, tuple) else self.sizes

    @property
    def flat_sizes(self) -> tuple:
        return flatten_nested(self.sizes)

    @property
    def is_flat(self) -> bool:
        return isinstance(self.sizes, int) or all(isinstance(s, int) for s in self.sizes)

    def __len__(self) -> int:
        return len(self.sizes) if isinstance(self.sizes, tuple) else 1

    def __eq__(self, other: object) -> bool:
        if not isinstance(other, Layout):
            return NotImplemented
        return (self.sizes, self.strides, self.axes) == (other.sizes, other.strides, other.axes)

    def __hash__(self) -> int:
        return hash((self.sizes, self.strides, self.axes))

    def __str__(self) -> str:
        return f"{self.sizes}:{self.strides}:{self.axes}"

    def __repr__(self) -> str:
        return f"Layout(sizes={self.sizes},strides={self.strides})"


class Swizzle:
    """XOR swizzle `off ^ ((off >> shift) & (((1 << bits) - 1) << base))`.

    The reference's gfx950 GEMMs use `Swizzle(3, 3, 4)` (8-byte slots of 64-byte
    rows) and `Swizzle(2, 4, 4)` (16-byte granules, direct-to-LDS path); the HIP
    tile kernel's 128-byte rows use `Swizzle(3, 4, 4)`: 16-byte granule index
    XOR ((row >> 1) & 7).
    """

    __slots__ = ("bits", "base", "shift")

    def __init__(self, bits: int, base: int, shift: int) -> None:
        self.bits, self.base, self.shift = bits, base, shift

    def __call__(self, offset: int) -> int:
        return offset ^ ((offset >> self.shift) & (((1 << self.bits) - 1) << self.base))

    def __eq__(self, other: object) -> bool:
        if not isinstance(other, Swizzle):
            return NotImplemented
        return (self.bits, self.base, self.shift) == (other.bits, other.base, other.shift)

    def __repr__(self) -> str:
        return f"Swizzle(bits={self.bits}, base={self.base}, shift={self.shift})"


# Swizzle of the HIP tile kernel's LDS stage (rows of 128 bytes).
TILE_LDS_SWIZZLE = Swizzle(3, 4, 4)


def make_layout(*layouts: Layout) -> Layout:
    """Each argument becomes one mode of the result."""
    return Layout(tuple(l.sizes for l in layouts), tuple(l.strides for l in layouts))


def tile(layout: Layout, tile_sizes: tuple, *, axes: Optional[tuple] = None) -> Layout:
    """Split every mode into (inter-tile, intra-tile) parts; result modes are all
    inter parts followed by all intra parts.  A tuple entry `(t0, t1, ...)` tiles
    one mode hierarchically (t0 innermost)."""
    sizes, strides = flatten_nested(layout.sizes), flatten_nested(layout.strides)
    if len(tile_sizes) != len(sizes):
        raise AssertionError(f"tile_sizes rank {len(tile_sizes)} != layout rank {len(sizes)}")
    inter: list = []
    intra: list = []
    for size, stride, ts in zip(sizes, strides, tile_sizes):
        levels = (ts,) if isinstance(ts, int) else tuple(ts)
        intra.append((levels[0], stride))
        span = levels[0]
        for t in levels[1:]:
            inter.append((t, span * stride))
            span *= t
        if size % span:
            raise AssertionError(f"tile {ts} does not divide layout dim {size}")
        inter.append((size // span, span * stride))
    modes = inter + intra
    out_axes = None
    if axes is not None:
        fa = flatten_nested(axes)
        out_axes = fa + (None,) * (len(modes) - len(fa))
    return Layout(tuple(m[0] for m in modes), tuple(m[1] for m in modes), axes=out_axes)
