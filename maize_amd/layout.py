"""Host-side layout algebra: nested shapes and strides, and tiled_divide.

Mirrors the reference's CuTe-like crate (crates/maize_cob/src/layout: tuple.rs, shape.rs, stride.rs, mod.rs,
tile.rs, algorithm.rs) with the same names, results and error values, on plain nested Python tuples of ints
instead of its TupleOrValue enum.  The reference does not use it in its kernel; here it describes -- and the
tests check -- how the kernels of this package cut a matrix: the persistent walk of the tile list, the
workgroup / wave / matrix-instruction tiles of C, the reference's own row-panel walk.

    Layout(Shape(64, 32), Stride(32, 1))                  a 64 x 32 row-major matrix
    tiled_divide(layout, Tile((2, 2), (4, 4)))            per mode: 2 tiles of 4 elements side by side, repeated

tiled_divide (algorithm.rs:4-21): for every mode with extent a, stride d, `num_tiles` c and `tile_size` s the
result has shape (c, (a / (c s), s)) and stride (d s, (d s c, d)): coordinate (t, (q, e)) is element
(q c + t) s + e of the mode -- c workers side by side, each taking every c-th tile of s elements.
"""
from __future__ import annotations

MISMATCHED_LENGTH = "MismatchedLength"
MISMATCHED_TOPOLOGY = "MismatchedTopology"
DIVISIBILITY = "Divisibility"


class TupleWalkError(Exception):
    """reason: (MISMATCHED_LENGTH | MISMATCHED_TOPOLOGY, 0, 1) or (DIVISIBILITY,); trace: the indices that lead
    to the offending entry, innermost first as the walk unwinds (tuple.rs:96-108; Layout.try_new reverses it)."""

    def __init__(self, reason, trace):
        super().__init__(f"{reason} at {trace}")
        self.reason, self.trace = tuple(reason), list(trace)

    def __eq__(self, other):
        return isinstance(other, TupleWalkError) and self.reason == other.reason and self.trace == other.trace

    __hash__ = None


def _norm(x):
    """Nested tuples / lists / Shape / Stride of non-negative ints -> nested tuples."""
    if isinstance(x, (Shape, Stride)):
        return x.get()
    if isinstance(x, (tuple, list)):
        return tuple(_norm(v) for v in x)
    if isinstance(x, bool) or not isinstance(x, int) or x < 0:
        raise TypeError(f"layout entries are non-negative integers or tuples of them, not {x!r}")
    return x


def apply(t, f):
    """f on every leaf, same nesting (tuple.rs:171-181)."""
    return tuple(apply(v, f) if isinstance(v, tuple) else f(v) for v in t)


def apply2(a, b, f):
    """f on every pair of leaves of two tuples of the same topology (tuple.rs:217-255).  As in the reference the
    top-level walk is a zip (a longer operand is cut short); nested tuples must agree in kind and length."""
    out = []
    for i, (x, y) in enumerate(zip(a, b)):
        if isinstance(x, tuple) != isinstance(y, tuple):
            raise TupleWalkError((MISMATCHED_TOPOLOGY, 0, 1), [i])
        if isinstance(x, tuple):
            if len(x) != len(y):
                raise TupleWalkError((MISMATCHED_LENGTH, 0, 1), [i])
            try:
                out.append(apply2(x, y, f))
            except TupleWalkError as e:
                e.trace.append(i)
                raise
        else:
            try:
                out.append(f(x, y))
            except TupleWalkError as e:        # f reports a leaf-level reason with an empty trace
                raise TupleWalkError(e.reason, [i]) from None
    return tuple(out)


def same_topology(a, b):
    apply2(a, b, lambda *_: None)


def canonicalize(t):
    """Every entry that is a 1-tuple is replaced by its only element; other tuple entries are canonicalized in turn
    (tuple.rs:8-25, 324-328).  The unwrapped element itself is left as it is, as in the reference."""
    return tuple((v[0] if len(v) == 1 else canonicalize(v)) if isinstance(v, tuple) else v for v in t)


def to_string(t):
    return "(" + ", ".join(to_string(v) if isinstance(v, tuple) else str(v) for v in t) + ")"


def leaves(t):
    for v in t:
        if isinstance(v, tuple):
            yield from leaves(v)
        else:
            yield v


class _Nested:
    def __init__(self, *values):
        self._t = _norm(values)

    @classmethod
    def from_tuple(cls, t):
        self = cls()
        self._t = _norm(t)
        return self

    def get(self):
        return self._t

    def __len__(self):
        return len(self._t)

    def same_topology(self, other):
        same_topology(self._t, other.get())

    def canonicalize(self):
        return type(self).from_tuple(canonicalize(self._t))

    def __eq__(self, other):
        return type(self) is type(other) and self._t == other._t

    __hash__ = None

    def __repr__(self):
        return to_string(self._t)


class Shape(_Nested):
    """Shape(3, 5, Shape(5, 2)) (shape.rs; the Python face of the reference takes the same arguments,
    crates/maize_py/src/shape.rs:27-33)."""


class Stride(_Nested):
    """Stride(4, 5, Stride(5, 2)) (stride.rs, crates/maize_py/src/stride.rs)."""


class Layout:
    """A shape and a stride of the same topology (mod.rs:9-66)."""

    def __init__(self, shape, stride):
        shape = shape if isinstance(shape, Shape) else Shape.from_tuple(shape)
        stride = stride if isinstance(stride, Stride) else Stride.from_tuple(stride)
        try:
            same_topology(shape.get(), stride.get())
        except TupleWalkError as e:
            raise TupleWalkError(e.reason, list(reversed(e.trace))) from None      # outermost index first (mod.rs:22-29)
        self._shape, self._stride = shape, stride

    @classmethod
    def combine(cls, left, right):
        return cls(Shape(left.shape().get(), right.shape().get()), Stride(left.stride().get(), right.stride().get()))

    def shape(self):
        return self._shape

    def stride(self):
        return self._stride

    def decompose(self):
        return self._shape, self._stride

    def __len__(self):
        return len(self._shape)

    def canonicalize(self):
        return Layout(self._shape.canonicalize(), self._stride.canonicalize())

    def __eq__(self, other):
        return isinstance(other, Layout) and self._shape == other._shape and self._stride == other._stride

    __hash__ = None

    def __repr__(self):
        return f"{self._shape!r}:{self._stride!r}"

    to_string = __repr__

    # -- what a layout is for: coordinates -> offsets (not in the reference, which stops at the algebra) --
    def size(self):
        n = 1
        for v in leaves(self._shape.get()):
            n *= v
        return n

    def offset(self, coord):
        """Inner product of a coordinate of the shape's topology with the strides; every entry is range-checked."""
        def walk(c, extent, stride):
            if len(c) != len(extent):
                raise TupleWalkError((MISMATCHED_LENGTH, 0, 1), [])
            total = 0
            for x, e, d in zip(c, extent, stride):
                if isinstance(x, tuple) != isinstance(e, tuple):
                    raise TupleWalkError((MISMATCHED_TOPOLOGY, 0, 1), [])
                if isinstance(x, tuple):
                    total += walk(x, e, d)
                else:
                    if x >= e:
                        raise IndexError(f"coordinate {x} out of range for extent {e}")
                    total += x * d
            return total

        return walk(_norm(coord), self._shape.get(), self._stride.get())


class Tile:
    """Per mode: `num_tiles` tiles of `tile_size` elements side by side (tile.rs)."""

    def __init__(self, num_tiles, tile_size):
        n, s = _norm(num_tiles if isinstance(num_tiles, (tuple, list)) else (num_tiles,)), \
               _norm(tile_size if isinstance(tile_size, (tuple, list)) else (tile_size,))
        self._t = apply2(n, s, lambda a, b: (a, b))
        self.num_tiles, self.tile_size = n, s

    def get(self):
        return self._t


def tiled_divide(num, div):
    """[a] ; (b) / [c] ; (d) == [c, [a / cd, d]] ; (db, (dbc, b))  (algorithm.rs:3-21)."""
    shape, stride = num.shape().get(), num.stride().get()
    same_topology(shape, div.num_tiles)
    tile_size, num_tiles = div.tile_size, div.num_tiles
    mul = lambda a, b: a * b
    tile_stride = apply2(stride, tile_size, mul)
    local_tile_stride = apply2(tile_stride, num_tiles, mul)
    full_tile_size = apply2(tile_size, num_tiles, mul)

    def div_exact(a, cd):
        if cd == 0 or a % cd:
            raise TupleWalkError((DIVISIBILITY,), [])
        return a // cd

    num_local_tiles = apply2(shape, full_tile_size, div_exact)
    return Layout(Shape(num_tiles, Shape(num_local_tiles, tile_size)), Stride(tile_stride, Stride(local_tile_stride, stride)))


# ---- the Python face of the reference (crates/maize_py: DType, Shape, Stride, Tile) -------------------------

class DType:
    """F32 / F64 (crates/maize_py/src/dtype.rs; crates/maize_cob/src/dtype/mod.rs)."""
    _names = ("F32", "F64")

    def __init__(self, name):
        if name not in self._names:
            raise ValueError(f"Invalid DType name '{name}'")
        self._name = name

    def to_str(self):
        return self._name

    @classmethod
    def try_from_str(cls, val):
        return cls(val) if val in cls._names else None

    @classmethod
    def from_str(cls, val):
        return cls(val)

    def __eq__(self, other):
        return isinstance(other, DType) and self._name == other._name

    __hash__ = None

    def __repr__(self):
        return f"DType.{self._name}"


DType.F32, DType.F64 = DType("F32"), DType("F64")


class TypedTile:
    """The bindings' Tile(shape, dtype) (crates/maize_py/src/tile.rs; a different thing from the algebra's Tile above,
    hence the other name here)."""

    def __init__(self, shape, dtype):
        if not isinstance(shape, Shape) or not isinstance(dtype, DType):
            raise TypeError("Tile(shape: Shape, dtype: DType)")
        self.shape, self.dtype = shape, dtype

    def __eq__(self, other):
        return isinstance(other, TypedTile) and self.shape == other.shape and self.dtype == other.dtype

    __hash__ = None

    def __repr__(self):
        return f"Tile(shape={self.shape!r}, dtype={self.dtype.to_str()})"


# ---- how this package's kernels cut a matrix, said with the algebra ---------------------------------------------

def row_major(rows, cols, ld=None):
    return Layout(Shape(rows, cols), Stride(cols if ld is None else ld, 1))


def persistent_walk(items, grid):
    """The work list of the persistent kernels: workgroup g takes items g, g + grid, g + 2 grid, ...:
    coordinate (g, (round, 0)).  `items` must be a multiple of `grid` for the algebra (the kernels simply stop
    at the end of the list)."""
    return tiled_divide(Layout(Shape(items), Stride(1)), Tile((grid,), (1,))).canonicalize()


def reference_row_panels(nrows, grid, panel=16):
    """The reference's row-panel walk: block bx handles rows bx * 16 + i * gridDim.x * 16
    (crates/maize_tile/src/gmem/row_panel.rs:95-109): coordinate (bx, (i, row in panel))."""
    return tiled_divide(Layout(Shape(nrows), Stride(1)), Tile((grid,), (panel,))).canonicalize()


def macro_tile_of_c(ldc, rows=256, cols=256):
    """One workgroup tile of C as the tile kernels' epilogues see it: 256 x 256 (the macro-tile kernels), 128 x 256
    (their half-height variants) or 128 x 128 (the four-stage kernels).  Rows: 2 waves (wm) x rows / 32 accumulator
    rows (i) x 16 lanes (l % 16); columns: 2 waves (wn) x cols / 32 accumulator columns (j) x 4 lane groups (l / 16)
    x 4 consecutive elements (v).  Returns f(wm, i, l16, wn, j, lg, v) -> element offset inside the tile, each mode
    divided step by step with tiled_divide."""
    if (rows, cols) not in ((256, 256), (128, 256), (128, 128)):
        raise ValueError("tiles are 256 x 256, 128 x 256 or 128 x 128")

    def cut(extent, stride, parts):
        # `parts` tiles of extent / parts elements, side by side, each once: coordinate (part, (0, rest))
        return tiled_divide(Layout(Shape(extent), Stride(stride)), Tile((parts,), (extent // parts,))).canonicalize()

    rows_by_wave, rows_by_acc = cut(rows, ldc, 2), cut(rows // 2, ldc, rows // 32)
    cols_by_wave, cols_by_acc, cols_by_group = cut(cols, 1, 2), cut(cols // 2, 1, cols // 32), cut(16, 1, 4)

    def offset(wm, i, l16, wn, j, lg, v):
        return (rows_by_wave.offset((wm, (0, 0))) + rows_by_acc.offset((i, (0, l16))) +
                cols_by_wave.offset((wn, (0, 0))) + cols_by_acc.offset((j, (0, 0))) + cols_by_group.offset((lg, (0, v))))

    return offset
