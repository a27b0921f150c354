"""The host-side layout algebra (maize_amd/layout.py) against the reference's own unit-test vectors
(crates/maize_cob/src/layout/algorithm.rs:23-56 test_divide_1d / test_divide_2d, mod.rs:76-110 test_layout,
tuple.rs:389-402 test_constructor), the Python face of the reference (crates/maize_py: DType, Shape, Stride,
Tile and their reprs), and the ways this package's kernels cut a matrix, said with tiled_divide."""
import re

import pytest

import maize_amd as mz
from maize_amd import layout as L
from maize_amd.layout import DType, Layout, Shape, Stride, Tile, TupleWalkError, TypedTile, tiled_divide


def test_divide_1d_is_the_reference_vector():
    lay = Layout(Shape(30), Stride(2))
    div = tiled_divide(lay, Tile((3,), (5,))).canonicalize()
    assert div == Layout(Shape(3, Shape(2, 5)), Stride(10, Stride(30, 2)))
    assert div.to_string() == "(3, (2, 5)):(10, (30, 2))"
    # what it means: 3 workers side by side, each taking every 3rd tile of 5 elements (stride 2 per element)
    assert div.offset((1, (0, 0))) == 2 * 5 and div.offset((0, (1, 0))) == 2 * 15 and div.offset((2, (1, 4))) == 2 * 29
    assert sorted(div.offset((t, (q, e))) for t in range(3) for q in range(2) for e in range(5)) == list(range(0, 60, 2))


def test_divide_2d_is_the_reference_vector():
    div = tiled_divide(Layout(Shape(64, 32), Stride(32, 1)), Tile((2, 2), (4, 4)))
    want = Layout(Shape(Shape(2, 2), Shape(Shape(8, 4), Shape(4, 4))),
                  Stride(Stride(4 * 32, 4 * 1), Stride(Stride(8 * 32, 8 * 1), Stride(32, 1))))
    assert div == want
    # every element of the matrix exactly once
    offs = sorted(div.offset(((tr, tc), ((qr, qc), (er, ec)))) for tr in range(2) for tc in range(2) for qr in range(8)
                  for qc in range(4) for er in range(4) for ec in range(4))
    assert offs == list(range(64 * 32))


def test_divide_rejects_what_the_reference_rejects():
    with pytest.raises(TupleWalkError) as e:
        tiled_divide(Layout(Shape(30), Stride(2)), Tile((4,), (5,)))          # 30 is not a multiple of 20
    assert e.value.reason == (L.DIVISIBILITY,) and e.value.trace == [0]
    with pytest.raises(TupleWalkError) as e:
        tiled_divide(Layout(Shape(64, Shape(8, 4)), Stride(32, Stride(4, 1))), Tile((2, 2), (4, 4)))
    assert e.value.reason == (L.MISMATCHED_TOPOLOGY, 0, 1) and e.value.trace == [1]


def test_layout_topology_errors_are_the_reference_vectors():
    shape, stride = (3, 5, (5, 2)), (4, 5, (5, 2))
    Layout(Shape(*shape), Stride(*stride))
    stride = (4, (3, 5), (5, 2))
    with pytest.raises(TupleWalkError) as e:
        Layout(Shape(*shape), Stride(*stride))
    assert e.value == TupleWalkError((L.MISMATCHED_TOPOLOGY, 0, 1), [1])
    shape = (3, (3, 5), (5, 2, (5,)))
    with pytest.raises(TupleWalkError) as e:
        Layout(Shape(*shape), Stride(*stride))
    assert e.value == TupleWalkError((L.MISMATCHED_LENGTH, 0, 1), [2])
    stride = (4, (3, 5), (5, 2, 5))
    with pytest.raises(TupleWalkError) as e:
        Layout(Shape(*shape), Stride(*stride))
    assert e.value == TupleWalkError((L.MISMATCHED_TOPOLOGY, 0, 1), [2, 2])


def test_constructor_nesting_and_canonical_form():
    t = Shape(Shape(3, 4), Shape(5, 6), 3)
    assert t.get() == ((3, 4), (5, 6), 3) and len(t) == 3 and repr(t) == "((3, 4), (5, 6), 3)"
    # canonical form: 1-tuples are unwrapped where they are entries of a tuple; the unwrapped entry is left alone
    assert L.canonicalize(((3,), ((2,), (5,)))) == (3, (2, 5))
    assert L.canonicalize((((7,),), (1, 2))) == ((7,), (1, 2))
    assert Layout.combine(Layout(Shape(2), Stride(1)), Layout(Shape(3, 4), Stride(4, 1))) == \
        Layout(Shape(Shape(2), Shape(3, 4)), Stride(Stride(1), Stride(4, 1)))
    with pytest.raises(TypeError):
        Shape(3, -1)
    with pytest.raises(TypeError):
        Shape(3, 1.5)


def test_python_face_of_the_reference():
    assert DType.from_str("F32").to_str() == "F32" and DType.try_from_str("F64") == DType.F64
    assert DType.try_from_str("BF16") is None
    with pytest.raises(ValueError, match=re.escape("Invalid DType name 'F16'")):
        DType.from_str("F16")
    assert repr(Shape(3, Shape(4, 5))) == "(3, (4, 5))" and repr(Stride()) == "()"
    assert repr(TypedTile(Shape(16, 16), DType.F32)) == "Tile(shape=(16, 16), dtype=F32)"
    assert TypedTile(Shape(16, 16), DType.F32) == TypedTile(Shape(16, 16), DType.from_str("F32"))
    with pytest.raises(TypeError):
        TypedTile((16, 16), DType.F32)


def test_the_reference_row_panel_walk():
    """Block bx handles rows bx * 16 + i * gridDim.x * 16 (crates/maize_tile/src/gmem/row_panel.rs:95-109)."""
    grid, nrows = 4, 4096
    walk = L.reference_row_panels(nrows, grid)
    for bx in range(grid):
        for i in (0, 1, 63):
            for r in (0, 15):
                assert walk.offset((bx, (i, r))) == bx * 16 + i * grid * 16 + r


def test_persistent_walk_matches_the_dispatcher():
    """Workgroup g of the persistent kernels computes tiles g, g + grid, ...: the dispatcher's grid for 8192^3 is one
    workgroup per compute unit, the list has 1024 tiles."""
    x = mz.gemm_desc(mz.GlobalMatrix(0x1000, 8192, 8192), mz.GlobalMatrix(0x10000000, 8192, 8192), mz.GlobalMatrix(0x20000000, 8192, 8192),
                     layout=mz.LAYOUT_NT)
    plan = mz.gemm_plan(x, compute_units=256)
    grid = plan["grid"][0]
    walk = L.persistent_walk(1024, grid)
    assert grid == 256 and walk.shape().get() == (256, (4, 1)) and walk.stride().get() == (1, (256, 1))
    assert [walk.offset((7, (r, 0))) for r in range(4)] == [7, 263, 519, 775]
    with pytest.raises(TupleWalkError):
        L.persistent_walk(1000, 256)                      # the algebra wants whole rounds; the kernels just stop at the end


def test_macro_tile_decomposition_is_the_epilogue_lane_map():
    """The macro-tile kernel's epilogue states: lane l of wave (wm, wn) holds, in accumulator (i, j), C[row = wm 128 +
    16 i + l % 16][col = wn 128 + 16 j + 4 (l / 16) + v].  The same map from tiled_divide, mode by mode."""
    ldc = 4104
    off = L.macro_tile_of_c(ldc)
    seen = set()
    for wm in range(2):
        for wn in range(2):
            for i in range(8):
                for j in range(8):
                    for lane in range(64):
                        for v in range(4):
                            o = off(wm, i, lane % 16, wn, j, lane // 16, v)
                            assert o == (wm * 128 + 16 * i + lane % 16) * ldc + wn * 128 + 16 * j + 4 * (lane // 16) + v
                            seen.add(o)
    assert len(seen) == 256 * 256                         # every element of the tile, once


@pytest.mark.parametrize("rows,cols", [(128, 256), (128, 128)])
def test_the_smaller_tiles_decompose_the_same_way(rows, cols):
    """The half-height and the 128 x 128 tile kernels keep the wave grid (2 x 2) and the lane map; only the number of
    accumulators per wave changes: lane l of wave (wm, wn) holds, in accumulator (i, j),
    C[row = wm rows/2 + 16 i + l % 16][col = wn cols/2 + 16 j + 4 (l / 16) + v]."""
    ldc = 2056
    off = L.macro_tile_of_c(ldc, rows, cols)
    seen = set()
    for wm in range(2):
        for wn in range(2):
            for i in range(rows // 32):
                for j in range(cols // 32):
                    for lane in range(64):
                        for v in range(4):
                            o = off(wm, i, lane % 16, wn, j, lane // 16, v)
                            assert o == (wm * (rows // 2) + 16 * i + lane % 16) * ldc + wn * (cols // 2) + 16 * j + 4 * (lane // 16) + v
                            seen.add(o)
    assert len(seen) == rows * cols
    with pytest.raises(ValueError):
        L.macro_tile_of_c(ldc, 64, 64)
