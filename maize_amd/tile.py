"""The reference's tile vocabulary on the host side of the gfx950 GEMM path.

The reference's caller (src/main.rs:31-90) *traces* a kernel: it declares the kernel and its
shared-memory ring, wraps the arguments as ``Matrix``, asks each matrix for its row / column
panels over a group of blocks, and calls ``sm80_gemm_smem_multibuffer`` on every (row panel,
column panel) pair.  Here the kernels are hand-written, so the same calls *describe* one: every
object below is a small host-side descriptor with the reference's name and meaning, the trace
is checked against what the kernels implement (where the reference panics at trace time, this
raises ``ValueError``), and ``finalize().compile(Gfx.Gfx950, ctx)`` resolves it to exactly the
launch ``maize_hip_gemm_bf16[_ex]`` makes for the same operands.

    RowPanel / ColPanel / *PanelIterLooper   crates/maize_tile/src/gmem/row_panel.rs:10-161, col_panel.rs:10-158
    Tile, TilePair, tile types               crates/maize_tile/src/lib.rs:87-108,231-265, pair.rs:3-8
    BlockX / BlockY / Wave (was Warp)        crates/maize_tile/src/group/by_block.rs:10-75, warp.rs:10-37, mod.rs:19-48
    SyncMMAOp and the MMA catalogue          crates/maize_tile/src/mma/mod.rs:19-99, sm80.rs, sm80_derived.rs:5-28, sm89.rs
    KTile, gemm_smem_multibuffer             crates/maize_tile/src/gemm/mod.rs:35-90
"""
from dataclasses import dataclass

from . import _ffi
from .api import Gfx, Matrix, gemm_ex_desc, gemm_plan

# ---- tile types and shared-memory tiles ---------------------------------------------------------


@dataclass(frozen=True)
class TileTy:
    """A tile type: ROWS x COLS elements of ELEM_BYTES bytes (ConstSizeTileTy, lib.rs:90-93) and how the kernels
    lay it out in LDS.  swizzle "kc16": rows of 128 bytes along K, 16-byte chunk index XOR-ed with (row >> 1) & 7;
    "kn32": a row-major K x N tile, 32-byte granule index XOR-ed with row % 4 + 4 * bit3(row); "kn16": a row-major
    K x N tile of 8-bit elements, 16-byte chunk index XOR-ed with row % 8 + 8 * bit4(row)."""
    name: str
    rows: int
    cols: int
    elem_bytes: int
    swizzle: str

    @property
    def size_bytes(self):
        return self.rows * self.cols * self.elem_bytes


BF16_16x16 = TileTy("BF16_16x16", 16, 16, 2, "none")          # the reference's tile (lib.rs:98-108): accepted nowhere here
BF16_256x64 = TileTy("BF16_256x64", 256, 64, 2, "kc16")       # A stage; B stage when B is stored N x K
BF16_64x256 = TileTy("BF16_64x256", 64, 256, 2, "kn32")       # B stage of a row-major K x N B
F16_256x64 = TileTy("F16_256x64", 256, 64, 2, "kc16")
F16_64x256 = TileTy("F16_64x256", 64, 256, 2, "kn32")
F8_256x128 = TileTy("F8_256x128", 256, 128, 1, "kc16")        # 8-bit operands: 128 elements of K per 128-byte row
F8_128x256 = TileTy("F8_128x256", 128, 256, 1, "kn16")        # B stage of a row-major K x N 8-bit B (read back by ds_read_b64_tr_b8)
# A stages of the 128 x 256 tile kernels (a wave then owns 64 x 128 of C; the B stages are the ones above)
BF16_128x64 = TileTy("BF16_128x64", 128, 64, 2, "kc16")
F16_128x64 = TileTy("F16_128x64", 128, 64, 2, "kc16")
F8_128x128 = TileTy("F8_128x128", 128, 128, 1, "kc16")
# B stage of the 128 x 128 tile kernels for a row-major K x N B (stored N x K, their B stage is BF16_128x64 like their A stage)
BF16_64x128 = TileTy("BF16_64x128", 64, 128, 2, "kn32")
F16_64x128 = TileTy("F16_64x128", 64, 128, 2, "kn32")
F8_128x128_KN = TileTy("F8_128x128_KN", 128, 128, 1, "kn16")      # ... for a row-major K x N 8-bit B (stored N x K: F8_128x128)


@dataclass(frozen=True)
class Tile:
    """``Tile<T>``: one tile of type T in shared memory (lib.rs:231-265)."""
    ty: TileTy

    @property
    def size_bytes(self):
        return self.ty.size_bytes


@dataclass(frozen=True)
class TilePair:
    """``TilePair<TA, TB>``: one ring stage = an A tile and a B tile (pair.rs:3-8)."""
    a: Tile
    b: Tile

    @property
    def size_bytes(self):
        return self.a.size_bytes + self.b.size_bytes


@dataclass(frozen=True)
class SharedRing:
    """``[TilePair; PIPE]`` in LDS, as returned by ``alloc_aligned_shared`` (src/main.rs:42-44)."""
    pair: TilePair
    depth: int
    align: int

    @property
    def size_bytes(self):
        return self.pair.size_bytes * self.depth


@dataclass(frozen=True)
class KTile:
    """``KTile<K_TILE>``: elements of K consumed per ring stage (gemm/mod.rs:35)."""
    value: int


# ---- groups -----------------------------------------------------------------------------------

def xcd_run(pid, total):
    """Workgroup id -> position in the tile list: ids congruent mod 8 (one XCD) get a contiguous run."""
    per, tall = (total + 7) // 8, (total % 8) or 8
    xcd, local = pid % 8, pid // 8
    return xcd * per + local if xcd < tall else tall * per + (xcd - tall) * (per - 1) + local


def tile_of(idx, tm, tn, group_rows=4):
    """Position in the tile list -> (tile row, tile column): sweeps of `group_rows` tile rows."""
    group = idx // (group_rows * tn)
    first = group * group_rows
    gsz = min(tm - first, group_rows)
    inner = idx % (group_rows * tn)
    return first + inner % gsz, inner // gsz


class _Block:
    """A group of workgroups that shares out panels (Group, group/mod.rs:19-29).  In the reference BlockX strides
    row panels by gridDim.x and BlockY column panels by gridDim.y (row_panel.rs:95-109); here both are realised by one
    persistent 1-D grid whose workgroup g computes tiles g, g + grid, ... of an XCD-aware list, and index_size()
    reports that walk: for workgroup `pid`, the panel index of each tile it computes and the number of panels."""
    axis = None

    def __init__(self, kernel):
        self.kernel = kernel

    def index_size(self, pid, tm, tn, grid):
        total = tm * tn
        walk = [tile_of(xcd_run(i, total), tm, tn)[self.axis] for i in range(pid, total, grid)]
        return walk, (tm, tn)[self.axis]


class BlockX(_Block):
    axis = 0


class BlockY(_Block):
    axis = 1


class Wave:
    """The 64-lane wavefront (the reference's 32-lane ``Warp``, group/warp.rs:10-37): the group that issues one
    cooperative copy.  const_size() == 64: one 128-bit request per lane moves 1 KiB."""

    def __init__(self, kernel):
        self.kernel = kernel

    @staticmethod
    def const_size():
        return 64


# ---- panels -----------------------------------------------------------------------------------

@dataclass(frozen=True)
class RowPanel:
    """N rows x all columns of a matrix (row_panel.rs:10-23).  `rows` is the window: the static N for bulk panels,
    the dynamic remainder for the epilogue panel."""
    matrix: Matrix
    rows: int
    group: object
    ragged: bool = False

    def row_size(self):
        return self.rows

    def col_size(self):
        return self.matrix.ncols


@dataclass(frozen=True)
class ColPanel:
    matrix: Matrix
    cols: int
    group: object
    ragged: bool = False

    def row_size(self):
        return self.matrix.nrows

    def col_size(self):
        return self.cols


class PanelIterLooper:
    """The bulk panels of one matrix (RowPanelIterLooper / ColPanelIterLooper).  for_every_value calls `body` once
    with the panel that stands for all of them, as the reference's looper calls its body once at trace time
    (row_panel.rs:25-78)."""

    def __init__(self, panel, count):
        self.panel, self.count = panel, count

    def for_every_value(self, body):
        body(self.panel)


def _panel_iter(matrix, n, group, kind):
    if n <= 0:
        raise ValueError("panel height must be positive")
    extent = matrix.nrows if kind is RowPanel else matrix.ncols
    bulk, rest = extent // n, extent % n
    return PanelIterLooper(kind(matrix, n, group), bulk), kind(matrix, rest, group, ragged=True)


def collective_aligned_row_panel_iter(matrix, n, group):
    """``Matrix::collective_aligned_row_panel_iter::<N>(group)`` (row_panel.rs:85-161): (bulk panels of N rows,
    the ragged epilogue panel).  The reference's caller throws the epilogue panel away (src/main.rs:56-57); here the
    kernels compute it with the bulk (edge tiles), so it only tells how many rows are ragged."""
    return _panel_iter(matrix, n, group, RowPanel)


def collective_aligned_col_panel_iter(matrix, n, group):
    """``Matrix::collective_aligned_col_panel_iter::<N>(group)`` (col_panel.rs:88-158)."""
    return _panel_iter(matrix, n, group, ColPanel)


# ---- the MMA catalogue -------------------------------------------------------------------------

@dataclass(frozen=True)
class SyncMMAOp:
    """One matrix instruction as an operation on wave fragments (SyncMMAOp, mma/mod.rs:37-75): D = A.B + C.
    frag_*: 32-bit registers per lane of each fragment; family: which kernels are built on it."""
    name: str
    m: int
    n: int
    k: int
    in_type: int
    frag_a: int
    frag_b: int
    frag_c: int
    mnemonic: str
    family: str
    k_tile: int                 # elements of K per ring stage of that family


Gfx950MfmaBf16F32_16x16x32 = SyncMMAOp("Gfx950MfmaBf16F32_16x16x32", 16, 16, 32, _ffi.IN_BF16, 4, 4, 4, "v_mfma_f32_16x16x32_bf16", "mt256", 64)
Gfx950MfmaBf16F32_32x32x16 = SyncMMAOp("Gfx950MfmaBf16F32_32x32x16", 32, 32, 16, _ffi.IN_BF16, 4, 4, 16, "v_mfma_f32_32x32x16_bf16", "wave32", 16)
Gfx950MfmaF16F32_16x16x32 = SyncMMAOp("Gfx950MfmaF16F32_16x16x32", 16, 16, 32, _ffi.IN_F16, 4, 4, 4, "v_mfma_f32_16x16x32_f16", "mt256", 64)
Gfx950MfmaE4M3F32_16x16x128 = SyncMMAOp("Gfx950MfmaE4M3F32_16x16x128", 16, 16, 128, _ffi.IN_E4M3, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", "mt256", 128)
Gfx950MfmaE5M2F32_16x16x128 = SyncMMAOp("Gfx950MfmaE5M2F32_16x16x128", 16, 16, 128, _ffi.IN_E5M2, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", "mt256", 128)
Gfx950MfmaE4M3E5M2F32_16x16x128 = SyncMMAOp("Gfx950MfmaE4M3E5M2F32_16x16x128", 16, 16, 128, _ffi.IN_E4M3_E5M2, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", "mt256", 128)
Gfx950MfmaE5M2E4M3F32_16x16x128 = SyncMMAOp("Gfx950MfmaE5M2E4M3F32_16x16x128", 16, 16, 128, _ffi.IN_E5M2_E4M3, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", "mt256", 128)
Gfx950MfmaF32F32_16x16x4 = SyncMMAOp("Gfx950MfmaF32F32_16x16x4", 16, 16, 4, _ffi.IN_F32, 1, 1, 4, "v_mfma_f32_16x16x4_f32", "mt128", 32)
Gfx950MfmaF64F64_16x16x4 = SyncMMAOp("Gfx950MfmaF64F64_16x16x4", 16, 16, 4, _ffi.IN_F64, 2, 2, 8, "v_mfma_f64_16x16x4_f64", "mt128", 16)
MMA_CATALOGUE = (Gfx950MfmaBf16F32_16x16x32, Gfx950MfmaBf16F32_32x32x16, Gfx950MfmaF16F32_16x16x32, Gfx950MfmaE4M3F32_16x16x128,
                 Gfx950MfmaE5M2F32_16x16x128, Gfx950MfmaE4M3E5M2F32_16x16x128, Gfx950MfmaE5M2E4M3F32_16x16x128,
                 Gfx950MfmaF32F32_16x16x4, Gfx950MfmaF64F64_16x16x4)


# ---- the traced kernel --------------------------------------------------------------------------

class Accum:
    """What gemm_smem_multibuffer returns: the accumulator fragments of one (row panel, column panel) pair.  The
    reference only sums them into a trap guard (src/main.rs:71); store() names the C they are written to."""

    def __init__(self, kernel, op):
        self.kernel, self.op = kernel, op

    def store(self, c, out_type=_ffi.OUT_SAME, alpha=1.0, beta=0.0):
        a, b = self.op["a"].matrix, self.op["b"].matrix
        n = b.nrows if self.op["nt"] else b.ncols
        if (c.nrows, c.ncols) != (a.nrows, n):
            raise ValueError(f"C is {c.nrows}x{c.ncols}, the panels describe {a.nrows}x{n}")
        self.op.update(c=c, out_type=out_type, alpha=alpha, beta=beta)
        self.kernel.ops.append(self.op)


def gemm_smem_multibuffer(mma, ktile, a_panel, b_panel, smem, cp_group, cp_size):
    """``sm80_gemm_smem_multibuffer(&mma, KTile::<K>, a_panel, b_panel, smem, cp_group, cp_size)``
    (gemm/mod.rs:37-90): the K loop of one row panel against one column panel through a ring of TilePairs filled by
    cooperative copies of `cp_size` bytes per lane of `cp_group`.  Checks the description against what the kernels of
    `mma.family` implement and returns the accumulator."""
    if not isinstance(mma, SyncMMAOp):
        raise ValueError("mma must be an entry of the MMA catalogue")
    if not isinstance(a_panel, RowPanel):
        raise ValueError("a must be a RowPanel")
    kernel = cp_group.kernel
    nt = isinstance(b_panel, RowPanel)          # B stored N x K: its panels are row panels too
    if not nt and not isinstance(b_panel, ColPanel):
        raise ValueError("b must be a ColPanel (B stored K x N) or a RowPanel (B stored N x K)")
    k_a = a_panel.col_size()
    k_b = b_panel.col_size() if nt else b_panel.row_size()
    if k_a != k_b:
        raise ValueError(f"inner dimensions differ (A has K={k_a}, B has K={k_b})")
    if not isinstance(cp_group, Wave):
        raise ValueError("the cooperative copies are issued per wavefront: cp_group must be a Wave")
    if mma.family == "mt256":
        if ktile.value != mma.k_tile:
            raise ValueError(f"{mma.name}: a ring stage holds {mma.k_tile} elements of K, not {ktile.value}")
        if cp_size != 16:
            raise ValueError("direct-to-LDS copies are 16 bytes per lane")
        # The mainloop is generic in the panel height and the ring depth, like the reference's ([TilePair; PIPE],
        # KTile<N>, gemm/mod.rs:37-45), within what kernels exist: 256- or 128-row panels of A on a two-stage ring,
        # 128-row panels also on three stages (the stage of a 128 x 256 tile is 48 KiB: three fit the 160 KiB of LDS).
        b_cols = b_panel.rows if nt else b_panel.cols
        # ... and 128 x 128 tiles (128-row panels of A against 128-column panels of B) on a ring of four 32 KiB stages,
        # 16-bit or 8-bit operands.
        quarter = a_panel.rows == 128 and b_cols == 128
        if a_panel.rows not in (256, 128) or b_cols not in (256, 128) or (b_cols == 128 and not quarter):
            raise ValueError("the macro-tile kernels take panels of 256 or 128 rows (A) and 256 columns (B), or 128 rows and 128 columns")
        if quarter:
            if smem is None or smem.depth != 4:
                raise ValueError("the 128 x 128 tile kernels run a ring of four stages")
        elif smem is None or smem.depth not in (2, 3):
            raise ValueError("the macro-tile kernels run a ring of two or three stages")
        if smem.depth == 3 and a_panel.rows != 128:
            raise ValueError("three ring stages fit the LDS with 128-row panels of A only")
        es = 1 if mma.k_tile == 128 else 2
        want_a = (a_panel.rows, mma.k_tile, es, "kc16")
        want_b = (b_cols, mma.k_tile, es, "kc16") if nt else (mma.k_tile, b_cols, es, "kn32" if es == 2 else "kn16")
        for which, tile, want in (("A", smem.pair.a, want_a), ("B", smem.pair.b, want_b)):
            t = tile.ty
            if (t.rows, t.cols, t.elem_bytes, t.swizzle) != want:
                raise ValueError(f"{which} stage is {t.name}; {mma.name} with B stored {'N x K' if nt else 'K x N'} needs "
                                 f"{want[0]}x{want[1]} tiles of {want[2]}-byte elements, layout {want[3]}")
    elif mma.family == "wave32":
        if smem is not None:
            raise ValueError(f"{mma.name} is the any-shape kernel's instruction: operands go straight from global memory, no ring")
    op = dict(mma=mma, a=a_panel, b=b_panel, nt=nt, panel_rows=a_panel.rows if mma.family == "mt256" else None,
              panel_cols=(b_panel.rows if nt else b_panel.cols) if mma.family == "mt256" else None,
              pipe=smem.depth if smem is not None else None)
    return Accum(kernel, op)


class TracedKernel:
    """``new_hip_kernel()`` without a name: the kernel being described (new_ptx_kernel, codegen/mod.rs:50)."""

    def __init__(self):
        self.block = None
        self.ring = None
        self.ops = []

    def with_launch_bounds_2d(self, xy, min_blocks_per_cu=None, cluster=None):
        if cluster is not None:
            raise ValueError("thread-block clusters do not exist on gfx950")
        if xy[0] * xy[1] not in (256, 512):
            raise ValueError("the GEMM kernels run 4 wavefronts (256 threads; the skinny kernels 8)")
        self.block = (xy[0], xy[1], 1)
        return self

    def alloc_aligned_shared(self, pair, depth, align):
        """``intrinsics().alloc_aligned_shared::<[TilePair<..>; PIPE]>(align)`` (src/main.rs:42-44)."""
        ring = SharedRing(pair, depth, align)
        if ring.size_bytes > 160 * 1024:
            raise ValueError(f"{ring.size_bytes} bytes of LDS requested, a compute unit has 163840")
        self.ring = ring
        return ring

    def cx(self):
        return self

    def finalize(self):
        if self.block is None:
            raise ValueError("launch bounds not set")
        if len(self.ops) != 1:
            raise ValueError(f"the trace must hold exactly one stored GEMM, it holds {len(self.ops)}")
        return PreLoadGemm(self)


_TYPE_TAG = {_ffi.IN_BF16: "bf16", _ffi.IN_F16: "f16", _ffi.IN_E4M3: "e4m3", _ffi.IN_E5M2: "e5m2",
             _ffi.IN_E4M3_E5M2: "e4m3e5m2", _ffi.IN_E5M2_E4M3: "e5m2e4m3"}


def described_kernel(desc, mma, nt, panel_rows, pipe, compute_units, panel_cols=256):
    """The kernel that a description of the mainloop (panel height of A, ring depth) names for `desc`, or None when
    the dispatcher's own choice already is of that family.  A description is honoured wherever a kernel of its family
    accepts the descriptor -- also where the dispatcher by itself would rather take another family (128-row tiles for
    a product of many rounds, say) -- and refused (ValueError) where none does."""
    from .api import MaizeError
    chosen = gemm_plan(desc, compute_units=compute_units)["kernel"]
    base = f"maize_gemm_{_TYPE_TAG[mma.in_type]}_mt256_{'nt' if nt else 'nn'}"
    if panel_cols == 128:                              # 128 x 128 tiles
        names = [f"maize_gemm_{_TYPE_TAG[mma.in_type]}_t128_{'nt' if nt else 'nn'}"]
        if chosen == names[0]:
            return None
    elif panel_rows == 256:
        if "_h128" not in chosen and "_t128_" not in chosen:
            return None                                # a 256-row kernel, a split of one, or a few-row kernel: the dispatcher's
        names = [base, base + "_ktail", base + "_gen", base + "_ktail_gen"]
    else:
        tag = "_h128r3" if pipe == 3 else "_h128"
        if tag in chosen and (pipe == 3 or "_h128r3" not in chosen):
            return None
        names = [base + tag, base + tag + "_gen"]
    for name in names:
        try:
            gemm_plan(desc, kernel=name, compute_units=compute_units)
            return name
        except MaizeError:
            continue
    raise ValueError(f"no kernel with {panel_rows}-row panels of A{' and 128-column panels of B' if panel_cols == 128 else ''} on {pipe} ring stages runs this product "
                     f"(tried {', '.join(names)})")


class PreLoadGemm:
    def __init__(self, traced):
        self.traced = traced

    def compile(self, target, ctx):
        if target is not Gfx.Gfx950:
            raise ValueError(f"unsupported target {target!r}: only Gfx.Gfx950 code is carried")
        op = self.traced.ops[0]
        a, b, c = op["a"].matrix, op["b"].matrix, op["c"]
        desc = gemm_ex_desc(a, b, c, layout=_ffi.LAYOUT_NT if op["nt"] else _ffi.LAYOUT_NN, out_type=op["out_type"], alpha=op["alpha"],
                            beta=op["beta"], in_type=op["mma"].in_type)
        forced = "maize_gemm_bf16_wave32" if op["mma"].family == "wave32" else None
        if op["mma"].family == "mt256":
            forced = described_kernel(desc, op["mma"], op["nt"], op["panel_rows"], op["pipe"], ctx.info()["compute_units"], op["panel_cols"])
        return LoadedGemm(ctx, desc, forced, op["mma"])


class LoadedGemm:
    """The described kernel, resolved: which kernel of the code object runs it, with what grid."""

    def __init__(self, ctx, desc, forced, mma):
        self.ctx, self.desc, self.forced, self.mma = ctx, desc, forced, mma
        self.plan = gemm_plan(desc, kernel=forced, compute_units=ctx.info()["compute_units"])

    @property
    def kernel_name(self):
        return self.plan["kernel"]

    def launch(self, stream=None):
        self.ctx.gemm_bf16(self.desc, stream=stream, kernel=self.forced)
