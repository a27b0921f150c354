"""CPU-only checks of the dispatcher: for a sweep of descriptors, the kernel it picks accepts
the descriptor, the grid covers every output tile exactly once, split-K geometry leaves no
empty or over-long K range, and the workspace the library allocates is at least what the
kernels address.  These are the memory-safety preconditions of the hand-written kernels; no
device is touched (maize_hip_gemm_plan needs none)."""
import itertools

import pytest

import maize_amd as mz
from maize_amd import _ffi

TICKET_BYTES = 16384 * 4
CUS = 256


def desc(m, n, k, layout=mz.LAYOUT_NN, batch=1, base=0x10000):
    a = mz.GlobalMatrix(base, m, k)
    b = mz.GlobalMatrix(base + (1 << 32), k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(base + (1 << 32), n, k)
    c = mz.GlobalMatrix(base + (2 << 32), m, n)
    return mz.gemm_desc(a, b, c, layout=layout, batch=batch, stride_a=m * k, stride_b=k * n, stride_c=m * n)


def cdiv(a, b):
    return (a + b - 1) // b


SHAPES = [
    (4096, 4096, 4096), (4000, 4104, 4032), (8192, 8192, 8192), (16, 14336, 4096), (2048, 2048, 2048),
    (1, 1, 1), (33, 17, 65), (128, 128, 64), (256, 256, 64), (257, 264, 72), (4096, 4104, 256), (4128, 4096, 4096),
    (4104, 4096, 512), (16, 64, 256), (16, 56, 256), (8, 512, 8192), (16, 14336, 4128), (16, 28672, 16384),
    (300, 4000, 40), (4096, 8, 4096), (8, 8, 8), (1024, 1032, 1024), (8200, 4096, 2048), (4096, 8200, 2048),
]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("batch", [1, 3])
def test_selected_kernel_supports_the_descriptor_and_its_grid_covers_c(m, n, k, layout, batch):
    d = desc(m, n, k, layout, batch)
    p = mz.gemm_plan(d, compute_units=CUS)
    assert p["kernel"] in mz.kernel_names()
    assert mz.kernel_supports(p["kernel"], d)
    check_plan(p, m, n, k, layout, batch)


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_every_kernel_that_accepts_a_descriptor_plans_a_covering_grid(m, n, k, layout):
    d = desc(m, n, k, layout)
    for name in mz.kernel_names():
        if not mz.kernel_supports(name, d):
            with pytest.raises(mz.MaizeError):
                mz.gemm_plan(d, kernel=name, compute_units=CUS)
            continue
        for cus in (1, 8, 80, 256, 304):
            check_plan(mz.gemm_plan(d, kernel=name, compute_units=cus), m, n, k, layout, 1, cus)


def check_plan(p, m, n, k, layout, batch, cus=CUS):
    gx, gy, gz = p["grid"]
    splitk = p["kernel"].endswith("_splitk")
    packed = p["kernel"].endswith("_packed")
    persistent = ("_mt256_" in p["kernel"] and not p["kernel"].endswith("_edge")) or "_t128_" in p["kernel"]   # (batch members in grid.x)
    assert gx >= 1 and gy >= 1 and gz == (1 if persistent else batch)
    assert gy <= 65535 and gz <= 65535 and gx < (1 << 31)
    name = p["kernel"]
    if name == "maize_gemm_bf16_wave32":
        assert p["block"] == (256, 1, 1)
        assert gx == cdiv(n, 64) and gy == cdiv(m, 64)
        assert p["workspace_bytes"] == 0 and p["ksplit"] == 0
    elif name.endswith("_packed_gen"):
        # the general-epilogue kernel on zero-padded copies, C stored by the first pass: persistent over the tiles, the
        # workspace holds the copies only, no reduce pass.  C takes 128-bit stores.
        n8, k8 = (n + 7) // 8 * 8, (k + 63) // 64 * 64           # K padded to whole K tiles
        assert n8 == n and p["reduce_grid"] == 0 and p["ksplit"] == 0 and p["split_first"] == 0
        resident = cus - cus % 8 if cus >= 8 else cus
        assert p["block"] == (256, 1, 1) and gy == 1 and gx == min(cdiv(m, 256) * cdiv(n, 256) * batch, resident)
        assert TICKET_BYTES <= p["workspace_bytes"] <= TICKET_BYTES + 2 * batch * (m * k8 + n8 * k8)
    elif packed:
        # the split-K kernels on zero-padded copies: work items over the padded extents, then the reduce pass
        # over the real C; the workspace also holds the copies
        n8, k8 = (n + 7) // 8 * 8, (k + 7) // 8 * 8
        ks = p["ksplit"]
        items = cdiv(m, 256) * cdiv(n8, 256) * batch * ks
        resident = cus - cus % 8 if cus >= 8 else cus
        assert p["block"] == (256, 1, 1) and gy == 1 and 1 <= ks <= 64 and gx == min(items, resident)
        assert cdiv(cdiv(k8, 64), ks) * (ks - 1) < cdiv(k8, 64)
        assert TICKET_BYTES + items * 256 * 256 * 4 <= p["workspace_bytes"] <= TICKET_BYTES + items * 256 * 256 * 4 + 2 * batch * (m * k8 + n8 * k8)
        assert p["reduce_grid"] == cdiv(m * cdiv(n, 8) * batch, 256)
    elif splitk:
        # (tile, K range) work items, one fp32 partial tile each, then the reduce pass over runs of 8 columns
        # (tiles of 256 x 256, or of 128 x 256 -- flagged to the reduce pass by bit 0 of the launch flag)
        assert p["block"] == (256, 1, 1) and gy == 1 and k % 8 == 0 and n % 8 == 0
        ks = p["ksplit"]
        tile_rows = 128 if "_h128" in name else 256
        assert p["split_first"] == (1 if tile_rows == 128 else 0)
        items = cdiv(m, tile_rows) * cdiv(n, 256) * batch * ks
        resident = cus - cus % 8 if cus >= 8 else cus
        assert 1 <= ks <= 64 and gx == min(items, resident)
        nk = cdiv(k, 64)
        assert cdiv(nk, ks) * (ks - 1) < nk                    # no empty range
        assert p["workspace_bytes"] == TICKET_BYTES + items * tile_rows * 256 * 4 and p["workspace_bytes"] <= (1 << 32) + TICKET_BYTES
        assert p["reduce_grid"] == cdiv(m * cdiv(n, 8) * batch, 256)
    elif "_h128" in name:
        # 128 x 256 tiles, persistent over all of them; the plain form wants whole K tiles, the general form any K % 8 == 0
        assert p["reduce_grid"] == 0 and p["workspace_bytes"] == 0 and p["split_first"] == 0 and p["ksplit"] == 1
        assert p["block"] == (256, 1, 1) and gy == 1
        assert ("_nt" in name) == (layout == mz.LAYOUT_NT)
        assert k % 8 == 0 and n % 8 == 0 and (name.endswith("_gen") or k % 64 == 0)
        resident = cus - cus % 8 if cus >= 8 else cus
        assert gx == min(cdiv(m, 128) * cdiv(n, 256) * batch, resident)
    elif name.endswith("_ragged_m"):
        # the mirror image: whole tile rows only, up to sixteen ragged last rows ride along in the first sixteen tile rows' K loops
        assert p["reduce_grid"] == 0 and p["workspace_bytes"] == 0 and p["split_first"] == 0 and p["ksplit"] == 1
        assert p["block"] == (256, 1, 1) and gy == 1 and gz == 1
        assert ("_nt" in name) == (layout == mz.LAYOUT_NT)
        assert k % 64 == 0 and 1 <= m % 256 <= 16 and m // 256 >= 16
        resident = cus - cus % 8 if cus >= 8 else cus
        assert gx == min((m // 256) * cdiv(n, 256) * batch, resident)
    elif name.endswith("_ragged"):
        # whole tile columns only: the eight or sixteen ragged last columns ride along in the first sixteen tile columns' K loops
        assert p["reduce_grid"] == 0 and p["workspace_bytes"] == 0 and p["split_first"] == 0 and p["ksplit"] == 1
        assert p["block"] == (256, 1, 1) and gy == 1 and gz == 1
        assert ("_nt" in name) == (layout == mz.LAYOUT_NT)
        assert k % 64 == 0 and n % 256 in (8, 16) and n // 256 >= 16
        resident = cus - cus % 8 if cus >= 8 else cus
        assert gx == min(cdiv(m, 256) * (n // 256) * batch, resident)
    elif "_mt256_" in name:
        assert p["reduce_grid"] == 0
        assert p["block"] == (256, 1, 1) and gy == 1
        assert ("_nt" in name) == (layout == mz.LAYOUT_NT)
        assert k % 8 == 0 and n % 8 == 0
        if "ktail" not in name:
            assert k % 64 == 0
        tm, tn = cdiv(m, 256), cdiv(n, 256)
        if persistent:
            # one workgroup per compute unit (a multiple of 8) walks all tiles of all batch members
            resident = cus - cus % 8 if cus >= 8 else cus
            assert gx == min(tm * tn * batch, resident) and p["split_first"] == 0 and p["workspace_bytes"] == 0
            assert gx == tm * tn * batch or gx % 8 == 0 or cus < 8
        elif p["split_first"] == 0:
            # an edge kernel without an edge to split: persistent over the tiles of one batch member, batch in grid.z
            resident = cus - cus % 8 if cus >= 8 else cus
            assert gx == min(tm * tn, resident) and p["workspace_bytes"] == 0
        else:
            assert name.endswith("_edge") and batch == 1
            mode, whole = p["split_first"] >> 30, (p["split_first"] & 0x3FFFFFFF) - 1
            ks = p["ksplit"]
            assert mode in (1, 2) and 2 <= ks <= 16
            nedge = tm if mode == 1 else tn
            assert whole == (tm * (tn - 1) if mode == 1 else (tm - 1) * tn)
            # persistent: the whole tiles, then the (edge tile, K range) items, shared out over one workgroup per compute unit
            resident = cus - cus % 8 if cus >= 8 else cus
            assert gx == min(whole + nedge * ks, resident)
            # the edge that is split is narrow: its partial tiles are cheap to combine
            assert (n - (tn - 1) * 256 if mode == 1 else m - (tm - 1) * 256) <= 32
            # K ranges: ceil(steps / ks) steps each, none empty, each at least 4 steps long
            nk = cdiv(k, 64)
            per = cdiv(nk, ks)
            assert per * (ks - 1) < nk and per >= 4
            # one ticket counter per edge tile, one fp32 tile per (edge tile, range)
            assert nedge <= 16384
            assert p["workspace_bytes"] >= TICKET_BYTES + nedge * ks * 256 * 256 * 4
            assert p["workspace_bytes"] < (1 << 31)
    elif name.startswith("maize_gemm_bf16_skinny_nn"):
        rows = {"maize_gemm_bf16_skinny_nn": 16, "maize_gemm_bf16_skinny_nn_m32": 32, "maize_gemm_bf16_skinny_nn_m64": 64}[name]
        # bit 1 of the launch flag: the slab's workgroups share the additions -- row-group kernels with 256 KiB or more
        # of partial tiles per slab (the kernel then uses two counters per slab and 16 bits of arrival numbers)
        shares = bool(p["split_first"] & 2)
        assert shares == (rows >= 32 and (rows // 16) * p["ksplit"] >= 16 and p["ksplit"] >= 2)
        assert not shares or (p["ksplit"] <= 16 and gx * batch <= 8192)
        assert p["block"] == (512, 1, 1)
        assert layout == mz.LAYOUT_NN and m <= rows and n % 8 == 0
        ks = p["ksplit"]
        assert gx == cdiv(n, 256) and gy == ks and 1 <= ks <= 16
        assert k % 32 == 0                                     # whole 32-row blocks
        nblk = k // 32
        assert cdiv(nblk, ks) * (ks - 1) < nblk                # no empty range
        assert ks == 1 or gx * ks * batch <= cus                # K is split only within one round of workgroups
        if ks > 1:
            assert nblk // ks >= 8                             # the 8-slot ring is filled at least once
            assert gx * batch <= 16384                         # one ticket counter per (batch member, slab)
            assert p["workspace_bytes"] >= TICKET_BYTES + gx * batch * ks * rows * 256 * 4
            assert p["workspace_bytes"] < (1 << 31)
        else:
            assert p["workspace_bytes"] == 0
    elif name.startswith("maize_gemm_bf16_skinny_nt"):
        rows = {"maize_gemm_bf16_skinny_nt": 16, "maize_gemm_bf16_skinny_nt_m32": 32, "maize_gemm_bf16_skinny_nt_m64": 64}[name]
        shares = bool(p["split_first"] & 2)
        assert shares == (rows >= 32 and (rows // 16) * p["ksplit"] >= 16 and p["ksplit"] >= 2)
        assert not shares or (p["ksplit"] <= 16 and gx * batch <= 8192)
        assert p["block"] == (512, 1, 1)
        assert layout == mz.LAYOUT_NT and m <= rows and n % 8 == 0 and k % 8 == 0
        ks = p["ksplit"]
        nblk = cdiv(k, 64)                                     # blocks of 128 bytes per row
        assert gx == cdiv(n, 256) and gy == ks and 1 <= ks <= 16
        assert cdiv(nblk, ks) * (ks - 1) < nblk                # no empty range
        if ks > 1:
            assert nblk // ks >= 4                             # the 4-slot ring is filled at least once
            assert gx * batch <= 16384
            assert p["workspace_bytes"] >= TICKET_BYTES + gx * batch * ks * rows * 256 * 4
            assert p["workspace_bytes"] < (1 << 31)
        else:
            assert p["workspace_bytes"] == 0
    elif "_t128_" in name:
        # 128 x 128 tiles, one workgroup per tile of the flattened (batch, tile) list, whole K, no workspace
        assert p["block"] == (256, 1, 1) and (gy, gz) == (1, 1)
        assert gx == cdiv(m, 128) * cdiv(n, 128) * batch
        assert k % (64 if name.startswith(("maize_gemm_bf16", "maize_gemm_f16")) else 128) == 0 and n % 8 == 0
        assert p["ksplit"] == 1 and p["workspace_bytes"] == 0 and p["reduce_grid"] == 0
    else:
        raise AssertionError(f"no invariants written for kernel {name}")


def test_north_star_configurations_get_the_kernels_they_were_designed_for():
    picks = {
        (4096, 4096, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn",
        (4000, 4104, 4032, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_ragged",     # eight ragged columns behind sixteen tile columns ride along in the whole tiles' K loops
        (4000, 4120, 4032, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_edge",       # twenty-four: a narrow last tile column, cut over K
        (4000, 4104, 4040, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_ktail_edge", # a K tail: the edge-splitting kernel takes any K % 8 == 0
        (4096, 2056, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn",            # eight tile columns only, and no round to save
        (4100, 4096, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_ragged_m",   # four ragged rows behind sixteen tile rows: the mirror image
        (4104, 4096, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt_ragged_m",
        (4120, 4096, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_edge",       # twenty-four rows: a short last tile row, cut over K
        (8192, 8192, 8192, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt",
        (16, 14336, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_skinny_nn",
        (2048, 2048, 2048, mz.LAYOUT_NN, 32): "maize_gemm_bf16_mt256_nn",
        (2048, 2048, 2048, mz.LAYOUT_NN, 1): "maize_gemm_bf16_t128_nn",              # 64 tiles: partial tiles would cost more than they save, 128 tiles of 128 rows fill half the chip, 256 of 128 x 128 all of it (23.5 -> 22.0 us)
        (768, 8192, 8192, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_h128r3",       # 384 tiles of 128 x 128 would be two rounds: 192 of 128 x 256 on three ring stages
        (1024, 4096, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_t128_nt",              # 256 tiles of 128 x 128, one round (40.7 -> 34.3 us)
        (512, 14336, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_h128r3",      # 112 tiles: 224 of 128 rows are one round
        (1024, 1024, 8192, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_h128r3_splitk",  # few tiles, a long K: 128-row tiles cut over K (ranges of 16 steps: three stages)
        (64, 4096, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt_h128r3_splitk",  # eight ranges of 8 steps: three ring stages (18.0 -> 16.7 us)
        (64, 2048, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt_h128_splitk",    # thirteen ranges of 5: two
        (16, 4096, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_skinny_nt",              # N x K weights streamed once
        (16, 14336, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_skinny_nt",
        (17, 4096, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_skinny_nt_m32",          # 17 .. 32 rows: two row groups
        (64, 14336, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_skinny_nt_m64",         # 33 .. 64 rows and many slabs: four
        (64, 14336, 2048, mz.LAYOUT_NT, 1): "maize_gemm_bf16_t128_nt",               # ... a K of up to 2048, or 192 tiles and more: one round of 128 x 128 tiles (18.6 -> 15.8 us; weights from HBM 24.5 -> 22.3)
        (64, 28672, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_t128_nt",
        (65, 14336, 4096, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt_h128r3_splitk",  # more than 64 rows
        (32, 14336, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_skinny_nn_m32",
        (64, 14336, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_skinny_nn_m64",
        (64, 8192, 8192, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_h128r3_splitk", # 64 rows, 32 slabs: the tile kernel cut over K
        (33, 17, 65, mz.LAYOUT_NN, 1): "maize_gemm_bf16_wave32",
        (4096, 4099, 4096, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_splitk",      # odd N: operands read where they lie, C written element-wise by the reduce pass
        (1000, 50257, 768, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt_splitk",
        (4096, 4096, 4100, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt_packed_gen",  # K % 8 != 0: both operands repacked, C stored by the first pass
        (64, 4096, 4100, mz.LAYOUT_NT, 1): "maize_gemm_bf16_mt256_nt_packed",        # ... few tiles: split over K, reduce pass
        (511, 513, 1027, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_packed",       # K % 8 != 0 again
        (100, 203, 72, mz.LAYOUT_NN, 1): "maize_gemm_bf16_wave32",                  # too small to pay for the copies
        (17, 50257, 768, mz.LAYOUT_NN, 1): "maize_gemm_bf16_mt256_nn_splitk",       # no copy of B is needed: odd rows are read where they lie
    }
    for (m, n, k, layout, batch), want in picks.items():
        assert mz.gemm_plan(desc(m, n, k, layout, batch), compute_units=CUS)["kernel"] == want


def test_split_k_of_few_tiles_fills_the_chip_once():
    p = mz.gemm_plan(desc(64, 4096, 4096), compute_units=CUS)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk" and 8 <= p["ksplit"] <= 16 and p["grid"] == (16 * p["ksplit"], 1, 1)
    p = mz.gemm_plan(desc(256, 256, 16384), compute_units=CUS)                    # two tiles of 128 rows
    assert 16 <= p["ksplit"] <= 64 and p["grid"] == (2 * p["ksplit"], 1, 1)
    p = mz.gemm_plan(desc(1024, 1024, 8192), compute_units=CUS)                   # 32 tiles of 128 rows
    assert 2 <= p["ksplit"] <= 16 and p["grid"][0] == 32 * p["ksplit"]
    p = mz.gemm_plan(desc(64, 4096, 4096), kernel="maize_gemm_bf16_mt256_nn_splitk", compute_units=CUS)          # the 256-row form by name
    assert 8 <= p["ksplit"] <= 16 and p["grid"] == (16 * p["ksplit"], 1, 1)
    # more than half a chip of tiles, or a short K: no split
    assert mz.gemm_plan(desc(4096, 2304, 4096), compute_units=CUS)["kernel"] == "maize_gemm_bf16_mt256_nn"
    assert mz.gemm_plan(desc(512, 512, 448), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nn"            # (in 128-row tiles: 13.3 -> 8.4 us; 128 x 128: 7.7)


def test_a_quarter_to_half_a_tile_per_compute_unit_is_split_too():
    """56 to 128 tiles on 256 compute units leave most of the chip idle for a whole walk of K: two or four K ranges
    per tile pay for the partial tiles (measured: 256 x 14336 x 4096 67 -> 46 us, 768 x 8192 x 8192 128 -> 110 us) --
    or, where one round of them is cheaper than the split, tiles of 128 rows (768 x 8192 x 8192 94 us, 2048^3 37 -> 29)."""
    p = mz.gemm_plan(desc(256, 14336, 4096), compute_units=CUS)                  # 112 tiles of 128 rows: whole K -- in 224 tiles of 128 x 128 (39.6 -> 36.6 us)
    assert p["kernel"] == "maize_gemm_bf16_t128_nn" and p["ksplit"] == 1 and p["grid"] == (224, 1, 1)
    p = mz.gemm_plan(desc(256, 14336, 4096), kernel="maize_gemm_bf16_mt256_nn_h128r3", compute_units=CUS)
    assert p["ksplit"] == 1 and p["grid"] == (112, 1, 1)
    p = mz.gemm_plan(desc(128, 14336, 4096), compute_units=CUS)                  # one row of tiles: cut over K (38 us against 54.7 whole)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk" and p["ksplit"] == 4 and p["grid"] == (224, 1, 1)   # (ranges of 16 steps: three stages)
    p = mz.gemm_plan(desc(768, 8192, 8192), compute_units=CUS)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3" and p["ksplit"] == 1 and p["grid"] == (192, 1, 1)
    p = mz.gemm_plan(desc(640, 8192, 4096, layout=mz.LAYOUT_NT), compute_units=CUS)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nt_h128r3" and p["grid"] == (160, 1, 1)
    assert mz.gemm_plan(desc(2048, 2048, 2048), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nn"
    assert mz.gemm_plan(desc(2048, 2048, 2048), compute_units=CUS)["grid"] == (256, 1, 1)
    # (products of more than 256 tiles of 128 x 128, which would be two rounds of those)
    assert mz.gemm_plan(desc(768, 8192, 960), compute_units=CUS)["kernel"] == "maize_gemm_bf16_mt256_nn_h128"          # 15 K steps: the two-stage loop
    assert mz.gemm_plan(desc(768, 8192, 1024), compute_units=CUS)["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3"       # 16 steps: three stages (512 x 8192 x 1024: 15.2 -> 14.6 us now that no step is padded)
    assert mz.gemm_plan(desc(1536, 4096, 1536), compute_units=CUS)["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3"      # 24 steps (1024 x 4096 x 1536, 128 tiles: 23.5 -> 19.7 us)
    # (up to 256 of them: one round of 128 x 128 tiles -- 512 x 8192 x 1024 14.0 -> 13.6 us, 512 x 2048 x 1792 19.8 -> 17.7)
    assert mz.gemm_plan(desc(512, 8192, 1024), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nn"
    assert mz.gemm_plan(desc(512, 2048, 1792), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nn"
    assert mz.gemm_plan(desc(512, 2048, 1792), kernel="maize_gemm_bf16_mt256_nn_h128", compute_units=CUS)["grid"] == (32, 1, 1)
    # K ranges of 28 steps or more run on the three-stage kernels too, whichever way B is stored (a row-major B costs
    # them 3-7 % more per step, not the 60 % it was once priced at)
    p = mz.gemm_plan(desc(512, 4096, 14336, layout=mz.LAYOUT_NT), compute_units=CUS)       # (61 us; two stages 67.5, 256-row split 65)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nt_h128r3_splitk" and p["ksplit"] == 4 and p["grid"] == (256, 1, 1)
    p = mz.gemm_plan(desc(512, 4096, 14336), compute_units=CUS)                            # (65 us; two stages 67.7, 256-row split 69)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk" and p["ksplit"] == 4 and p["grid"] == (256, 1, 1)
    p = mz.gemm_plan(desc(384, 4096, 14336), compute_units=CUS)                            # (51 us; 256-row split 61.6)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk"
    # a named 128-row split kernel gets the same number of ranges for either layout of B
    for m, n, k in ((512, 4096, 14336), (1024, 4096, 14336), (512, 8192, 8192)):
        nn_plan = mz.gemm_plan(desc(m, n, k), kernel="maize_gemm_bf16_mt256_nn_h128r3_splitk", compute_units=CUS)
        nt_plan = mz.gemm_plan(desc(m, n, k, layout=mz.LAYOUT_NT), kernel="maize_gemm_bf16_mt256_nt_h128r3_splitk", compute_units=CUS)
        assert nn_plan["ksplit"] == nt_plan["ksplit"] and nn_plan["grid"] == nt_plan["grid"], (m, n, k, nn_plan, nt_plan)
    # two long K ranges on most compute units cost more per step than the model's 0.52 (0.66-0.74 measured): one round of
    # 128 x 128 tiles takes over (N x K | K x N: 512 x 8192 x 8192 70.2 -> 58.5 us | 69.2 -> 63.0, 2048 x 2048 x 8192 69.5 -> 62.5 | 69.4 -> 65.0,
    # 384 x 8192 x 8192 N x K 57.8 -> 52.5)
    for m, n, k in ((512, 8192, 8192), (2048, 2048, 8192)):
        assert mz.gemm_plan(desc(m, n, k, layout=mz.LAYOUT_NT), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nt"
        assert mz.gemm_plan(desc(m, n, k), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nn"
        p = mz.gemm_plan(desc(m, n, k), kernel="maize_gemm_bf16_mt256_nn_h128r3_splitk", compute_units=CUS)
        assert p["ksplit"] == 2
    assert mz.gemm_plan(desc(384, 8192, 8192, layout=mz.LAYOUT_NT), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nt"
    # ... and against the 256-row kernels' shorter ranges, from 96 steps per range on (1024 x 4096 x 14336: two ranges of 112 steps
    # 112.9 us, 128 x 128 tiles 110.6, the 256-row kernel in four ranges 104.6; 768 x 4096 x 14336 97.5 against 85.7 in five)
    for layout, tag in ((mz.LAYOUT_NN, "nn"), (mz.LAYOUT_NT, "nt")):
        p = mz.gemm_plan(desc(1024, 4096, 14336, layout=layout), compute_units=CUS)
        assert p["kernel"] == f"maize_gemm_bf16_mt256_{tag}_splitk" and p["ksplit"] == 4
        p = mz.gemm_plan(desc(768, 4096, 14336, layout=layout), compute_units=CUS)
        assert p["kernel"] == f"maize_gemm_bf16_mt256_{tag}_splitk" and p["ksplit"] == 5
        p = mz.gemm_plan(desc(1024, 4096, 11008, layout=layout), kernel=f"maize_gemm_bf16_mt256_{tag}_h128r3_splitk", compute_units=CUS)
        assert p["ksplit"] == 2                                                            # (86 steps per range: the 128-row cut stays ahead of the 256-row one, 84.7 us)
    # (... where N x K has one round of 128 x 128 tiles at 77.8 us; K x N 85.2 against 86.2: the cut)
    assert mz.gemm_plan(desc(1024, 4096, 11008, layout=mz.LAYOUT_NT), compute_units=CUS)["kernel"] == "maize_gemm_bf16_t128_nt"
    assert mz.gemm_plan(desc(1024, 4096, 11008), compute_units=CUS)["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk"
    p = mz.gemm_plan(desc(384, 6144, 4096), compute_units=CUS)                             # (three ranges 33 us; two 35; whole 39)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk" and p["ksplit"] == 3 and p["grid"] == (216, 1, 1)
    p = mz.gemm_plan(desc(384, 6144, 4096, layout=mz.LAYOUT_NT), compute_units=CUS)        # (N x K: 144 tiles of 128 x 128 30.9 us, three ranges 31.5)
    assert p["kernel"] == "maize_gemm_bf16_t128_nt" and p["grid"] == (144, 1, 1)
    assert mz.gemm_plan(desc(4096, 2304, 2048), compute_units=CUS)["kernel"] == "maize_gemm_bf16_mt256_nn"       # 288 tiles of 128 rows would need two rounds
    assert mz.gemm_plan(desc(1024, 14336, 4096), compute_units=CUS)["kernel"] == "maize_gemm_bf16_mt256_nn"   # 224 tiles: one round as it is


def test_skinny_nt_takes_any_n():
    """N x K weights with an odd number of rows (50257) keep the streaming kernel; C then goes out element by element."""
    p = mz.gemm_plan(desc(16, 50257, 768, layout=mz.LAYOUT_NT), compute_units=CUS)
    assert p["kernel"] == "maize_gemm_bf16_skinny_nt" and p["split_first"] == 1 and p["grid"][0] == cdiv(50257, 256)
    p = mz.gemm_plan(desc(16, 50264, 768, layout=mz.LAYOUT_NT), compute_units=CUS)
    assert p["kernel"] == "maize_gemm_bf16_skinny_nt" and p["split_first"] == 0
    # a K x N B with odd N has rows of B on 2-byte boundaries only: the NN streaming kernel takes them too
    p = mz.gemm_plan(desc(16, 50257, 768), compute_units=CUS)
    assert p["kernel"] == "maize_gemm_bf16_skinny_nn" and p["split_first"] == 1
    assert mz.gemm_plan(desc(16, 50264, 768), compute_units=CUS)["split_first"] == 0
    # ... but A's rows must be 16-byte material (its blocks are fetched in fragment order, 16 bytes per lane)
    d = desc(16, 50257, 768)
    d.a.ptr += 2
    assert "skinny" not in mz.gemm_plan(d, compute_units=CUS)["kernel"]


def test_skinny_split_fills_the_chip_without_overshooting():
    p = mz.gemm_plan(desc(16, 14336, 4096), compute_units=CUS)
    assert p["grid"] == (56, 4, 1)                              # 224 workgroups on 256 compute units
    p = mz.gemm_plan(desc(16, 14336, 4096), compute_units=64)
    assert p["grid"] == (56, 1, 1)                              # already a workgroup per compute unit
    p = mz.gemm_plan(desc(16, 256, 8192), compute_units=CUS)
    assert p["grid"][0] == 1 and p["ksplit"] == 16             # capped at 16 ranges


def test_plan_rejects_bad_arguments():
    d = desc(64, 64, 64)
    with pytest.raises(mz.MaizeError) as e:
        mz.gemm_plan(d, kernel="no_such_kernel")
    assert e.value.code == _ffi.MAIZE_ERR_KERNEL
    with pytest.raises(mz.MaizeError) as e:
        mz.gemm_plan(d, compute_units=0)
    assert e.value.code == _ffi.MAIZE_ERR_ARG
    assert _ffi.lib().maize_hip_gemm_plan(None, None, 256, None) == _ffi.MAIZE_ERR_NULL
    bad = desc(64, 64, 64)
    bad.c.nrows = 65
    with pytest.raises(mz.MaizeError) as e:
        mz.gemm_plan(bad)
    assert e.value.code == _ffi.MAIZE_ERR_SHAPE


def ex_desc(m, n, k, layout=mz.LAYOUT_NN, batch=1, in_type=mz.IN_BF16, lda=0, ldb=0, ldc=0, esz=2, csz=2, base=0x10000):
    a = mz.GlobalMatrix(base, m, k)
    b = mz.GlobalMatrix(base + (1 << 40), k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(base + (1 << 40), n, k)
    c = mz.GlobalMatrix(base + (2 << 40), m, n)
    sa = (m - 1) * (lda or k) + k
    sb = ((k - 1) * (ldb or n) + n) if layout == mz.LAYOUT_NN else ((n - 1) * (ldb or k) + k)
    sc = (m - 1) * (ldc or n) + n
    return mz.gemm_ex_desc(a, b, c, layout=layout, batch=batch, stride_a=sa, stride_b=sb, stride_c=sc, lda=lda, ldb=ldb, ldc=ldc,
                           in_type=in_type)


def test_the_dispatchers_choice_always_plans_when_named():
    """plan(NULL) names a kernel; plan(that kernel) must then succeed too -- or plan(NULL) itself must be the error.
    Fuzzed descriptors include rows of 16 MiB and more (beyond the fp32 / fp64 kernels' tile offsets) and products
    whose packed form has more partial tiles than the workspace can address."""
    import random
    rng = random.Random(7)
    cases = [
        dict(m=100, n=15, k=5000000, layout=mz.LAYOUT_NT, in_type=mz.IN_F64),
        dict(m=16, n=4194320, k=1024, layout=mz.LAYOUT_NN, in_type=mz.IN_F32),
        dict(m=40000, n=40001, k=1024, layout=mz.LAYOUT_NN),
        dict(m=4096, n=1048576, k=63, layout=mz.LAYOUT_NT, in_type=mz.IN_E4M3),
        dict(m=14336, n=14336, k=24, layout=mz.LAYOUT_NN, batch=32, in_type=mz.IN_E4M3),
        dict(m=14336, n=14337, k=24, layout=mz.LAYOUT_NN, batch=32),
    ]
    dims = [1, 7, 15, 16, 24, 63, 64, 100, 257, 1024, 4099, 40001, 1 << 20, (1 << 22) + 16, 5000000]
    for _ in range(400):
        m, n, k = rng.choice(dims), rng.choice(dims), rng.choice(dims)
        if m * n > 1 << 34 or m * k > 1 << 34 or n * k > 1 << 34:
            continue
        cases.append(dict(m=m, n=n, k=k, layout=rng.choice([mz.LAYOUT_NN, mz.LAYOUT_NT]), batch=rng.choice([1, 1, 2, 32]),
                          in_type=rng.choice([mz.IN_BF16, mz.IN_F16, mz.IN_E4M3, mz.IN_E5M2, mz.IN_F32, mz.IN_F64]),
                          lda=rng.choice([0, 0, k + 8, k + (1 << 22)])))
    refused = 0
    for kw in cases:
        d = ex_desc(**kw)
        try:
            p = mz.gemm_plan(d, compute_units=CUS)
        except mz.MaizeError as e:
            if e.code == _ffi.MAIZE_ERR_SHAPE:     # the any-shape kernel's grid: 64 rows per workgroup, at most 65535 of them
                assert kw["m"] > 64 * 65535 and "wave32" in e.message, (kw, e)
                continue
            assert e.code == _ffi.MAIZE_ERR_KERNEL and kw.get("in_type") in (mz.IN_F32, mz.IN_F64), (kw, e)
            refused += 1
            continue
        q = mz.gemm_plan(d, kernel=p["kernel"], compute_units=CUS)     # raises if the kernel refuses or cannot plan
        assert q["grid"] == p["grid"] and q["workspace_bytes"] == p["workspace_bytes"], (kw, p, q)
    assert refused >= 2                                          # the two wide cases at the top, at least


def test_huge_packed_products_fall_through_to_the_any_shape_kernel():
    for kw in (dict(m=40000, n=40001, k=1024), dict(m=4096, n=1048576, k=63, layout=mz.LAYOUT_NT, in_type=mz.IN_E4M3),
               dict(m=14336, n=14336, k=24, batch=32, in_type=mz.IN_E4M3)):
        p = mz.gemm_plan(ex_desc(**kw), compute_units=CUS)
        assert p["kernel"] == "maize_gemm_bf16_wave32", (kw, p)


def test_rows_beyond_the_wide_kernels_offsets_are_an_error_not_a_launch():
    for kw in (dict(m=100, n=15, k=5000000, layout=mz.LAYOUT_NT, in_type=mz.IN_F64),
               dict(m=16, n=4194320, k=1024, layout=mz.LAYOUT_NN, in_type=mz.IN_F32)):
        with pytest.raises(mz.MaizeError) as e:
            mz.gemm_plan(ex_desc(**kw), compute_units=CUS)
        assert e.value.code == _ffi.MAIZE_ERR_KERNEL


def _padding_step_is_the_last_tile_of_b(k, ksplit, steps_per_trip):
    """True when a K range that is not the last one is padded (to a whole trip of the unrolled loop) with a step
    that falls on B's last K tile, which belongs to a later range."""
    nk_all = cdiv(k, 64)
    per = cdiv(nk_all, ksplit)
    for z in range(ksplit):
        kt0 = z * per
        nk = max(0, min(per, nk_all - kt0))
        padded = cdiv(nk, steps_per_trip) * steps_per_trip
        if nk and kt0 + nk < nk_all and kt0 + padded > nk_all - 1:
            return True
    return False


def test_the_special_value_families_hold_a_range_padded_with_bs_last_tile():
    """Odd N, row-major B: the kernels write B's last element into the landed K tile that holds row K - 1.  A split
    whose non-final range is padded with that very tile is the case where the write must not happen (A is zero
    there, the element may be Inf).  The dispatcher produces such splits on its own; the GPU special-value test has
    to keep one, whatever the cost model does later."""
    from tests.test_gpu_special_values import FAMILIES
    hit = []
    for name, m, n, k, layout in FAMILIES:
        if layout != mz.LAYOUT_NN or n % 2 == 0:
            continue
        p = mz.gemm_plan(desc(m, n, k), kernel=name, compute_units=CUS)
        if not p["kernel"].endswith("_splitk") or p["ksplit"] < 2:
            continue
        if _padding_step_is_the_last_tile_of_b(k, p["ksplit"], 3 if "r3" in p["kernel"] else 2):
            hit.append((p["kernel"], name is None))
    assert any(kern.endswith("_h128_splitk") for kern, _ in hit), hit
    assert any(kern.endswith("_h128r3_splitk") for kern, _ in hit), hit
    assert any(kern == "maize_gemm_bf16_mt256_nn_splitk" for kern, _ in hit), hit
    assert any(auto for _, auto in hit), hit


def _steps_of_the_ranges(k, ksplit):
    nk = cdiv(k, 64)
    per = cdiv(nk, max(1, ksplit))
    return [min(per, nk - z * per) for z in range(max(1, ksplit)) if nk - z * per > 0]


def test_the_named_three_stage_cases_have_a_ragged_m_and_a_step_count_off_three():
    """The GPU suite runs the three-stage 128-row kernels by name (tests/test_gpu_random_products.py: H128R3_CASES).  Here,
    without a device: each kernel accepts its case, M is no multiple of 128, and some K range runs a number of steps
    that is no multiple of three (the loop runs three steps per trip; the steps left over run on copies of the step behind
    it); both layouts, the plain, general and split-K forms are all there."""
    from tests.test_gpu_random_products import H128R3_CASES
    for name, layout, m, n, k, kw in H128R3_CASES:
        brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
        x = mz.gemm_ex_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x1000, brows, bcols), mz.GlobalMatrix(0x1000, m, n), layout=layout,
                            in_type=mz.IN_F16 if kw.get("half") else mz.IN_BF16, out_type=mz.OUT_F32 if kw.get("out_f32") else mz.OUT_SAME,
                            alpha=kw.get("alpha", 1.0), beta=kw.get("beta", 0.0))
        plan = mz.gemm_plan(x, kernel=name, compute_units=CUS)
        assert plan["kernel"] == name and m % 128 != 0, name
        assert any(s % 3 for s in _steps_of_the_ranges(k, plan["ksplit"] if name.endswith("_splitk") else 1)), (name, plan)
    names = {c[0] for c in H128R3_CASES}
    for lay in ("nn", "nt"):
        for form in ("_h128r3", "_h128r3_gen", "_h128r3_splitk"):
            assert f"maize_gemm_bf16_mt256_{lay}{form}" in names


def test_operands_past_the_memory_side_cache_are_priced_by_their_bytes_too():
    """The 128-row tile choice prices bytes as well as K steps: a 470 MB weight matrix (28672 x 8192) against 96 .. 128
    rows is bound by its stream from HBM, which two K ranges on 224 compute units draw faster than 112 whole tiles on
    112 of them (measured, K x N: 95.7 / 100.5 us against 123.6 / 129.9; N x K: 119.2 / 122.8 against 122.9 / 125.0);
    with 192 rows the whole tiles already occupy 224 units and stay (122.9 us against 146.3 split).  Operands that fit
    the cache keep the choice the K steps make."""
    for m in (96, 128):
        for layout in (mz.LAYOUT_NN, mz.LAYOUT_NT):
            p = mz.gemm_plan(desc(m, 28672, 8192, layout), kernel=f"maize_gemm_bf16_mt256_{'nn' if layout == mz.LAYOUT_NN else 'nt'}_h128r3_splitk", compute_units=CUS)
            assert p["ksplit"] == 2 and p["grid"][0] == 224, p
            # ... and 224 tiles of 128 x 128 draw the same stream without the second launch (N x K 119.7 -> 107.4 us, K x N 99.2 -> 97.9)
            p = mz.gemm_plan(desc(m, 28672, 8192, layout), compute_units=CUS)
            assert "_t128_" in p["kernel"] and p["grid"][0] == 224, p
    for layout in (mz.LAYOUT_NN, mz.LAYOUT_NT):
        p = mz.gemm_plan(desc(192, 28672, 8192, layout), compute_units=CUS)
        assert p["kernel"].endswith("_h128r3") and p["ksplit"] <= 1, p
    p = mz.gemm_plan(desc(96, 28672, 4096), compute_units=CUS)          # 235 MB: stays in whole tiles (of 128 x 128: one round of 224)
    assert p["kernel"] == "maize_gemm_bf16_t128_nn" and p["ksplit"] == 1, p


def test_the_boundary_between_whole_128_row_tiles_and_their_split():
    """640 x 8192 x 4096 with B stored N x K, 160 tiles of 128 x 256: whole tiles on three ring stages (45.9 us) beat
    the split over K (56.7 us), which an earlier rule took here."""
    p = mz.gemm_plan(desc(640, 8192, 4096, mz.LAYOUT_NT), compute_units=CUS)
    assert p["kernel"] == "maize_gemm_bf16_mt256_nt_h128r3" and p["grid"][0] == 160, p


def test_an_odd_number_of_k_steps_takes_the_loop_that_leaves_after_its_first_step():
    """The plain 256-row kernel's statement loop pads an odd step count with a step on a zero tile; the assembly loop
    does not.  Even counts, K tails, split edges and the general epilogue keep their kernels."""
    for layout, tag in ((mz.LAYOUT_NN, "nn"), (mz.LAYOUT_NT, "nt")):
        for k in (192, 576, 1088, 3008):
            assert mz.gemm_plan(desc(4096, 4096, k, layout), compute_units=CUS)["kernel"] == f"maize_gemm_bf16_mt256_{tag}_asm", (tag, k)
        for k in (256, 1024, 4096):
            assert mz.gemm_plan(desc(4096, 4096, k, layout), compute_units=CUS)["kernel"] == f"maize_gemm_bf16_mt256_{tag}", (tag, k)
        assert mz.gemm_plan(desc(4096, 4096, 576 + 8, layout), compute_units=CUS)["kernel"] == f"maize_gemm_bf16_mt256_{tag}_ktail"
        assert mz.gemm_plan(desc(4000, 4120, 4032, layout), compute_units=CUS)["kernel"] == f"maize_gemm_bf16_mt256_{tag}_edge"
        x = ex_desc(4096, 4096, 576, layout)
        x.alpha = 0.5
        p = mz.gemm_plan(x, compute_units=CUS)
        assert p["kernel"] == f"maize_gemm_bf16_mt256_{tag}_gen", p
