"""maize_hip_gemm_bf16_noalloc against maize_hip_gemm_bf16: same kernels, same bits, scratch from the fixed
per-GPU array instead of an allocated workspace.  Runs last (file name): a failure here must not hide other tests."""
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.gpu_util import CANARY, PAD

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _both(ctx, m, n, k, layout=mz.LAYOUT_NN, dist="normal"):
    """Runs the product through both entry points (C surrounded by canaries) and returns the two results, the
    plan and the inputs."""
    if dist == "normal":
        a, b = mz.gen.normal_bf16(m * k, mz.gen.SEED_A, 1.0), mz.gen.normal_bf16(k * n, mz.gen.SEED_B, 0.02)
    else:
        a, b = mz.gen.uniform_bf16(m * k, mz.gen.SEED_A), mz.gen.uniform_bf16(k * n, mz.gen.SEED_B)
    if layout == mz.LAYOUT_NT:
        b = np.ascontiguousarray(b.reshape(k, n).T).ravel()
    da, db = ctx.upload(a), ctx.upload(b)
    outs = []
    plan = None
    try:
        for noalloc in (False, True):
            dc = ctx.upload(np.full(m * n + 2 * PAD, CANARY, dtype=np.uint16))
            try:
                desc = mz.gemm_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n) if layout == mz.LAYOUT_NN else mz.Matrix(db, n, k),
                                    mz.Matrix(dc, m, n, offset_elems=PAD), layout=layout)
                plan = mz.gemm_plan(desc, compute_units=ctx.info()["compute_units"])
                _say(f"noalloc: {m}x{n}x{k} layout={layout} entry={'noalloc' if noalloc else 'alloc'} kernel={plan['kernel']} "
                     f"ksplit={plan['ksplit']} workspace={plan['workspace_bytes']}")
                if noalloc:
                    ctx.gemm_bf16_noalloc(desc)
                else:
                    ctx.gemm_bf16(desc)
                ctx.sync()
                out = dc.download(np.uint16)
            finally:
                dc.free()
            assert np.all(out[:PAD] == CANARY) and np.all(out[PAD + m * n:] == CANARY), "kernel wrote outside C"
            outs.append(out[PAD:PAD + m * n])
    finally:
        da.free(); db.free()
    return outs[0], outs[1], plan, a, b


def test_noalloc_matches_the_allocating_entry_point_twice_in_a_row(ctx, oracle):
    # Two calls in a row on the same GPU, the second with a smaller input: it finds the first call's partial tiles in
    # the scratch array and must not be disturbed by them.  Both shapes split K (the scratch is really used).
    for (m, n, k) in ((16, 14336, 4096), (9, 2304, 2048)):
        ref, got, plan, a, b = _both(ctx, m, n, k)
        assert plan["workspace_bytes"] > 0 and plan["ksplit"] > 1, plan
        assert plan["workspace_bytes"] <= mz.NOALLOC_MAX_WORKSPACE_BYTES
        assert np.array_equal(ref, got), f"{m}x{n}x{k}: {int((ref != got).sum())} elements differ"
        full, f64, ab = oracle.ref_gemm(a, b, m, n, k, want_f64=True, want_abs=True)
        s = oracle.compare(got, full, f64, ab, k)
        oracle.assert_parity(s, "noalloc")


@pytest.mark.parametrize("shape", [(64, 4096, 4096, mz.LAYOUT_NN), (16, 4096, 4096, mz.LAYOUT_NT), (4000, 4120, 4032, mz.LAYOUT_NN),
                                   (512, 512, 512, mz.LAYOUT_NN)],
                         ids=["splitk_mt256", "skinny_nt", "edge_split", "no_scratch_needed"])
def test_noalloc_every_scratch_user(ctx, shape):
    m, n, k, layout = shape
    ref, got, plan, _, _ = _both(ctx, m, n, k, layout=layout, dist="uniform")
    assert np.array_equal(ref, got), f"{plan['kernel']}: {int((ref != got).sum())} elements differ"


def test_noalloc_refuses_what_does_not_fit(ctx):
    # A packed product: 272 partial tiles of 256 KiB and two operand copies, far beyond the fixed array.
    m, n, k = 4096, 4099, 4096
    da, db, dc = ctx.malloc(m * k * 2), ctx.malloc(k * n * 2), ctx.upload(np.full(m * n, CANARY, dtype=np.uint16))
    try:
        desc = mz.gemm_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n), mz.Matrix(dc, m, n))
        plan = mz.gemm_plan(desc, compute_units=ctx.info()["compute_units"])
        assert plan["workspace_bytes"] > mz.NOALLOC_MAX_WORKSPACE_BYTES, plan
        with pytest.raises(mz.MaizeError) as e:
            ctx.gemm_bf16_noalloc(desc)
        assert e.value.code == -7 and "scratch" in e.value.message, e.value
        ctx.sync()
        assert np.all(dc.download(np.uint16) == CANARY), "a refused call launched something"
    finally:
        da.free(); db.free(); dc.free()


def test_noalloc_reset_restores_the_ticket_counters(ctx):
    """maize_hip_noalloc_reset is the recovery after calls that overlapped on one GPU against the rule, or after an
    aborted launch: it zeroes the array's ticket counters.  Here a product runs, the counters are
    reset, and the next product -- a kernel that takes tickets -- is bit-identical
    to the allocating entry point's."""
    m, n, k = 16, 14336, 4096
    ref, got, plan, _, _ = _both(ctx, m, n, k)
    assert plan["ksplit"] > 1 and np.array_equal(ref, got)
    _say("noalloc: reset")
    ctx.noalloc_reset()
    ctx.sync()
    ref2, got2, _, _, _ = _both(ctx, m, n, k)
    assert np.array_equal(ref2, ref) and np.array_equal(got2, ref)
    with pytest.raises(mz.MaizeError):
        mz._ffi.check(mz._ffi.lib().maize_hip_noalloc_reset(None, None))
