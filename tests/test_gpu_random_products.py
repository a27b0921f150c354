"""Seeded random products through the dispatcher (kernel = NULL): extents drawn around the boundaries the kernels care
about (16 / 32 / 64 rows, multiples of 8, 16, 64, 128 and 256 and their neighbours), both layouts, bf16 / half / E4M3 /
E5M2 operands, padded and odd leading dimensions, plain and scaled epilogues, bf16 / half / fp32 C.  Every case is
checked against the oracle to the bar of its operand type (the helpers of test_gpu_gemm_ex.py and
test_gpu_gemm_f8.py); the test also reports which kernels the cases reached."""
import collections
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.test_gpu_gemm_ex import run_ex
from tests.test_gpu_gemm_f8 import run_f8

pytestmark = pytest.mark.gpu


def _say(msg):
    print(f"[random] {msg}", file=sys.stderr, flush=True)


def draw_extent(rng, kind):
    """kind 'rows': mostly small (the few-row kernels' range) with some large; 'cols' / 'depth': around tile boundaries."""
    if kind == "rows" and rng.random() < 0.4:
        return int(rng.choice([1, 2, 7, 13, 16, 17, 24, 29, 32, 33, 48, 50, 63, 64, 65, 100, 128]))
    base = int(rng.choice([64, 256, 512, 768, 1024, 2048, 4096, 8192] if kind != "depth" else [128, 256, 512, 1024, 2048, 4096, 8192]))
    base *= int(rng.choice([1, 1, 1, 2, 3]))
    delta = int(rng.choice([0, 0, 0, 0, 0, 0, 8, -8, 16, -16, 24, 40, 64, -64, 1, -3]))
    return max(1, base + delta)


def draw_case(rng):
    fmt = str(rng.choice(["bf16", "bf16", "f16", "e4m3", "e5m2"]))
    layout = int(rng.choice([mz.LAYOUT_NN, mz.LAYOUT_NT]))
    while True:
        m, n, k = draw_extent(rng, "rows"), draw_extent(rng, "cols"), draw_extent(rng, "depth")
        if m * n * k <= 6e8 and m * n <= 4e6:          # keeps the oracle to a fraction of a second per case
            break
    bcols = n if layout == mz.LAYOUT_NN else k
    def ld(cols):
        r = rng.random()
        return None if r < 0.65 else cols + int(rng.choice([8, 16, 64])) if r < 0.95 else cols + int(rng.choice([1, 3, 5, 7]))
    kw = dict(lda=ld(k), ldb=ld(bcols), ldc=ld(n))
    r = rng.random()
    if r < 0.25:
        kw.update(alpha=float(rng.choice([0.5, -1.25, 2.0])), beta=float(rng.choice([0.0, 0.75, -0.5, 1.0])))
    elif r < 0.4:
        kw.update(out_f32=True, alpha=float(rng.choice([1.0, 3.0])), beta=float(rng.choice([0.0, -0.5])))
    return fmt, layout, m, n, k, kw


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_random_products_through_the_dispatcher(ctx, oracle, seed):
    rng = np.random.default_rng(seed)
    reached = collections.Counter()
    for i in range(40):
        fmt, layout, m, n, k, kw = draw_case(rng)
        label = f"random {seed}.{i}"
        _say(f"{label}: {fmt} {'NT' if layout else 'NN'} {m}x{n}x{k} {kw}")
        if fmt in ("bf16", "f16"):
            took = run_ex(ctx, oracle, m, n, k, layout=layout, half=fmt == "f16", seed=seed * 100 + i, label=label, **kw)
        else:
            took = run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, seed=seed * 100 + i, label=label, **kw)
        reached[took.replace("maize_gemm_", "")] += 1
    _say(f"seed {seed}: kernels reached: {dict(reached)}")
    assert len(reached) >= 8           # the draw is wide enough to be worth its time


def draw_midsize_case(rng):
    """Half a round of 128-row tiles, give or take, and a K of 24 to 72 steps: the range where the dispatcher moves between
    the 128-row kernels on two and three ring stages, their split-K form and the 256-row kernels."""
    fmt = str(rng.choice(["bf16", "bf16", "f16", "e4m3", "e5m2"]))
    layout = int(rng.choice([mz.LAYOUT_NN, mz.LAYOUT_NT]))
    m = int(rng.choice([384, 512, 640, 768, 1000, 1024, 1536, 2048])) + int(rng.choice([0, 0, 0, 8, -8, 24]))
    n = int(rng.choice([1024, 2048, 3072, 4096])) + int(rng.choice([0, 0, 0, 16, -16, 48]))
    step = 64 if fmt in ("bf16", "f16") else 128
    k = int(rng.integers(24, 73)) * step + int(rng.choice([0, 0, 0, 16, -16, 32]))
    bcols = n if layout == mz.LAYOUT_NN else k
    def ld(cols):
        return None if rng.random() < 0.7 else cols + int(rng.choice([16, 64]))
    kw = dict(lda=ld(k), ldb=ld(bcols), ldc=ld(n))
    r = rng.random()
    if r < 0.25:
        kw.update(alpha=float(rng.choice([0.5, -1.25])), beta=float(rng.choice([0.0, 0.75])))
    elif r < 0.4:
        kw.update(out_f32=True, alpha=float(rng.choice([1.0, 3.0])), beta=float(rng.choice([0.0, -0.5])))
    return fmt, layout, m, n, k, kw


@pytest.mark.parametrize("seed", [11, 12])
def test_random_midsize_products_with_a_long_k(ctx, oracle, seed):
    rng = np.random.default_rng(seed)
    reached = collections.Counter()
    for i in range(12):
        fmt, layout, m, n, k, kw = draw_midsize_case(rng)
        label = f"midsize {seed}.{i}"
        _say(f"{label}: {fmt} {'NT' if layout else 'NN'} {m}x{n}x{k} {kw}")
        if fmt in ("bf16", "f16"):
            took = run_ex(ctx, oracle, m, n, k, layout=layout, half=fmt == "f16", seed=seed * 100 + i, label=label, **kw)
        else:
            took = run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, seed=seed * 100 + i, label=label, **kw)
        reached[took.replace("maize_gemm_", "")] += 1
    _say(f"seed {seed}: kernels reached: {dict(reached)}")
    assert any("h128r3" in name for name in reached)


# The three-stage 128-row kernels by name, not by the luck of a draw: every one of them on a ragged M (no multiple of
# 128) and a K whose step count is no multiple of three (the loop runs three steps per trip and pads with zero tiles),
# both layouts, K tails for the kernels that take them, half operands once.  (The loop runs three steps per trip; the one
# or two steps left over have copies of their own behind it.)
H128R3_CASES = [
    ("maize_gemm_bf16_mt256_nn_h128r3", mz.LAYOUT_NN, 1000, 2048, 64 * 31, {}),
    ("maize_gemm_bf16_mt256_nt_h128r3", mz.LAYOUT_NT, 904, 1024, 64 * 32, {}),
    ("maize_gemm_bf16_mt256_nn_h128r3_gen", mz.LAYOUT_NN, 1000, 2056, 64 * 34 + 8, dict(alpha=-1.25, beta=0.75)),
    ("maize_gemm_bf16_mt256_nt_h128r3_gen", mz.LAYOUT_NT, 648, 1032, 64 * 31 + 16, dict(out_f32=True, alpha=3.0, beta=-0.5)),
    ("maize_gemm_f16_mt256_nn_h128r3_gen", mz.LAYOUT_NN, 520, 1024, 64 * 29, dict(half=True)),
    ("maize_gemm_bf16_mt256_nn_h128r3_splitk", mz.LAYOUT_NN, 392, 1024, 64 * 61, {}),
    ("maize_gemm_bf16_mt256_nt_h128r3_splitk", mz.LAYOUT_NT, 264, 2048, 64 * 61 + 8, {}),
    ("maize_gemm_f16_mt256_nt_h128r3_splitk", mz.LAYOUT_NT, 200, 1536, 64 * 64, dict(half=True, out_f32=True)),
]


@pytest.mark.parametrize("case", H128R3_CASES, ids=lambda c: f"{c[0].replace('maize_gemm_', '')}-{c[2]}x{c[3]}x{c[4]}")
def test_the_three_stage_kernels_by_name(ctx, oracle, case):
    name, layout, m, n, k, kw = case
    took = run_ex(ctx, oracle, m, n, k, layout=layout, kernel=name, seed=7, label=f"named {name}", **kw)
    assert took == name
