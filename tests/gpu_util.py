"""Shared helpers of the GPU parity tests: upload, launch through the C ABI, download, compare."""
import numpy as np

import maize_amd as mz

CANARY = 0xDEAD  # bf16 bit pattern written around C; must survive every launch
PAD = 64         # canary elements on each side of C


def f32_of(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def run_gemm(ctx, a, b, m, n, k, layout=mz.LAYOUT_NN, batch=1, stride_a=None, stride_b=None, stride_c=None,
             kernel=None, stream=None):
    """C = A.B on the device through maize_hip_gemm_bf16[_with]; returns C as uint16 of
    (batch-1)*stride_c + m*n elements.  C is surrounded by canaries, gaps between batch members
    are pre-filled with the canary too, and all of them are checked after the launch."""
    a = np.ascontiguousarray(a, dtype=np.uint16).ravel()
    b = np.ascontiguousarray(b, dtype=np.uint16).ravel()
    sa = m * k if stride_a is None else stride_a
    sb = k * n if stride_b is None else stride_b
    sc = m * n if stride_c is None else stride_c
    clen = (batch - 1) * sc + m * n
    da, db = ctx.upload(a), ctx.upload(b)
    chost = np.full(clen + 2 * PAD, CANARY, dtype=np.uint16)
    dc = ctx.upload(chost)
    try:
        A = mz.Matrix(da, m, k)
        B = mz.Matrix(db, k, n) if layout == mz.LAYOUT_NN else mz.Matrix(db, n, k)
        Cm = mz.Matrix(dc, m, n, offset_elems=PAD)
        desc = mz.gemm_desc(A, B, Cm, layout=layout, batch=batch, stride_a=sa, stride_b=sb, stride_c=sc)
        ctx.gemm_bf16(desc, stream=stream, kernel=kernel)
        ctx.sync(stream)
        out = dc.download(np.uint16)
    finally:
        da.free(); db.free(); dc.free()
    assert np.all(out[:PAD] == CANARY) and np.all(out[PAD + clen:] == CANARY), "kernel wrote outside C"
    c = out[PAD:PAD + clen]
    for i in range(batch - 1):
        gap = c[i * sc + m * n:(i + 1) * sc]
        assert np.all(gap == CANARY), "kernel wrote into the gap between batch members"
    return c


def check_against_oracle(oracle, got, a, b, m, n, k, layout=mz.LAYOUT_NN, batch=1, stride_a=None, stride_b=None,
                         stride_c=None, label=""):
    """Full comparison against the oracle; returns the stats dict and asserts the parity bar."""
    sc = m * n if stride_c is None else stride_c
    ref, f64, ab = oracle.ref_gemm(a, b, m, n, k, layout=layout, batch=batch, stride_a=stride_a, stride_b=stride_b,
                                   stride_c=stride_c, want_f64=True, want_abs=True)
    g = np.concatenate([got[i * sc:i * sc + m * n] for i in range(batch)])
    r = np.concatenate([ref[i * sc:i * sc + m * n] for i in range(batch)])
    s = oracle.compare(g, r, f64, ab, k)
    oracle.assert_parity(s, label)                 # no failure, and the sums as accurate as fp32 accumulation is
    return s


def sample_rows(m, count=40, tile=256, seed=0):
    """Rows that cover the first/last rows, both sides of every kind of tile boundary and random ones."""
    rows = {0, 1, m - 1, m - 2, m // 2}
    for t in (16, 32, 64, 128, tile):
        for base in (t, (m // t) * t):
            for d in (-1, 0, 1):
                rows.add(base + d)
    rng = np.random.default_rng(seed)
    rows.update(int(x) for x in rng.integers(0, m, count))
    return np.array(sorted(r for r in rows if 0 <= r < m), dtype=np.uint32)


def check_rows_against_oracle(oracle, got, a, b, m, n, k, rows, layout=mz.LAYOUT_NN, label=""):
    ref, f64, ab = oracle.ref_gemm_rows(a, b, m, n, k, rows, layout=layout)
    g = np.asarray(got, dtype=np.uint16).reshape(m, n)[rows]
    s = oracle.compare(g, ref, f64, ab, k)
    oracle.assert_parity(s, label)
    return s
