"""CPU model of the two LDS pipelines (prime / wait-consume-refill / drain), checked for the
properties the reference's CpAsyncPipeline promises (crates/maize_core/src/intrinsics/cuda/
cp_async.rs:122-210): every K tile is copied exactly once and consumed exactly once, in order,
never before its copy has completed for every wave, and no ring slot is refilled while a wave
may still be reading it.

The model replays each wave's instruction stream as the kernels issue it (the request slots,
ring depth and counter waits are read from the kernel sources, not retyped here) and tracks
barrier epochs: waves only synchronise at workgroup barriers, so an access in epoch e of one
wave can race with any access in epoch e of another.  A direct-to-LDS request issued in epoch e
is complete for everyone from epoch e+1 on only if the wave waited for it before the barrier.
Mutated schedules (a late barrier, a short counter wait, a request slot past the barrier) must
be rejected, which shows the checks have teeth."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KDIR = os.path.join(ROOT, "maize_amd", "csrc", "kernels")


class Hazard(AssertionError):
    pass


# ---------------------------------------------------------------------------------------
# macro-tile kernel: two-stage ring, 16 requests per tile per wave spread over MFMA slots
# ---------------------------------------------------------------------------------------

# how the K step numbers its MFMA slots and places the requests (16 pieces per wave and K tile with 256-row tiles, 12
# with 128-row tiles; AFTER = the slots of a step behind its barrier: 32, or 16 with 128-row tiles)
MT256_SLOT_FACTS = ("constexpr int DS = (IS8 && H128) ? (R3 ? 2 : 1) : IS8 ? 2 : H128 ? (R3 ? 4 : 3) : DMA_STRIDE;", "constexpr int AFTER = 16 * (NE - EB);",
                    "constexpr int NP = PA + 8;", "constexpr int PA = BMT / 32;",
                    "constexpr int NE = (IS8 && H128) ? 2 : (IS8 || H128) ? 4 : 8;",
                    "constexpr int EB = (IS8 && H128) ? 1 : IS8 ? 2 : H128 ? 3 : 6;",
                    "const int slot = e >= EB ? 16 * (e - EB) + s : AFTER + 16 * e + s;",
                    "if (slot >= 2 && (slot - 2) % DS == 0 && (slot - 2) / DS < NP) {",
                    # early pieces: those behind the barrier of step t itself (NST = 2 ring stages, or 3)
                    "if (DS * pc + 2 < AFTER) dma(pc, A0 + (NST - 1) * ASTR, B0 + (NST - 1) * TILE, k_begin + (NST - 1) * BKE);",
                    "k_early = k_begin + NST * BKE;", "k_late = k_begin + (NST - 1) * BKE;",
                    "if (e >= EB) dma((slot - 2) / DS, ca, cb, k_early);", "else         dma((slot - 2) / DS, na, nb, k_late);")


def mt256_issue_slots():
    """MFMA slot (counted from the barrier of step t, 128 slots per step) at which each of the 16 pieces of tile
    t + 2 is requested, as the kernel source defines it."""
    src = open(os.path.join(KDIR, "gemm_mt256.hpp")).read()
    stride = int(re.search(r"constexpr int DMA_STRIDE = (\d+);", src).group(1))
    assert "constexpr int issue_slot(int pc) { return DMA_STRIDE * pc + 2; }" in src
    for fact in MT256_SLOT_FACTS:
        assert fact in src, fact
    return [stride * pc + 2 for pc in range(16)]


# where the K step issues its fragment reads: slot s of an eighth issues reads s * RPS .. of the group the next eighth needs
MT256_READ_LINES = ("for (int rb = r * RPS; rb < (r + 1) * RPS; ++rb) {",
                    # (whole tiles: narrow == 0, nbr == NBR, nar == NAR; the K ranges of an edge tile read a subset)
                    "const int nbr = narrow == 1 ? NBR / 2 : NBR, nar = narrow == 2 ? NAR / 2 : NAR;",
                    "if (h4 == 0 && rb < NBR && narrow != 1) read_b(1, kh, cur, rb);",
                    "if (h4 == 1 && r < NAR && narrow != 2) read_a(1, kh, cur, r);",
                    "if (h4 == 2 && r < nar) { if (!last_half) read_a(0, 1, cur, r); else read_a(0, 0, cur ^ 1, r); }",
                    "if (h4 == 3 && rb < nbr) { if (!last_half) read_b(0, 1, cur, rb); else read_b(0, 0, cur ^ 1, rb); }")


def mt256_reads_per_eighth(nt):
    """A K step is 8 eighths of 16 MFMAs; each needs one new group of 4 fragments beyond what the eighth
    before it holds: 4 reads of 128 bits, or 8 transposing reads of 64 bits for a group of a row-major B.
    Within a K half the groups come in the order B1, A1, then A0 and B0 of the next half (the source states it)."""
    src = open(os.path.join(KDIR, "gemm_mt256.hpp")).read()
    assert "constexpr int NBR = TR8 ? 16 : (IS8 || !NT) ? 8 : 4;" in src and "constexpr int RPS = TR8 ? 2 : 1;" in src
    for line in MT256_READ_LINES:
        assert line in src, line
    assert "if (e == EB) {" in src
    nbr = 4 if nt else 8
    # reads that bring in eighth e (issued during e - 1): e = 0: A0 and B0 (the first of them, A0, a whole eighth earlier)
    return [nbr, nbr, 4, 0, nbr, nbr, 4, 0], nbr


def mt256_wave_program(nk, slots, nt, barrier_eighth=6):
    """Instruction stream of one wave for nk K tiles: a list of
    ("dma", tile, piece, stage) | ("wait_all",) | ("barrier",) | ("read", tile, eighth, stage) | ("mfma", tile, eighth).
    Eighth e of a step issues, in its first slots, the reads of the group that eighth e + 1 needs -- except
    that A group 0 of the next K half is read one eighth earlier (during e = 2 and e = 6), its buffer being free."""
    _, nbr = mt256_reads_per_eighth(nt)
    # (eighth whose MFMAs need it, number of reads, read from the next tile?) issued during eighth e
    issued = {0: (1, nbr, False), 1: (2, 4, False), 2: (4, 4, False), 3: (4, nbr, False),
              4: (5, nbr, False), 5: (6, 4, False), 6: (0, 4, True), 7: (0, nbr, True)}
    ops = []
    for pc in range(16):
        ops.append(("dma", 0, pc, 0))
    ops += [("wait_all",), ("barrier",)]
    ops += [("read", 0, 0, 0)] * (4 + nbr)
    early = [pc for pc in range(16) if slots[pc] < 32]
    for pc in early:
        ops.append(("dma", 1, pc, 1))
    k_early, k_late = 2, 1
    steps = nk + (nk & 1)                                   # the loop body holds two steps
    for t in range(steps):
        cur, nxt = t & 1, (t & 1) ^ 1
        for e in range(8):
            if e == barrier_eighth:
                ops += [("wait_all",), ("barrier",)]
            need, n, next_tile = issued[e]
            for s in range(16):
                ops.append(("mfma", t, e))
                if s < n:
                    ops.append(("read", t + 1, need, nxt) if next_tile else ("read", t, need, cur))
                slot = 16 * (e - 6) + s if e >= 6 else 32 + 16 * e + s
                for pc in range(16):
                    if slots[pc] == slot:
                        ops.append(("dma", k_early, pc, cur) if e >= 6 else ("dma", k_late, pc, nxt))
        k_early += 1
        k_late += 1
    ops.append(("wait_all",))
    return ops, steps


def check_two_stage(ops, steps, nreads, parts=4, pieces=16, nst=2):
    """`nreads`: fragment reads per part of a K step if a number; a list gives, per part, how many reads of the
    tile must have been issued before the part's first MFMA (cumulative).  `nst`: ring stages; with more than two a
    barrier may stand with younger requests still in flight (("wait_keep", n) waits for all but the n youngest)."""
    cumulative = [nreads * (q + 1) for q in range(parts)] if isinstance(nreads, int) else list(nreads)
    assert len(cumulative) == parts
    epoch = 0
    dma_epoch = {}          # (tile, piece) -> epoch of issue
    completed = set()       # (tile, piece) waited for by this wave
    pending = []
    visible_from = {}       # (tile, piece) -> first epoch in which every wave may read it
    last_read_epoch = {}    # tile -> epoch of its last fragment read
    stage_of = {}
    reads_seen = {}
    consumed = []
    for op in ops:
        if op[0] == "dma":
            _, tile, pc, stage = op
            if (tile, pc) in dma_epoch:
                raise Hazard(f"piece {pc} of tile {tile} requested twice")
            if stage != tile % nst:
                raise Hazard(f"tile {tile} requested into stage {stage}")
            # WAR: the stage still holds tile-nst; every wave must be past its last read of it
            old = tile - nst
            if old >= 0 and last_read_epoch.get(old, -1) >= epoch:
                raise Hazard(f"tile {tile} piece {pc} overwrites tile {old} in epoch {epoch}, still being read")
            if old >= 0 and old < steps and reads_seen.get(old, 0) < cumulative[-1]:
                raise Hazard(f"tile {tile} overwrites tile {old} before all of its fragments were read")
            dma_epoch[(tile, pc)] = epoch
            stage_of[tile] = stage
            pending.append((tile, pc))
        elif op[0] == "wait_all":
            completed.update(pending)
            pending = []
        elif op[0] == "wait_keep":
            keep = op[1]
            done = pending[:len(pending) - keep] if keep else pending
            completed.update(done)
            pending = pending[len(done):]
        elif op[0] == "barrier":
            if pending and nst == 2:
                raise Hazard("barrier with requests of this wave still in flight")
            epoch += 1
            for key in completed:
                visible_from.setdefault(key, epoch)
        elif op[0] == "read":
            _, tile, quarter, stage = op
            if stage != tile % nst:
                raise Hazard(f"tile {tile} read from stage {stage}")
            for pc in range(pieces):
                if visible_from.get((tile, pc), 1 << 30) > epoch:
                    raise Hazard(f"tile {tile} quarter {quarter} read in epoch {epoch} before piece {pc} is complete")
            last_read_epoch[tile] = epoch
            reads_seen[tile] = reads_seen.get(tile, 0) + 1
        elif op[0] == "mfma":
            _, tile, quarter = op
            if reads_seen.get(tile, 0) < cumulative[quarter]:
                raise Hazard(f"tile {tile} quarter {quarter} multiplied before its fragments were read")
            if not consumed or consumed[-1] != (tile, quarter):
                consumed.append((tile, quarter))
    if pending:
        raise Hazard("requests still in flight at the end of the K loop")
    want = [(t, q) for t in range(steps) for q in range(parts)]
    if consumed != want:
        raise Hazard("K tiles not consumed exactly once, in order")
    for t in range(steps + 1):
        got = sorted(pc for (tile, pc) in dma_epoch if tile == t)
        if t < steps and got != list(range(pieces)):
            raise Hazard(f"tile {t}: pieces requested {got}")
    return max(t for (t, _) in dma_epoch)


def mt256_cumulative_reads(nt):
    """Fragment reads of a tile that must have been issued before eighth e multiplies: per eighth the groups
    (A, B) = (0,0), (0,1), (1,1), (1,0) of K half e / 4."""
    _, nbr = mt256_reads_per_eighth(nt)
    first = 4 + nbr                       # A0, B0 of K half 0
    half = [first, first + nbr, first + nbr + 4, first + nbr + 4]
    return half + [half[3] + 4 + nbr, half[3] + 4 + 2 * nbr, half[3] + 8 + 2 * nbr, half[3] + 8 + 2 * nbr]


@pytest.mark.parametrize("nk", [1, 2, 3, 7, 64])
@pytest.mark.parametrize("nt", [False, True])
def test_macro_tile_schedule_is_hazard_free(nk, nt):
    slots = mt256_issue_slots()
    assert all(0 <= s < 96 for s in slots), "every request of tile t+2 must be issued a quarter of a step before the barrier of step t+1"
    ops, steps = mt256_wave_program(nk, slots, nt)
    last_tile = check_two_stage(ops, steps, mt256_cumulative_reads(nt), parts=8)
    # tiles past the end are requested (through a zero-length descriptor) but never multiplied
    assert steps <= last_tile <= steps + 1


def test_macro_tile_checker_rejects_broken_schedules():
    slots = mt256_issue_slots()
    need = mt256_cumulative_reads(True)
    # barrier one eighth early: fragments of the current tile are still being read behind it
    ops, steps = mt256_wave_program(8, slots, True, barrier_eighth=5)
    with pytest.raises(Hazard):
        check_two_stage(ops, steps, need, parts=8)
    # barrier one eighth late: the next tile is read before it is known to be complete
    ops, steps = mt256_wave_program(8, slots, True, barrier_eighth=7)
    with pytest.raises(Hazard):
        check_two_stage(ops, steps, need, parts=8)
    # a request scheduled past the next barrier never gets issued
    bad = list(slots)
    bad[5] = 128
    ops, steps = mt256_wave_program(8, bad, True)
    with pytest.raises(Hazard):
        check_two_stage(ops, steps, need, parts=8)
    # a missing wait before the barrier: data not guaranteed to have landed
    ops, steps = mt256_wave_program(8, slots, True)
    k = [i for i, o in enumerate(ops) if o == ("wait_all",)][3]
    with pytest.raises(Hazard):
        check_two_stage(ops[:k] + ops[k + 1:], steps, need, parts=8)
    # a fragment read dropped from an eighth: its MFMAs would run on stale registers
    ops, steps = mt256_wave_program(8, slots, True)
    k = [i for i, o in enumerate(ops) if o[0] == "read" and o[1] == 3][5]
    with pytest.raises(Hazard):
        check_two_stage(ops[:k] + ops[k + 1:], steps, need, parts=8)


# ---------------------------------------------------------------------------------------
# 128 x 256 tiles: one A group per wave.  A K step is four eighths -- per K half (A0, B0), (A0, B1) --, the second of
# each pair reads the next half's (or tile's) A0 and B0, the barrier stands in front of the last eighth, 12 pieces per
# wave and K tile, one every three MFMA slots
# ---------------------------------------------------------------------------------------

H128_READ_LINES = ("if (h4 == 0 && rb < NBR) read_b(1, kh, cur, rb);",
                   "if (h4 == 1 && r < NAR) { if (!last_half) read_a(0, 1, cur, r); else read_a(0, 0, nxt, r); }",
                   "if (h4 == 1 && rb < NBR) { if (!last_half) read_b(0, 1, cur, rb); else read_b(0, 0, nxt, rb); }",
                   "const int nxt = R3 ? (cur + 1) % 3 : cur ^ 1, lat = R3 ? (cur + 2) % 3 : cur ^ 1;",
                   "lds_ptr const ca = A0 + cur * ASTR, cb = B0 + cur * TILE, na = A0 + lat * ASTR, nb = B0 + lat * TILE, pb = B0 + nxt * TILE;",
                   "const int kh = IS8 ? 0 : H128 ? e >> 1 : e >> 2, h4 = H128 ? e & 1 : e & 3;",
                   "const int buf = H128 ? bi : bi ^ (IS8 ? st : kh);",
                   "else if (H128) lds_read128(fa[kh][r], a_rd[kh], st * (ASTR / 2048) + r);")


def h128_wave_program(nk, nt, barrier_at=3, ds=3, drop_read=None):
    src = open(os.path.join(KDIR, "gemm_mt256.hpp")).read()
    for fact in MT256_SLOT_FACTS + H128_READ_LINES:
        assert fact in src, fact
    nbr = 4 if nt else 8
    slots = [ds * pc + 2 for pc in range(12)]
    # reads issued during eighth e: (eighth that needs them, how many, from the next tile?)
    issued = {0: (1, nbr, False), 1: (2, 4 + nbr, False), 2: (3, nbr, False), 3: (0, 4 + nbr, True)}
    ops = [("dma", 0, pc, 0) for pc in range(12)]
    ops += [("wait_all",), ("barrier",)]
    ops += [("read", 0, 0, 0)] * (4 + nbr)
    ops += [("dma", 1, pc, 1) for pc in range(12) if slots[pc] < 16]
    k_early, k_late = 2, 1
    steps = nk + (nk & 1)
    nread = 0
    for t in range(steps):
        cur, nxt = t & 1, (t & 1) ^ 1
        for e in range(4):
            if e == barrier_at:
                ops += [("wait_all",), ("barrier",)]
            need, n, next_tile = issued[e]
            for sl in range(16):
                ops.append(("mfma", t, e))
                for _ in range((1 if sl < 4 else 0) + (1 if sl < nbr else 0) if n > nbr else (1 if sl < n else 0)):
                    nread += 1
                    if nread != drop_read:
                        ops.append(("read", t + 1, need, nxt) if next_tile else ("read", t, need, cur))
                slot = sl if e == 3 else 16 + 16 * e + sl
                for pc in range(12):
                    if slots[pc] == slot:
                        ops.append(("dma", k_early, pc, cur) if e == 3 else ("dma", k_late, pc, nxt))
        k_early += 1
        k_late += 1
    ops.append(("wait_all",))
    return ops, steps


def h128_cumulative_reads(nt):
    nbr = 4 if nt else 8
    return [4 + nbr, 4 + 2 * nbr, 8 + 3 * nbr, 8 + 4 * nbr]


@pytest.mark.parametrize("nk", [1, 2, 3, 7, 64])
@pytest.mark.parametrize("nt", [False, True])
def test_half_height_tile_schedule_is_hazard_free(nk, nt):
    ops, steps = h128_wave_program(nk, nt)
    last_tile = check_two_stage(ops, steps, h128_cumulative_reads(nt), parts=4, pieces=12)
    assert steps <= last_tile <= steps + 1


def test_half_height_tile_checker_rejects_broken_schedules():
    need = h128_cumulative_reads(True)
    with pytest.raises(Hazard):                 # barrier one eighth early: the tile is refilled while its last B group is still being read
        check_two_stage(*h128_wave_program(8, True, barrier_at=2), need, parts=4, pieces=12)
    with pytest.raises(Hazard):                 # requests five slots apart: the last ones would come after the next barrier
        check_two_stage(*h128_wave_program(8, True, ds=6), need, parts=4, pieces=12)
    with pytest.raises(Hazard):                 # a fragment read dropped: MFMAs on stale registers
        check_two_stage(*h128_wave_program(8, True, drop_read=30), need, parts=4, pieces=12)


# ---------------------------------------------------------------------------------------
# 128 x 256 tiles with three ring stages: the same step, but tile t+1 sits complete in the next stage, the late pieces
# issued before the barrier of step t are tile t+2's (into the stage after that one), the early pieces behind it tile
# t+3's (into the stage step t has just read), and the wait in front of the barrier leaves the twelve requests of tile
# t+2 in flight.  Two whole tiles are requested before the first step; three steps per trip
# ---------------------------------------------------------------------------------------

H128R3_LINES = ('if (R3) asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\\n\\ts_barrier" ::: "memory");',
                "for (uint32_t kt = 0; kt < nk; kt += NST) {", "if (R3) step(2);",
                "for (int pc = 0; pc < NP; ++pc) dma(pc, A1, B1, k_begin + BKE);",
                'static_assert(!R3 || NP == 12, "the counted waits of the three-stage ring assume twelve pieces per K tile");')


def h128r3_wave_program(nk, nt, barrier_at=3, ds=4, keep=12, drop_read=None):
    src = open(os.path.join(KDIR, "gemm_mt256.hpp")).read()
    for fact in MT256_SLOT_FACTS + H128_READ_LINES + H128R3_LINES:
        assert fact in src, fact
    nbr = 4 if nt else 8
    slots = [ds * pc + 2 for pc in range(12)]
    issued = {0: (1, nbr, False), 1: (2, 4 + nbr, False), 2: (3, nbr, False), 3: (0, 4 + nbr, True)}
    ops = [("dma", 0, pc, 0) for pc in range(12)] + [("dma", 1, pc, 1) for pc in range(12)]
    ops += [("wait_all",), ("barrier",)]
    ops += [("read", 0, 0, 0)] * (4 + nbr)
    ops += [("dma", 2, pc, 2) for pc in range(12) if slots[pc] < 16]
    k_early, k_late = 3, 2
    steps = 3 * ((nk + 2) // 3)
    nread = 0
    for t in range(steps):
        cur, nxt, lat = t % 3, (t + 1) % 3, (t + 2) % 3
        for e in range(4):
            if e == barrier_at:
                ops += [("wait_keep", keep), ("barrier",)]
            need, n, next_tile = issued[e]
            for sl in range(16):
                ops.append(("mfma", t, e))
                for _ in range((1 if sl < 4 else 0) + (1 if sl < nbr else 0) if n > nbr else (1 if sl < n else 0)):
                    nread += 1
                    if nread != drop_read:
                        ops.append(("read", t + 1, need, nxt) if next_tile else ("read", t, need, cur))
                slot = sl if e == 3 else 16 + 16 * e + sl
                for pc in range(12):
                    if slots[pc] == slot:
                        ops.append(("dma", k_early, pc, cur) if e == 3 else ("dma", k_late, pc, lat))
        k_early += 1
        k_late += 1
    ops.append(("wait_all",))
    return ops, steps


@pytest.mark.parametrize("nk", [1, 2, 3, 7, 28, 64])
@pytest.mark.parametrize("nt", [False, True])
def test_three_stage_schedule_is_hazard_free(nk, nt):
    ops, steps = h128r3_wave_program(nk, nt)
    last_tile = check_two_stage(ops, steps, h128_cumulative_reads(nt), parts=4, pieces=12, nst=3)
    assert steps + 1 <= last_tile <= steps + 2          # tiles past the end are requested (zero-length descriptor), never multiplied


def test_three_stage_checker_rejects_broken_schedules():
    need = h128_cumulative_reads(True)
    with pytest.raises(Hazard):                 # a wait that leaves one request more in flight: the next tile's last piece may not have landed
        check_two_stage(*h128r3_wave_program(9, True, keep=13), need, parts=4, pieces=12, nst=3)
    with pytest.raises(Hazard):                 # barrier one eighth early: the stage is refilled while its last B group is still being read
        check_two_stage(*h128r3_wave_program(9, True, barrier_at=2), need, parts=4, pieces=12, nst=3)
    with pytest.raises(Hazard):                 # requests six slots apart: the last ones are never issued
        check_two_stage(*h128r3_wave_program(9, True, ds=6), need, parts=4, pieces=12, nst=3)
    with pytest.raises(Hazard):                 # a fragment read dropped: MFMAs on stale registers
        check_two_stage(*h128r3_wave_program(9, True, drop_read=30), need, parts=4, pieces=12, nst=3)


# ---------------------------------------------------------------------------------------
# 128 x 128 tiles (gemm_t128.hpp): four ring stages, eight pieces per wave and K tile.  A K step is two K halves of 16
# MFMAs: K half 1's reads, K half 0's MFMAs with the pieces of tile t + 3 behind every second one, the wait that keeps
# sixteen requests in flight, the barrier, K half 0's reads of tile t + 1, K half 1's MFMAs
# ---------------------------------------------------------------------------------------
T128_LINES = ("request(0u, 0u);", "request(BKE, 1u);", "request(2u * BKE, 2u);",
              'asm volatile("s_waitcnt vmcnt(16)\\n\\ts_barrier" ::: "memory");\n    if constexpr (!IS8) {\n    read_half(0, 0u);',
              "const uint32_t so = (kt & 3u) * STAGE, so_next = ((kt + 1u) & 3u) * STAGE;\n        asm volatile(\"s_waitcnt lgkmcnt(0)\");",
              "const TileReq r = tile_req((kt + 3u) * BKE, (kt + 3u) & 3u);\n#pragma unroll\n        for (int i = 0; i < 4; ++i)",
              "constexpr int HALF_READS = NT ? 8 : 12, PER_SLOT = NT ? 1 : 2;",
              "for (int q = (4 * i + j) * PER_SLOT; q < (4 * i + j + 1) * PER_SLOT; ++q)\n                    if (q < HALF_READS) read_one(1, so, q);",
              "if (j & 1) {\n                    piece(r, (4 * i + j) >> 1);",
              'asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\\n\\ts_barrier" ::: "memory");\n#pragma unroll\n        for (int i = 0; i < 4; ++i)',
              "if (q < HALF_READS) read_one(0, so_next, q);",
              "for (int q = 0; q < 8; ++q) piece(r, q);")
# ... on 8-bit operands: a step splits by accumulator rows -- rows 0-1 need A fragments 0, 1 and all of B (12 reads, two behind
# each of the first six MFMAs of the half step before), rows 2-3 A fragments 2, 3 (4 reads, one behind each of the first four
# MFMAs of rows 0-1); one request behind each of rows 0-1's eight MFMAs; two steps per trip, the count rounded up to an even
# number with a tile past K
T128_F8_LINES = ("constexpr int NEXT_READS = TR8 ? 20 : 12, NEXT_PER_SLOT = TR8 ? 3 : 2;",
                 "for (int q = 0; q < NEXT_READS; ++q) read_next(std::integral_constant<int, 0>{}, 0u, q);",
                 "asm volatile(\"s_waitcnt lgkmcnt(0)\");\n            const TileReq r = tile_req((kt + 3u) * BKE, (kt + 3u) & 3u);",
                 "mfma8(acc[i][j], set, j, a8[i]);",
                 "if (4 * i + j < 4) rd128(a8[2 + (4 * i + j) / 2][(4 * i + j) & 1], a_rd[(4 * i + j) & 1] + so, 2 + (4 * i + j) / 2);\n                    piece(r, 4 * i + j);",
                 'asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\\n\\ts_barrier" ::: "memory");\n#pragma unroll\n            for (int i = 2; i < 4; ++i)',
                 "for (int q = NEXT_PER_SLOT * (4 * (i - 2) + j); q < NEXT_PER_SLOT * (4 * (i - 2) + j + 1); ++q)\n                        if (q < NEXT_READS) read_next(std::integral_constant<int, 1 - S>{}, so_next, q);",
                 "for (uint32_t kt = 0; kt < nk; kt += 2u) {\n            step8(std::integral_constant<int, 0>{}, kt);\n            step8(std::integral_constant<int, 1>{}, kt + 1u);")


def t128_f8_wave_program(nk, keep=16, reads_before_barrier=False, late_rows=4, tr=False):
    """tr: B stored K x N -- a fragment of B is four transposing reads, the next tile's reads are 20, three behind an MFMA."""
    src = open(os.path.join(KDIR, "gemm_t128.hpp")).read()
    for fact in T128_LINES + T128_F8_LINES:
        assert fact in src, fact
    nxt, per = (20, 3) if tr else (12, 2)
    steps = nk + (nk & 1)
    ops = [("dma", t, pc, t % 4) for t in range(3) for pc in range(8)]
    ops += [("wait_keep", keep), ("barrier",)]
    ops += [("read", 0, 0, 0)] * nxt
    for t in range(steps):
        for m in range(8):
            ops.append(("mfma", t, 0))
            if m < late_rows:
                ops.append(("read", t, 1, t % 4))
            ops.append(("dma", t + 3, m, (t + 3) % 4))
        if reads_before_barrier:
            ops += [("read", t + 1, 0, (t + 1) % 4)] * nxt
        ops += [("wait_keep", keep), ("barrier",)]
        for m in range(8):
            ops.append(("mfma", t, 1))
            if not reads_before_barrier:
                ops += [("read", t + 1, 0, (t + 1) % 4)] * max(0, min(per, nxt - per * m))
    ops.append(("wait_all",))
    return ops, steps


@pytest.mark.parametrize("tr", [False, True])
@pytest.mark.parametrize("nk", [1, 2, 3, 4, 5, 8, 33])
def test_tiles_of_128_by_128_8bit_schedule_is_hazard_free(nk, tr):
    ops, steps = t128_f8_wave_program(nk, tr=tr)
    first = 20 if tr else 12
    assert check_two_stage(ops, steps, [first, first + 4], parts=2, pieces=8, nst=4) == steps + 2


def test_tiles_of_128_by_128_8bit_checker_rejects_broken_schedules():
    with pytest.raises(Hazard):                 # a wait that leaves one request more in flight
        check_two_stage(*t128_f8_wave_program(9, keep=17), [12, 16], parts=2, pieces=8, nst=4)
    with pytest.raises(Hazard):                 # the next tile read in front of the barrier
        check_two_stage(*t128_f8_wave_program(9, reads_before_barrier=True), [12, 16], parts=2, pieces=8, nst=4)
    with pytest.raises(Hazard):                 # A fragment 3's reads dropped: rows 2-3 multiply stale registers
        check_two_stage(*t128_f8_wave_program(9, late_rows=2), [12, 16], parts=2, pieces=8, nst=4)


def t128_wave_program(nk, nt, keep=16, primed=3, ahead=3, reads_before_barrier=False, stages=4):
    src = open(os.path.join(KDIR, "gemm_t128.hpp")).read()
    for fact in T128_LINES:
        assert fact in src, fact
    assert int(re.search(r"constexpr int BT = 128, BK = 64, NS = (\d+);", src).group(1)) == 4
    half = 8 if nt else 12                        # LDS reads of one K half: 4 of A + 4 of B, or 8 transposing ones
    per_slot = 1 if nt else 2                     # ... one (two) behind each of the other half's first MFMAs
    ops = [("dma", t, pc, t % stages) for t in range(primed) for pc in range(8)]
    ops += [("wait_keep", keep), ("barrier",)]
    ops += [("read", 0, 0, 0)] * half
    for t in range(nk):
        for m in range(16):
            ops.append(("mfma", t, 0))
            ops += [("read", t, 1, t % stages)] * (per_slot if m * per_slot < half else 0)
            if m & 1:
                ops.append(("dma", t + ahead, m >> 1, (t + ahead) % stages))
        if reads_before_barrier:
            ops += [("read", t + 1, 0, (t + 1) % stages)] * half
        ops += [("wait_keep", keep), ("barrier",)]
        for m in range(16):
            ops.append(("mfma", t, 1))
            if not reads_before_barrier:
                ops += [("read", t + 1, 0, (t + 1) % stages)] * (per_slot if m * per_slot < half else 0)
    ops.append(("wait_all",))
    return ops, nk


@pytest.mark.parametrize("nk", [1, 2, 3, 4, 5, 7, 64])
@pytest.mark.parametrize("nt", [False, True])
def test_tiles_of_128_by_128_schedule_is_hazard_free(nk, nt):
    ops, steps = t128_wave_program(nk, nt)
    half = 8 if nt else 12
    last_tile = check_two_stage(ops, steps, [half, 2 * half], parts=2, pieces=8, nst=4)
    assert last_tile == steps + 2                       # tiles past the end are requested (zero-length descriptor) and read, never multiplied


def test_tiles_of_128_by_128_checker_rejects_broken_schedules():
    need = [8, 16]
    with pytest.raises(Hazard):                 # a wait that leaves one request more in flight: the next tile's last piece may not have landed
        check_two_stage(*t128_wave_program(9, True, keep=17), need, parts=2, pieces=8, nst=4)
    with pytest.raises(Hazard):                 # the next tile read in front of the barrier: another wave's pieces may not have landed
        check_two_stage(*t128_wave_program(9, True, reads_before_barrier=True), need, parts=2, pieces=8, nst=4)
    with pytest.raises(Hazard):                 # a tile requested four steps ahead goes into the stage that is being read
        check_two_stage(*t128_wave_program(9, True, ahead=4, primed=4, keep=24), need, parts=2, pieces=8, nst=4)
    with pytest.raises(Hazard):                 # a ring primed with two tiles: the same wait no longer covers tile t + 1
        check_two_stage(*t128_wave_program(9, True, primed=2, ahead=2), need, parts=2, pieces=8, nst=4)


# ---------------------------------------------------------------------------------------
# 128 x 256 tiles on 8-bit operands: a K tile is one matrix instruction deep, so a K step is the pair (A0, B0), (A0, B1)
# with the barrier between the two; the second eighth reads the next tile's A0 (8 reads) and B0 (8, or 16 transposing
# ones, two per slot); 12 pieces per wave and K tile, one per MFMA slot behind the barrier
# ---------------------------------------------------------------------------------------

def h128_f8_wave_program(nk, tr, barrier_at=1, ds=1, nst=2, keep=12):
    """nst = 3: the three-stage ring (two whole tiles requested in front, tile t+3 behind the barrier of step t, the wait
    leaves the `keep` youngest requests in flight)."""
    src = open(os.path.join(KDIR, "gemm_mt256.hpp")).read()
    for fact in MT256_SLOT_FACTS + H128_READ_LINES + H128R3_LINES + ("if (IS8 && H128) lds_read128(fa8[st][r >> 1][r & 1], a_rd[r & 1], st * (ASTR / 2048) + (r >> 1));",
                                                                     "u32x4 fa8[NST][4][2], fb8[2][4][2];", '"v"(operand8(fa8[H128 ? cur : ai][r4]))'):
        assert fact in src, fact
    nbr, per_slot = (16, 2) if tr else (8, 1)
    slots = [ds * pc + 2 for pc in range(12)]
    ops = [("dma", t, pc, t) for t in range(nst - 1) for pc in range(12)]
    ops += [("wait_all",), ("barrier",)]
    ops += [("read", 0, 0, 0)] * (8 + nbr)
    ops += [("dma", nst - 1, pc, nst - 1) for pc in range(12) if slots[pc] < 16]
    k_early, k_late = nst, nst - 1
    steps = nst * ((nk + nst - 1) // nst)
    for t in range(steps):
        cur, nxt, lat = t % nst, (t + 1) % nst, (t + nst - 1) % nst
        for e in range(2):
            if e == barrier_at:
                ops += [("wait_all",) if nst == 2 else ("wait_keep", keep), ("barrier",)]
            for sl in range(16):
                ops.append(("mfma", t, e))
                if e == 0:                                   # B group 1 of this tile
                    ops += [("read", t, 1, cur)] * (per_slot if sl * per_slot < nbr else 0)
                else:                                        # A group 0 and B group 0 of the next tile
                    ops += [("read", t + 1, 0, nxt)] * ((1 if sl < 8 else 0) + (per_slot if sl * per_slot < nbr else 0))
                slot = sl if e == 1 else 16 + sl
                for pc in range(12):
                    if slots[pc] == slot:
                        ops.append(("dma", k_early, pc, cur) if e == 1 else ("dma", k_late, pc, lat))
        k_early += 1
        k_late += 1
    ops.append(("wait_all",))
    return ops, steps


@pytest.mark.parametrize("tr", [False, True])
@pytest.mark.parametrize("nk", [1, 2, 3, 7, 32])
def test_8bit_half_height_tile_schedule_is_hazard_free(nk, tr):
    nbr = 16 if tr else 8
    ops, steps = h128_f8_wave_program(nk, tr)
    last_tile = check_two_stage(ops, steps, [8 + nbr, 8 + 2 * nbr], parts=2, pieces=12)
    assert steps <= last_tile <= steps + 1
    ops, steps = h128_f8_wave_program(nk, tr, nst=3, ds=2)
    last_tile = check_two_stage(ops, steps, [8 + nbr, 8 + 2 * nbr], parts=2, pieces=12, nst=3)
    assert steps + 1 <= last_tile <= steps + 2


def test_8bit_half_height_tile_checker_rejects_broken_schedules():
    with pytest.raises(Hazard):                 # no barrier between the two eighths: the next tile is read before it is known to be complete
        check_two_stage(*h128_f8_wave_program(8, False, barrier_at=2), [16, 24], parts=2, pieces=12)
    with pytest.raises(Hazard):                 # barrier in front of the first eighth: the stage is refilled while B group 1 is still being read
        check_two_stage(*h128_f8_wave_program(8, False, barrier_at=0), [16, 24], parts=2, pieces=12)
    with pytest.raises(Hazard):                 # requests three slots apart: the last ones would never be issued
        check_two_stage(*h128_f8_wave_program(8, False, ds=3), [16, 24], parts=2, pieces=12)
    with pytest.raises(Hazard):                 # three stages, a wait that leaves thirteen requests in flight
        check_two_stage(*h128_f8_wave_program(9, False, nst=3, ds=2, keep=13), [16, 24], parts=2, pieces=12, nst=3)
    with pytest.raises(Hazard):                 # three stages, barrier in front of the first eighth
        check_two_stage(*h128_f8_wave_program(9, False, nst=3, ds=2, barrier_at=0), [16, 24], parts=2, pieces=12, nst=3)
    with pytest.raises(Hazard):                 # three stages, requests three slots apart: the last two would never be issued
        check_two_stage(*h128_f8_wave_program(9, False, nst=3, ds=3), [16, 24], parts=2, pieces=12, nst=3)


# ---------------------------------------------------------------------------------------
# 8-bit macro-tile kernel: the same template with a K tile one matrix instruction deep: a K step is four groups of
# 16 MFMAs, the barrier in front of the third, a group is 8 reads, one request per two MFMA slots.  With a row-major
# B (transposing reads) a B group is 16 reads, two per MFMA slot.
# ---------------------------------------------------------------------------------------

def f8_constants():
    src = open(os.path.join(KDIR, "gemm_mt256.hpp")).read()
    for fact in MT256_SLOT_FACTS + ("constexpr int NAR = IS8 ? 8 : 4;", "const bool last_half = IS8 || kh == 1;",
                 "constexpr int NBR = TR8 ? 16 : (IS8 || !NT) ? 8 : 4;", "constexpr int RPS = TR8 ? 2 : 1;",
                 "constexpr bool TR8 = IS8 && !NT;") + MT256_READ_LINES:
        assert fact in src, fact
    return dict(ne=4, eb=2, ds=2, reads=8)


def f8_wave_program(nk, barrier_at=None, ds=None, tr=False):
    """tr: row-major B.  The groups read during group e of a step: B1, A1, then A0 and B0 of the next tile."""
    c = f8_constants()
    b_reads = 16 if tr else c["reads"]
    per_group = [b_reads, c["reads"], c["reads"], b_reads]
    eb = c["eb"] if barrier_at is None else barrier_at
    ds = c["ds"] if ds is None else ds
    slots = [ds * pc + 2 for pc in range(16)]
    # reads issued during group e: (group whose MFMAs need them, from the next tile?)
    issued = {0: (1, False), 1: (2, False), 2: (0, True), 3: (0, True)}
    ops = [("dma", 0, pc, 0) for pc in range(16)]
    ops += [("wait_all",), ("barrier",)]
    ops += [("read", 0, 0, 0)] * (c["reads"] + b_reads)
    ops += [("dma", 1, pc, 1) for pc in range(16) if slots[pc] < 32]
    k_early, k_late = 2, 1
    steps = nk + (nk & 1)
    for t in range(steps):
        cur, nxt = t & 1, (t & 1) ^ 1
        for e in range(c["ne"]):
            if e == eb:
                ops += [("wait_all",), ("barrier",)]
            need, next_tile = issued[e]
            for sl in range(16):
                ops.append(("mfma", t, e))
                if sl < 8:                                  # all of a group's reads in the first half of the group before
                    for _ in range(per_group[e] // 8):
                        ops.append(("read", t + 1, need, nxt) if next_tile else ("read", t, need, cur))
                slot = 16 * (e - c["eb"]) + sl if e >= c["eb"] else 32 + 16 * e + sl
                for pc in range(16):
                    if slots[pc] == slot:
                        ops.append(("dma", k_early, pc, cur) if e >= c["eb"] else ("dma", k_late, pc, nxt))
        k_early += 1
        k_late += 1
    ops.append(("wait_all",))
    return ops, steps


F8_CUMULATIVE = [16, 24, 32, 32]      # reads of a tile that must have been issued before group e multiplies: A0 B0 | B1 | A1 | -
F8_CUMULATIVE_TR = [24, 40, 48, 48]   # ... with 16 reads per B group


@pytest.mark.parametrize("tr", [False, True])
@pytest.mark.parametrize("nk", [1, 2, 3, 7, 32])
def test_8bit_macro_tile_schedule_is_hazard_free(nk, tr):
    ops, steps = f8_wave_program(nk, tr=tr)
    last_tile = check_two_stage(ops, steps, F8_CUMULATIVE_TR if tr else F8_CUMULATIVE, parts=4)
    assert steps <= last_tile <= steps + 1


def test_8bit_macro_tile_checker_rejects_broken_schedules():
    with pytest.raises(Hazard):                 # barrier one group late: the next tile is read before it is known to be complete
        check_two_stage(*f8_wave_program(8, barrier_at=3), F8_CUMULATIVE, parts=4)
    with pytest.raises(Hazard):                 # barrier one group early: the stage is refilled while its last group is still being read
        check_two_stage(*f8_wave_program(8, barrier_at=1), F8_CUMULATIVE, parts=4)
    with pytest.raises(Hazard):                 # requests four slots apart: the last ones would come after the next barrier and never be issued
        check_two_stage(*f8_wave_program(8, ds=5), F8_CUMULATIVE, parts=4)
    for kw in (dict(barrier_at=3), dict(barrier_at=1)):
        with pytest.raises(Hazard):             # the same with a row-major B
            check_two_stage(*f8_wave_program(8, tr=True, **kw), F8_CUMULATIVE_TR, parts=4)
    with pytest.raises(Hazard):                 # 8 reads per B group where a row-major B needs 16: MFMAs on stale registers
        check_two_stage(*f8_wave_program(8), F8_CUMULATIVE_TR, parts=4)


# ---------------------------------------------------------------------------------------
# skinny kernels (1, 2 or 4 groups of 16 rows): 8-slot ring, per wave 2 pieces per block plus the A blocks it has the
# duty for (row group r of the block in slot x is fetched by wave (x + r) % 8), counter wait instead of wait-all
# ---------------------------------------------------------------------------------------

def skinny_constants():
    src = open(os.path.join(KDIR, "gemm_skinny.hpp")).read()
    ring = int(re.search(r"constexpr int RING = (\d+);", src).group(1))
    waits = [int(x) for x in re.findall(r"s_waitcnt vmcnt\((\d+)\)\\n\\ts_barrier", src)]
    # one row group: two waits, with and without an A block among the loads that may stay in flight; more row
    # groups: 12 pieces plus 0 .. 4 A blocks, picked by a count
    assert waits[:2] == [12, 13] and waits[2:] == [12, 13, 14, 15, 16]
    # the duty rule and the rule that picks the wait, as written in the kernel
    assert "if (wave == (uint32_t)((ai + r) & 7))" in src
    assert re.search(r"if \(wave == \(uint32_t\)ai \|\| wave == \(uint32_t\)pi\) asm volatile\(\"s_waitcnt vmcnt\(12\)", src)
    assert "later += (((wave - (uint32_t)r - (uint32_t)ai) & 7u) - 1u) < 6u ? 1u : 0u;" in src
    for n in range(5):
        assert re.search(r"(case %d|default): asm volatile\(\"s_waitcnt vmcnt\(%d\)" % (n, 12 + n), src)
    primed = len(re.findall(r"request\(\d+, s\d+, \d+\);", src))
    return ring, (12, 13), primed


def skinny_wait(wave, cur, refill, waits, mr):
    """The counter value a wave waits for before block `cur`'s barrier, as the kernel picks it."""
    if mr == 1:
        return waits[0] if wave in (cur, refill) else waits[1]
    return 12 + sum(1 for r in range(mr) if 0 <= ((wave - r - cur) & 7) - 1 < 6)


def skinny_wave_program(nb, ring, waits, primed, wave=0, mr=1):
    """The program of one wave: ("request", block, slot, loads), ("wait", n), ("barrier",), ("consume", block, slot)."""
    loads = lambda slot: 2 + sum(1 for r in range(mr) if (slot + r) % 8 == wave)
    ops = []
    for j in range(primed):
        ops.append(("request", j, j % ring, loads(j % ring)))
    turns = -(-nb // ring) * ring
    for b in range(turns):
        cur, refill = b % ring, (b + primed) % ring
        ops += [("wait", skinny_wait(wave, cur, refill, waits, mr)), ("barrier",)]
        ops.append(("request", b + primed, refill, loads(refill)))
        ops.append(("consume", b, cur))
    ops.append(("wait", 0))
    return ops, turns, None


def check_ring(ops, turns, loads_per_request, ring):
    epoch = 0
    issued = []                 # blocks in request order
    loads = []                  # one entry per load, in issue order: the block it belongs to
    done = 0                    # number of loads known complete for this wave (the counter retires them in order)
    visible_from = {}
    consumed_epoch = {}
    slot_holds = {}
    consumed = []
    for op in ops:
        if op[0] == "request":
            _, blk, slot = op[:3]
            old = slot_holds.get(slot)
            if old is not None:
                if old not in consumed_epoch:
                    raise Hazard(f"block {blk} overwrites block {old}, never consumed")
                if consumed_epoch[old] >= epoch:
                    raise Hazard(f"block {blk} overwrites block {old} in the epoch it is read in")
            slot_holds[slot] = blk
            issued.append(blk)
            loads += [blk] * (op[3] if len(op) > 3 else loads_per_request)
        elif op[0] == "wait":
            # the counter retires loads in order: at most op[1] of the newest may be outstanding
            done = max(done, len(loads) - op[1])
        elif op[0] == "barrier":
            epoch += 1
            pending = set(loads[done:])
            for blk in issued:
                if blk not in pending:
                    visible_from.setdefault(blk, epoch)
        elif op[0] == "consume":
            _, blk, slot = op
            if slot_holds.get(slot) != blk:
                raise Hazard(f"block {blk} expected in slot {slot}, which holds {slot_holds.get(slot)}")
            if visible_from.get(blk, 1 << 30) > epoch:
                raise Hazard(f"block {blk} consumed in epoch {epoch} before every wave's share has landed")
            consumed_epoch[blk] = epoch
            consumed.append(blk)
    if done != len(loads):
        raise Hazard("loads still in flight at the end")
    if consumed != list(range(turns)):
        raise Hazard("blocks not consumed exactly once, in order")
    if sorted(issued) != list(range(len(issued))):
        raise Hazard("blocks not requested exactly once")


@pytest.mark.parametrize("mr", [1, 2, 4])
@pytest.mark.parametrize("nb", [8, 16, 32, 128, 9])
def test_skinny_ring_is_hazard_free(nb, mr):
    ring, waits, primed = skinny_constants()
    assert primed == ring - 1
    for wave in range(8):
        ops, turns, lpr = skinny_wave_program(nb, ring, waits, primed, wave, mr)
        check_ring(ops, turns, lpr, ring)
        # every wait is exact: it leaves just the loads issued after the current block's in flight
        issued = []
        for op in ops:
            if op[0] == "request":
                issued += [op[1]] * op[3]
            elif op[0] == "consume":
                # loads of later blocks, except this turn's refill (block op[1] + primed), which is issued after the wait
                newer = sum(1 for blk in issued if op[1] < blk < op[1] + primed)
                assert last_wait == newer, (wave, op, last_wait, newer)
            elif op[0] == "wait":
                last_wait = op[1]


def test_skinny_checker_rejects_broken_rings():
    ring, waits, primed = skinny_constants()
    for wave in (0, 3, 7):
        ops, turns, lpr = skinny_wave_program(32, ring, (waits[0] + 1, waits[1] + 1), primed, wave)   # waits for one load too few
        with pytest.raises(Hazard):
            check_ring(ops, turns, lpr, ring)
        ops, turns, lpr = skinny_wave_program(32, ring, (waits[1], waits[1]), primed, wave)           # ignores where the duty falls
        with pytest.raises(Hazard):
            check_ring(ops, turns, lpr, ring)
        for mr in (2, 4):               # more row groups: the wait of the one-group kernel leaves an A block unaccounted for
            ops, turns, lpr = skinny_wave_program(32, ring, waits, primed, wave, mr)
            lax = [("wait", o[1] + 1) if o[0] == "wait" and o[1] else o for o in ops]
            with pytest.raises(Hazard):
                check_ring(lax, turns, lpr, ring)
    ops, turns, lpr = skinny_wave_program(32, ring - 1, waits, primed)       # ring one slot short: refill hits the block being read
    with pytest.raises(Hazard):
        check_ring(ops, turns, lpr, ring - 1)
    ops, turns, lpr = skinny_wave_program(32, ring, waits, primed)
    swapped = [o for o in ops]
    i = next(k for k, o in enumerate(swapped) if o[0] == "barrier")
    del swapped[i]                                                         # first barrier missing
    with pytest.raises(Hazard):
        check_ring(swapped, turns, lpr, ring)


# ---------------------------------------------------------------------------------------
# skinny NT kernel: 4-slot ring private to each wave (it fetches, reads and multiplies only its own 32
# rows -- tests/cpu/check_maps.cpp proves that from the index maps), 6 loads per block, no barrier
# ---------------------------------------------------------------------------------------

def skinny_nt_constants():
    src = open(os.path.join(KDIR, "gemm_skinny_nt.hpp")).read()
    ring = int(re.search(r"constexpr int RING = (\d+);", src).group(1))
    src = src[:src.index("void body_rows(")]               # the one-group kernel; the row-group kernel is modelled below
    body = src[src.index("auto turn = "):]
    waits = [int(x) for x in re.findall(r's_waitcnt vmcnt\((\d+)\)" ::: "memory"\);\n\s+__builtin_amdgcn_sched_barrier', body)]
    assert len(waits) == 1 and "s_barrier" not in body[:body.index("request(0, s0, 0)")]
    ahead = int(re.search(r"request\(b \+ (\d+), prev, pi\);", src).group(1))
    primed = len(re.findall(r"request\(\d+, s\d+, \d+\);", src))
    return ring, waits[0], primed, ahead


def skinny_nt_wave_program(nb, ring, wait, primed, ahead):
    ops = [("request", j, j % ring) for j in range(primed)]
    turns = -(-nb // ring) * ring
    for b in range(turns):
        ops.append(("wait", wait))
        ops.append(("request", b + ahead, (b + ahead) % ring))
        ops.append(("consume", b, b % ring))
    ops.append(("wait", 0))
    return ops, turns


def check_private_ring(ops, turns, loads_per_request):
    issued, done, slot_holds, consumed = [], 0, {}, []
    for op in ops:
        if op[0] == "request":
            _, blk, slot = op[:3]
            old = slot_holds.get(slot)
            if old is not None and old not in consumed:         # program order of one wave: its reads of `old` are behind it
                raise Hazard(f"block {blk} overwrites block {old} before it is consumed")
            slot_holds[slot] = blk
            issued.append(blk)
        elif op[0] == "wait":
            done = max(done, len(issued) - -(-op[1] // loads_per_request))
        elif op[0] == "consume":
            _, blk, slot = op
            if slot_holds.get(slot) != blk:
                raise Hazard(f"block {blk} expected in slot {slot}, which holds {slot_holds.get(slot)}")
            if blk not in issued[:done]:
                raise Hazard(f"block {blk} consumed before its loads have landed")
            consumed.append(blk)
    if done != len(issued):
        raise Hazard("loads still in flight at the end")
    if consumed != list(range(turns)) or sorted(issued) != list(range(len(issued))):
        raise Hazard("blocks not requested once and consumed once, in order")


@pytest.mark.parametrize("nb", [4, 16, 32, 128, 9, 1])
def test_skinny_nt_ring_is_hazard_free(nb):
    ring, wait, primed, ahead = skinny_nt_constants()
    assert primed == ring - 1 == ahead
    ops, turns = skinny_nt_wave_program(nb, ring, wait, primed, ahead)
    check_private_ring(ops, turns, 6)
    assert wait == 6 * (primed - 1)                              # exactly the blocks behind the current one stay in flight


def test_skinny_nt_checker_rejects_broken_rings():
    ring, wait, primed, ahead = skinny_nt_constants()
    with pytest.raises(Hazard):                                  # waits for one request too few
        check_private_ring(*skinny_nt_wave_program(32, ring, wait + 6, primed, ahead), 6)
    with pytest.raises(Hazard):                                  # refill aimed at the slot that is about to be read
        check_private_ring(*skinny_nt_wave_program(32, ring - 1, wait, primed, ahead), 6)


# ---------------------------------------------------------------------------------------
# skinny NT kernels with 2 or 4 row groups: the ring is shared again (A blocks through LDS): 4 slots, per wave 4 pieces
# of B per block plus the A pieces it has the duty for (piece i of the block in slot x: wave (x + i) % 8), one barrier
# per block, counter wait
# ---------------------------------------------------------------------------------------

def skinny_nt_rows_constants():
    src = open(os.path.join(KDIR, "gemm_skinny_nt.hpp")).read()
    src = src[src.index("void body_rows("):]
    waits = [int(x) for x in re.findall(r"s_waitcnt vmcnt\((\d+)\)\\n\\ts_barrier", src)]
    assert waits == [8, 9, 10]
    assert "if (wave == (uint32_t)((ai + i) & 7))" in src                                   # the duty rule
    assert "later += wave == (uint32_t)((((ai + x) % RING) + i) & 7) ? 1u : 0u;" in src and "for (int x = 1; x <= 2; ++x)" in src
    for n in range(3):
        assert re.search(r"(case %d|default): asm volatile\(\"s_waitcnt vmcnt\(%d\)" % (n, 8 + n), src)
    ahead = int(re.search(r"request\(b \+ (\d+), prev, pi\);", src).group(1))
    primed = len(re.findall(r"request\(\d+, s\d+, \d+\);", src))
    return 4, primed, ahead


def skinny_nt_rows_program(nb, ring, primed, ahead, wave, mr, slack=0):
    loads = lambda slot: 4 + sum(1 for i in range(2 * mr) if (slot + i) % 8 == wave)
    ops = [("request", j, j % ring, loads(j % ring)) for j in range(primed)]
    turns = -(-nb // ring) * ring
    for b in range(turns):
        cur = b % ring
        later = sum(1 for x in (1, 2) for i in range(2 * mr) if ((cur + x) % ring + i) % 8 == wave)
        ops += [("wait", 8 + later + slack), ("barrier",)]
        ops.append(("request", b + ahead, (b + ahead) % ring, loads((b + ahead) % ring)))
        ops.append(("consume", b, cur))
    ops.append(("wait", 0))
    return ops, turns


@pytest.mark.parametrize("mr", [2, 4])
@pytest.mark.parametrize("nb", [4, 16, 32, 9, 1])
def test_skinny_nt_row_group_ring_is_hazard_free(nb, mr):
    ring, primed, ahead = skinny_nt_rows_constants()
    assert primed == ring - 1 == ahead
    for wave in range(8):
        ops, turns = skinny_nt_rows_program(nb, ring, primed, ahead, wave, mr)
        check_ring(ops, turns, None, ring)
        with pytest.raises(Hazard):                              # one load more left in flight: block b's last piece may be missing
            check_ring(*skinny_nt_rows_program(32, ring, primed, ahead, wave, mr, slack=1), None, ring)
