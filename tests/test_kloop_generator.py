"""The generated K loop (maize_amd/csrc/kernels/gen_kloop.py) replayed instruction by instruction on the CPU: every matrix
instruction multiplies the fragments it is meant to, no fragment is used before the wait that follows its read, the ring
stages are read and refilled on the right side of the barrier, and every request and deferred store is issued exactly
once.  (That the loop gives the statement loop's bits is the GPU test's business: test_gpu_asm_kloop.py.)"""
import importlib.util
import os
import re

import pytest

GEN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "maize_amd", "csrc", "kernels", "gen_kloop.py")


def load_generator(drain_steps=0):
    spec = importlib.util.spec_from_file_location(f"gen_kloop_{drain_steps}", GEN)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.DRAIN_STEPS = drain_steps
    mod.COMPACT = drain_steps > 0
    mod.NO_STORE = False
    return mod


def quad(text):
    lo, hi = re.fullmatch(r"v\[(\d+):(\d+)\]", text).groups()
    return int(lo), int(hi) - int(lo) + 1


class Replay:
    """One wave's view.  Fragment registers carry a tag (operand, stage, group, K half, row / column, [half]) from the read
    that filled them, and the index of that read until a wait on the LDS counter has passed."""

    def __init__(self, gen, nt):
        self.gen, self.nt = gen, nt
        self.tag, self.unwaited = {}, set()
        self.mfma_of, self.requests, self.stores = {}, [], []
        self.tail_mfma, self.tail_requests = {}, []
        self.mtail_form = False
        self.since_barrier_reads = set()       # stages read since the last barrier
        self.outstanding = []                  # vector-memory operations in issue order ("load", stage) / ("store", quad)

    def run(self, lines, stage_of_step):
        step = -1
        for ln in lines:
            op = ln.split()[0]
            if op == "ds_read_b128" and ("a_rdt" in ln or "b_rdt" in ln or "t_rd" in ln):
                # the block against the ragged columns: its A fragment from A's stage, its B fragment (N x K) from the stages of its own
                dst, addr, off = re.match(r"ds_read_b128 (\S+), %\[(\w+)\] offset:(\d+)", ln).groups()
                base, _ = quad(dst)
                stride = 2048 if addr.startswith("t_rd") else 32768         # the block's own tile, or a fragment of the whole tile's stage
                st = int(off) // stride
                assert int(off) % stride == 0
                # which operand the registers feed is told by where they sit: the A fragment's or the B fragment's
                side = "ta" if base == self.gen.FT_A else "tb"
                assert base in (self.gen.FT_A, self.gen.FT_B)
                assert addr.startswith("t_rd") == ((side == "tb") != self.mtail_form), f"{ln}: fragment from the wrong place"
                for k in range(4):
                    self.tag[base + k] = (side, st, 0, int(addr[-1]), 0, k)
                    self.unwaited.add(base + k)
            elif op == "ds_read_b64_tr_b16" and ("t_rd" in ln or "b_rdt" in ln):
                dst, addr, off = re.match(r"ds_read_b64_tr_b16 (\S+), %\[(t_rd0|b_rdt0)\] offset:(\d+)", ln).groups()
                base, n = quad(dst)
                if addr == "t_rd0":      # the ragged columns' own K x N tile: 32 bytes per row
                    st, kh, h = int(off) // 2048, (int(off) % 2048) // 1024, (int(off) % 1024) // 128
                    assert int(off) % 128 == 0 and not self.mtail_form
                else:                    # a column block of B's stage (ragged rows)
                    st, kh, h = int(off) // 32768, (int(off) % 32768) // 16384, (int(off) % 16384) // 2048
                    assert int(off) % 2048 == 0 and self.mtail_form
                assert n == 2 and h < 2
                for k in range(2):
                    self.tag[base + k] = ("tb", st, 0, kh, 0, 2 * h + k)
                    self.unwaited.add(base + k)
            elif op == "ds_read_b128":
                dst, addr, off = re.match(r"ds_read_b128 (\S+), %\[(\w+)\] offset:(\d+)", ln).groups()
                base, _ = quad(dst)
                slot = int(off) // 2048
                st, grp, r = slot // 16, (slot % 16) // 4, slot % 4
                kh = int(addr[-1])
                for k in range(4):
                    self.tag[base + k] = (addr[0], st, grp, kh, r, k)
                    self.unwaited.add(base + k)
                self.since_barrier_reads.add((addr[0], st))
            elif op == "ds_read_b64_tr_b16":
                dst, addr, off = re.match(r"ds_read_b64_tr_b16 (\S+), %\[b_rd(\d)\] offset:(\d+)", ln).groups()
                base, n = quad(dst)
                assert n == 2
                slot = int(off) // 2048
                st, kh, h = slot // 16, (slot % 16) // 8, slot % 2
                j = int(addr)
                for k in range(2):
                    self.tag[base + k] = ("b", st, j // 4, kh, j % 4, 2 * h + k)
                    self.unwaited.add(base + k)
                self.since_barrier_reads.add(("b", st))
            elif op == "s_waitcnt":
                if "lgkmcnt(0)" in ln:
                    self.unwaited.clear()
                m = re.search(r"vmcnt\((\d+)\)", ln)
                if m:
                    keep = int(m.group(1))
                    done = self.outstanding[:len(self.outstanding) - keep] if keep else self.outstanding
                    self.outstanding = self.outstanding[len(done):]
                    assert all(kind == "store" for kind, _ in self.outstanding), "a load still in flight behind the barrier's wait"
            elif op == "s_barrier":
                assert not self.unwaited, "barrier with fragment reads in flight"
                self.since_barrier_reads = set()
                self.behind_barrier = True
            elif op == "s_cselect_b32" and ln.split()[1] == f"s{self.gen.S_DB + 2},":
                step += 1                                   # B's length word for the tile at k_late opens a K step
                self.cur = stage_of_step(step)
                self.behind_barrier = False
                self.step = step
            elif op == "v_mfma_f32_16x16x32_bf16" and "%[ct]" in ln:
                b, a = re.match(r"\S+ %\[ct\], (\S+), (\S+), %\[ct\]", ln).groups()
                regs = {quad(a)[0] + k for k in range(4)} | {quad(b)[0] + k for k in range(4)}
                assert not regs & self.unwaited, f"{ln}: fragment read not waited for"
                ta = [self.tag[quad(a)[0] + k] for k in range(4)]
                tb = [self.tag[quad(b)[0] + k] for k in range(4)]
                assert [t[5] for t in ta] == [0, 1, 2, 3] and [t[5] for t in tb] == [0, 1, 2, 3]
                assert {t[0] for t in ta} == {"ta"} and {t[0] for t in tb} == {"tb"}
                assert {t[1] for t in ta + tb} == {self.cur} and len({t[3] for t in ta + tb}) == 1
                self.tail_mfma.setdefault(self.step, []).append(ta[0][3])
            elif op == "buffer_load_dword":
                assert (f"s[{self.gen.S_DA}:" in ln) == self.mtail_form      # through A's descriptor (ragged rows) or B's
                which, off = self.last_m0
                assert which == "t" and not self.behind_barrier and off // 2048 == self.cur ^ 1 and off % 2048 in (0, 256)
                self.tail_requests.append((self.step, off % 2048))
                self.outstanding.append(("load", off // 2048))
            elif op == "v_mfma_f32_16x16x32_bf16":
                acc, b, a, acc2 = re.match(r"\S+ (%\[c\d\d\]), (\S+), (\S+), (%\[c\d\d\])", ln).groups()
                assert acc == acc2
                i, j = int(acc[3]), int(acc[4])
                ta = [self.tag[quad(a)[0] + k] for k in range(4)]
                tb = [self.tag[quad(b)[0] + k] for k in range(4)]
                assert not ({quad(a)[0] + k for k in range(4)} | {quad(b)[0] + k for k in range(4)}) & self.unwaited, f"{ln}: fragment read not waited for"
                assert [t[5] for t in ta] == [0, 1, 2, 3] and [t[5] for t in tb] == [0, 1, 2, 3]
                assert len({t[:5] for t in ta}) == 1 and len({t[:5] for t in tb}) == 1
                (oa, sa, ga, ka, ra, _), (ob, sb, gb, kb, cb, _) = ta[0], tb[0]
                assert (oa, ob) == ("a", "b") and sa == sb == self.cur and ka == kb, f"{ln}: {ta[0]} x {tb[0]} in a step on stage {self.cur}"
                assert (4 * ga + ra, 4 * gb + cb) == (i, j), f"{ln}: multiplies A rows {4 * ga + ra}, B columns {4 * gb + cb}"
                self.mfma_of.setdefault((self.step, i, j), []).append(ka)
            elif op == "buffer_load_dwordx4":
                m0 = self.last_m0
                which, off = m0
                st, piece = off // 32768, (off % 32768) // 1024
                assert piece < 8
                if which == "a":
                    assert self.behind_barrier and st == self.cur and ("a", st) not in self.since_barrier_reads, "A's stage refilled while it may still be read"
                else:
                    assert not self.behind_barrier and st == self.cur ^ 1 and ("b", st) not in self.since_barrier_reads
                self.requests.append((self.step, which, st, piece))
                self.outstanding.append(("load", st))
            elif op == "s_add_u32" and ln.split()[1] == "m0,":
                base, off = re.match(r"s_add_u32 m0, %\[lds_(\w)\], (\d+)", ln).groups()      # lds_a, lds_b, lds_t
                self.last_m0 = (base, int(off))
            elif op == "buffer_store_dwordx4":
                base, n = quad(ln.split()[1].rstrip(","))
                assert n == 4 and (base - self.gen.CT0) % 4 == 0
                self.stores.append(((base - self.gen.CT0) // 4, self.last_rows))
                self.outstanding.append(("store", base))
            elif op == "s_mul_i32" and "c_row_bytes" in ln:
                self.last_rows = int(ln.rsplit(",", 1)[1])


@pytest.mark.parametrize("nt", [False, True], ids=["nn", "nt"])
@pytest.mark.parametrize("drain_steps", [0, 8, 16])
def test_generated_loop_multiplies_the_right_fragments(nt, drain_steps):
    gen = load_generator(drain_steps)
    em = gen.Emitter(nt, drain_steps > 0)
    em.loop()
    lines = [l for l in em.lines if not l.startswith("L_")]
    steps = drain_steps + 2
    rp = Replay(gen, nt)
    rp.run(lines, stage_of_step=lambda t: t & 1)
    assert rp.step == steps - 1
    # every accumulator: K half 0 then K half 1 of every step
    for t in range(steps):
        for i in range(8):
            for j in range(8):
                assert rp.mfma_of[(t, i, j)] == [0, 1], (t, i, j, rp.mfma_of.get((t, i, j)))
    assert sum(l.startswith("v_mfma") for l in lines) == 128 * steps
    # every step requests the eight pieces of A into its own stage and the eight of B into the other one
    for t in range(steps):
        got = sorted((w, p) for (s, w, st, p) in rp.requests if s == t)
        assert got == [("a", p) for p in range(8)] + [("b", p) for p in range(8)]
    # the deferred tile: 32 stores, each quad once, at the rows the epilogue's store of the same number writes
    if drain_steps:
        assert sorted(q for q, _ in rp.stores) == list(range(32))
        assert all(rows == 32 * (q // 8) + 4 * (q % 8) for q, rows in rp.stores)
        assert all(kind == "load" for kind, _ in rp.outstanding), "stores still in flight when the steady loop's first barrier has passed"
    else:
        assert not rp.stores and not any("buffer_store" in l for l in lines)


def test_replay_rejects_a_wrong_fragment():
    """The check has teeth: the same loop with one matrix instruction's A fragment swapped for its neighbour's."""
    gen = load_generator(0)
    em = gen.Emitter(True)
    em.loop()
    lines = list(em.lines)
    k = next(i for i, l in enumerate(lines) if l.startswith("v_mfma") and f"v[{gen.FA0}:{gen.FA0 + 3}]" in l)
    lines[k] = lines[k].replace(f"v[{gen.FA0}:{gen.FA0 + 3}]", f"v[{gen.FA0 + 4}:{gen.FA0 + 7}]")
    with pytest.raises(AssertionError):
        Replay(gen, True).run([l for l in lines if not l.startswith("L_")], stage_of_step=lambda t: t & 1)
    # ... and with the wait in front of the second eighth dropped (it multiplies the B group the first eighth read)
    lines = list(em.lines)
    k = [i for i, l in enumerate(lines) if l == "s_waitcnt lgkmcnt(0)"][1]
    del lines[k]
    with pytest.raises(AssertionError):
        Replay(gen, True).run([l for l in lines if not l.startswith("L_")], stage_of_step=lambda t: t & 1)


def test_the_default_make_target_builds_the_library_and_the_generated_loop_first():
    """`make` with no target must build libmaize_hip.so (a rule placed in front of `all` silently becomes the default
    target), and the code object depends on the generated include."""
    import subprocess
    csrc = os.path.dirname(os.path.dirname(GEN))
    plan = subprocess.run(["make", "-n", "-B", "-C", csrc], check=True, capture_output=True, text=True).stdout
    assert "gen_kloop.py" in plan and "gemm_kernels.hip" in plan and "libmaize_hip.so" in plan
    assert plan.index("gen_kloop.py") < plan.index("gemm_kernels.hip") < plan.index("libmaize_hip.so")


@pytest.mark.parametrize("nt", [False, True], ids=["nn", "nt"])
@pytest.mark.parametrize("rows", [False, True], ids=["columns", "rows"])
def test_the_ragged_block_rides_along(nt, rows):
    """The forms of the loop that also multiply one 16 x 16 block against the ragged last columns (rows): per K step two
    more matrix instructions (K half 0, then 1) on fragments of the step's own stage -- one from the whole tile's stage,
    one from the block's own tile -- read and waited for, and two 256-byte requests per wave into the other stage of that
    tile, in front of the barrier, through B's (A's) descriptor; the rest of the loop as before."""
    gen = load_generator(0)
    em = gen.Emitter(nt, False, not rows, rows)
    em.loop()
    lines = [l for l in em.lines if not l.startswith("L_")]
    rp = Replay(gen, nt)
    rp.mtail_form = rows
    rp.run(lines, stage_of_step=lambda t: t & 1)
    assert rp.step == 1
    for t in range(2):
        assert rp.tail_mfma[t] == [0, 1]
        assert sorted(o for s_, o in rp.tail_requests if s_ == t) == [0, 256]
        for i in range(8):
            for j in range(8):
                assert rp.mfma_of[(t, i, j)] == [0, 1]
    assert sum(l.startswith("v_mfma") for l in lines) == 2 * (128 + 2)
    if rows:
        # A's length word is set before the first request that goes through it
        first_request = next(i for i, l in enumerate(lines) if l.startswith("buffer_load_dword "))
        assert any(l.startswith(f"s_cselect_b32 s{gen.S_DA + 2}, %[a_bytes]") for l in lines[:first_request])
    # the plain form has none of it
    plain = gen.Emitter(nt)
    plain.loop()
    assert not any("%[ct]" in l or "lds_t" in l for l in plain.lines)
