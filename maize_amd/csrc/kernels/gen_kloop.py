#!/usr/bin/env python3
"""Generates kloop_gen.inc: the K loop of the 256 x 256 bf16 macro-tile kernel as ONE inline-assembly statement
with its own register assignment (run by the Makefile before the code object is compiled).

The loop is the schedule of gemm_mt256.hpp's step() -- eight eighths of 16 MFMAs per K step, one new fragment
group read per eighth, the sixteen 1 KiB requests of a step one every four MFMA slots, one barrier per step in
front of the seventh eighth, two ring stages -- written out instruction by instruction from the same table
(tests/test_schedule_model.py replays it), so that nothing of it depends on the compiler's register allocator:

  accumulators  acc[i][j]      the compiler's choice among the AccVGPRs ("+a" operands: a physical-register
                               constraint makes the compiler copy all 256 of them to vector registers behind the statement)
  A fragments   fa[ai][r]      v[FA0 + 16 ai + 4 r .. + 3]    (clobbered)
  B fragments   fb[buf][c]     v[FB0 + 16 buf + 4 c .. + 3]   (clobbered; a row-major B: low half = the k + 0..3 read,
                                                              high half = the k + 4..7 read of a transposing pair)
  scalars       s[SW .. SW + 19]                               (clobbered): working descriptors, byte offsets, counter

Everything else (address registers, per-piece offsets, descriptors' words, LDS bases) comes in as operands.
What this buys over the statement-by-statement loop: the trip can be left after its first step (an odd step
count no longer runs a step on a zero tile), and side work can be given registers of its own.

Forms written out (functions of kloop_gen.inc), each for B stored N x K (nt) and K x N (nn):
  kloop_asm_{nt,nn}          the plain loop
  kloop_asm_{nt,nn}_ntail    ... that also multiplies one 16 x 16 block against up to sixteen ragged last columns of B and C
  kloop_asm_{nt,nn}_mtail    ... against up to sixteen ragged last rows of A and C (Emitter.tail_*)
  kloop_asm_{nt,nn}_drain    (only with KLOOP_DRAIN_STEPS=n in the environment) ... that stores the previous C tile from
                             registers during its first n steps (Emitter.drain_side_work): measured slower, not built by default

Usage: gen_kloop.py OUT.inc
"""
import os
import sys

FA0, FB0 = 192, 224        # fragment registers v[192:223] (A), v[224:255] (B): the top of the file, so that the compiler keeps one contiguous range
SW = 80                    # working scalars s[80:99]
S_DA = SW                  # s[80:83]  descriptor of A (word 2 = bytes or 0)
S_DB = SW + 4              # s[84:87]  descriptor of B
S_KT = SW + 8              # s88       K steps done
S_OE = SW + 9              # s89       byte offset of the tile requested behind the barrier (k_early * 2)
S_OL = SW + 10             # s90       ... of the tile requested in front of it (k_late * 2)
S_T = SW + 11              # s91       scratch
S_BASE = SW + 12           # s[92:93]  row-major B: address of row k_late
S_REM = SW + 14            # s[94:95]  row-major B: bytes from there to the end of the view
DMA_STRIDE, EB, NE = 4, 6, 8
# Deferred C stores (the "drain" form of the loop): the previous C tile of this workgroup, already rounded to bf16 and
# turned through LDS into store order, is stored while the first DRAIN_STEPS K steps of the next one run, straight from
# registers.
CT0 = 64                   # v[64:191]: quad Q = 8 p + r in v[CT0 + 4 Q .. + 3]: what the epilogue's store r of pass p holds --
                           # 16 bytes (8 columns) per lane, 16 lanes per 256-byte row of the wave's half, rows 32 p + 4 r + l / 16
S_DC = SW + 16             # s[96:99]  descriptor of the C tile being drained
S_T2 = SW + 20             # s100      scratch of the requests
VT0 = 63                   # v63       per-lane byte offset of a request (read when the request issues: the next may overwrite it)
FT_A, FT_B = 184, 188     # v[184:187], v[188:191]: A and B fragment of the ragged block (the "ntail" / "mtail" forms of the loop)
DRAIN_POLICY = " nt"       # cache policy of the deferred stores (" nt": streaming, like the stores of the epilogue)
# K steps a deferred tile is stored over (an even divisor of 32: 32 / DRAIN_STEPS stores of 16 bytes per lane and step), or
# 0: no deferred stores, the build that ships.  Measured (4 x 4096^3, four tiles per workgroup): stores inside the K loop
# cost more than stores at the tile boundary -- the loop with them 437 us, the kernel that stores at once 419 us, the loop
# with the deferred tiles never stored 414 us -- whether spread over 16, 8 or 4 steps, streaming or write-back.
DRAIN_STEPS = int(os.environ.get("KLOOP_DRAIN_STEPS", "0"))
NO_STORE = bool(os.environ.get("KLOOP_NO_STORE"))   # timing experiments only: the deferred tile is never stored
COMPACT = DRAIN_STEPS > 0  # the deferred tile takes 128 registers: per-piece offsets are derived in the loop instead of held


def fa(ai, r):
    b = FA0 + 16 * ai + 4 * r
    return f"v[{b}:{b + 3}]"


def fb(buf, c, half=None):
    b = FB0 + 16 * buf + 4 * c
    if half is None:
        return f"v[{b}:{b + 3}]"
    return f"v[{b + 2 * half}:{b + 2 * half + 1}]"


def acc(i, j):
    return f"%[c{i}{j}]"


class Emitter:
    def __init__(self, nt, drain=False, ntail=False, mtail=False):
        self.nt = nt
        self.drain = drain
        self.ntail = ntail
        self.mtail = mtail
        assert not (ntail and mtail)
        self.lines = []

    # ---- the ragged last columns of B and C (N = 256 t + 8 or 16) -----------------------------------
    # Instead of a tile column of its own, the up to sixteen columns past the last whole tile column ride along: the
    # workgroup of tile (tm, tn) also computes rows 16 (tn % 16) .. + 15 of its row panel against them -- one 16 x 16
    # block, two matrix instructions per K step, all four waves alike (the block is the same in all of them; wave 0
    # stores it).  Its B tile, 64 x 16 elements (2 KiB), has two stages of its own at %[lds_t]; each wave brings in a
    # quarter with two 4-byte-per-lane requests behind B's last piece, into the stage of tile t+1; its A fragment is
    # read from A's stage (address registers %[a_rdt0/1] point at the block's rows).
    # The mirror image ("mtail"): up to sixteen ragged last rows of A and C (M = 256 t + 1 .. 16).  The workgroup of tile
    # (tm, tn) multiplies them against columns 16 (tm % 16) .. + 15 of its column panel: the B fragment comes from B's
    # stage (address registers %[b_rdt..]), the rows' A tile (16 x 64, K-contiguous, 2 KiB) has the two stages at
    # %[lds_t] and is requested through A's descriptor -- whose length word still stands for tile t+1 in front of the
    # barrier of step t -- at tile t+1's byte offset.
    def tail_request(self, j, stage):
        self.e(f"s_add_u32 m0, %[lds_t], {stage * 2048 + j * 256}")
        self.e("s_nop 0")
        if self.mtail:
            self.e(f"buffer_load_dword %[t_vo{j}], s[{S_DA}:{S_DA + 3}], s{S_OL} offen lds")
        else:
            soff = f"s{S_OL}" if self.nt else "0"
            self.e(f"buffer_load_dword %[t_vo{j}], s[{S_DB}:{S_DB + 3}], {soff} offen lds")

    def tail_reads(self, kh, st):
        if self.mtail:
            self.e(f"ds_read_b128 v[{FT_A}:{FT_A + 3}], %[t_rd{kh}] offset:{st * 2048}")
            if self.nt:
                self.e(f"ds_read_b128 v[{FT_B}:{FT_B + 3}], %[b_rdt{kh}] offset:{st * 32768}")
            else:
                for h in range(2):
                    self.e(f"ds_read_b64_tr_b16 v[{FT_B + 2 * h}:{FT_B + 2 * h + 1}], %[b_rdt0] offset:{st * 32768 + kh * 16384 + h * 2048}")
            return
        self.e(f"ds_read_b128 v[{FT_A}:{FT_A + 3}], %[a_rdt{kh}] offset:{st * 32768}")
        if self.nt:
            self.e(f"ds_read_b128 v[{FT_B}:{FT_B + 3}], %[t_rd{kh}] offset:{st * 2048}")
        else:
            for h in range(2):
                self.e(f"ds_read_b64_tr_b16 v[{FT_B + 2 * h}:{FT_B + 2 * h + 1}], %[t_rd0] offset:{st * 2048 + kh * 1024 + h * 128}")

    def tail_mfma(self):
        self.e(f"v_mfma_f32_16x16x32_bf16 %[ct], v[{FT_B}:{FT_B + 3}], v[{FT_A}:{FT_A + 3}], %[ct]")

    # ---- deferred C stores ----------------------------------------------------------------------
    # Step t of the first DRAIN_STEPS stores quads n t .. n t + n - 1 (n = 32 / DRAIN_STEPS).  The counter the barrier
    # waits on counts loads and stores alike and they retire in order: the stores go out behind the step's last request
    # and in front of the barrier, whose wait then leaves n operations outstanding -- them -- so that a store has a whole
    # K step to be acknowledged before the next barrier's wait reaches it.  Rows past M fall behind the descriptor's end; columns past N
    # carry the out-of-range bit in the lane's offset, as in the epilogue that stores at once.
    def drain_side_work(self, t, e, s):
        if not self.draining(t) or e not in (2, 3, 4, 5):
            return
        per_step = 32 // DRAIN_STEPS
        gap = 64 // per_step                               # matrix instructions between two stores
        slot = 16 * (e - 2) + s
        if slot % gap == gap // 2:
            q = per_step * t + slot // gap
            rows = 32 * (q // 8) + 4 * (q % 8)
            self.e(f"s_mul_i32 s{S_T}, %[c_row_bytes], {rows}")
            if not NO_STORE: self.e(f"buffer_store_dwordx4 v[{CT0 + 4 * q}:{CT0 + 4 * q + 3}], %[c_vo], s[{S_DC}:{S_DC + 3}], s{S_T} offen{DRAIN_POLICY}")

    def draining(self, t):
        return self.drain and t is not None and t < DRAIN_STEPS

    def e(self, s):
        self.lines.append(s)

    # ---- fragment reads -----------------------------------------------------------------------
    def read_a(self, ai, kh, st, r):
        self.e(f"ds_read_b128 {fa(ai, r)}, %[a_rd{kh}] offset:{(st * 16 + 4 * ai + r) * 2048}")

    def read_b(self, bi, kh, st, r):
        buf = bi ^ kh
        if self.nt:
            self.e(f"ds_read_b128 {fb(buf, r)}, %[b_rd{kh}] offset:{(st * 16 + 4 * bi + r) * 2048}")
        else:
            c, h = r >> 1, r & 1
            self.e(f"ds_read_b64_tr_b16 {fb(buf, c, h)}, %[b_rd{4 * bi + c}] offset:{(st * 16 + kh * 8 + h) * 2048}")

    @property
    def nbr(self):
        return 4 if self.nt else 8

    # ---- requests -----------------------------------------------------------------------------
    def request(self, pc, stage):
        """Piece pc (0..7: A, from the tile at k_early; 8..15: B, from the tile at k_late) into ring stage `stage`.
        The per-lane byte offset of piece i is that of piece i % 2 plus (i / 2) * 16 rows (K-contiguous tiles; the swizzle
        has period 16 rows), resp. that of piece i & 5 plus 4 rows if i & 2 (row-major B: the swizzle looks at bits 0, 1
        and 3 of the row): added here, on the vector unit, instead of holding eight offsets per operand in registers.
        (Not in the instruction's scalar offset: that one is outside the descriptor's range check, which the M and N
        edges rely on.)"""
        is_a, i = pc < 8, pc % 8
        base = "%[lds_a]" if is_a else "%[lds_b]"
        tmp = f"v{VT0}"
        if not COMPACT:
            vo = f"%[{'a' if is_a else 'b'}_vo{i}]"
        elif is_a or self.nt:
            rep, mult, step = i & 1, i >> 1, ("%[a_step]" if is_a else "%[b_step]")
            vo = f"%[{'a' if is_a else 'b'}_vo{rep}]"
            if mult:
                self.e(f"s_mul_i32 s{S_T2}, {step}, {mult}")
                self.e(f"v_add_u32 {tmp}, s{S_T2}, {vo}")
                vo = tmp
        else:
            rep = (i & 1) | (((i >> 2) & 1) << 1)
            vo = f"%[b_vo{rep}]"
            if i & 2:
                self.e(f"v_add_u32 {tmp}, %[b_step], {vo}")
                vo = tmp
        self.e(f"s_add_u32 m0, {base}, {stage * 32768 + i * 1024}")
        self.e("s_nop 0")
        if is_a:
            self.e(f"buffer_load_dwordx4 {vo}, s[{S_DA}:{S_DA + 3}], s{S_OE} offen lds")
        elif self.nt:
            self.e(f"buffer_load_dwordx4 {vo}, s[{S_DB}:{S_DB + 3}], s{S_OL} offen lds")
        else:
            self.e(f"buffer_load_dwordx4 {vo}, s[{S_DB}:{S_DB + 3}], 0 offen lds")

    def bytes_of_a(self):
        """Word 2 of A's descriptor for the tile at k_early: all of the view, or nothing at or past the end of the range."""
        self.e("s_cmp_lt_u32 %[k_early], %[k_end]")
        self.e(f"s_cselect_b32 s{S_DA + 2}, %[a_bytes], 0")

    def bytes_of_b(self):
        """... of B's for the tile at k_late.  A row-major B is re-based on the K tile's first row."""
        if self.nt:
            self.e("s_cmp_lt_u32 %[k_late], %[k_end]")
            self.e(f"s_cselect_b32 s{S_DB + 2}, %[b_bytes], 0")
            return
        self.e(f"s_mov_b32 s{S_DB}, s{S_BASE}")
        self.e(f"s_and_b32 s{S_DB + 1}, s{S_BASE + 1}, 0xffff")
        # bytes = min(remaining, 0x7fffffff), or 0 at or past the end of the range
        self.e(f"s_cmp_lg_u32 s{S_REM + 1}, 0")
        self.e(f"s_cselect_b32 s{S_T}, 0x7fffffff, s{S_REM}")
        self.e(f"s_min_u32 s{S_T}, s{S_T}, 0x7fffffff")
        self.e("s_cmp_lt_u32 %[k_late], %[k_end]")
        self.e(f"s_cselect_b32 s{S_DB + 2}, s{S_T}, 0")

    def advance(self):
        """One K step on: both tile positions, their byte offsets, and a row-major B's address and remainder."""
        self.e("s_add_u32 %[k_early], %[k_early], 64")
        self.e("s_add_u32 %[k_late], %[k_late], 64")
        self.e(f"s_add_u32 s{S_OE}, s{S_OE}, 128")
        self.e(f"s_add_u32 s{S_OL}, s{S_OL}, 128")
        if not self.nt:
            self.e(f"s_add_u32 s{S_BASE}, s{S_BASE}, %[b_step_lo]")
            self.e(f"s_addc_u32 s{S_BASE + 1}, s{S_BASE + 1}, %[b_step_hi]")
            self.e(f"s_sub_u32 s{S_REM}, s{S_REM}, %[b_step_lo]")
            self.e(f"s_subb_u32 s{S_REM + 1}, s{S_REM + 1}, %[b_step_hi]")

    # ---- one K step ---------------------------------------------------------------------------
    def step(self, cur, t=None):
        nxt = cur ^ 1
        self.bytes_of_b()                      # the requests in front of the barrier are B's eight pieces of tile t+1
        for e in range(NE):
            kh, h4 = e >> 2, e & 3
            ai = h4 >> 1
            bi = 1 if h4 in (1, 2) else 0
            last_half = kh == 1
            if e != EB:
                self.e("s_waitcnt lgkmcnt(0)")
            else:
                # every fragment this step still needs is in registers; tile t+1 has landed once all waves are here
                self.e(f"s_waitcnt vmcnt({32 // DRAIN_STEPS if self.draining(t) and not NO_STORE else 0}) lgkmcnt(0)")
                self.e("s_barrier")
                self.bytes_of_a()              # behind the barrier: A's eight pieces of tile t+2, into the stage just read
            for s in range(16):
                hi4 = s >> 2
                lo4 = 3 - (s & 3) if hi4 & 1 else s & 3
                r4, c4 = lo4, hi4
                self.e(f"v_mfma_f32_16x16x32_bf16 {acc(4 * ai + r4, 4 * bi + c4)}, {fb(bi ^ kh, c4)}, {fa(ai, r4)}, {acc(4 * ai + r4, 4 * bi + c4)}")
                r = s
                if h4 == 0 and r < self.nbr:
                    self.read_b(1, kh, cur, r)
                if h4 == 3 and r < self.nbr:
                    self.read_b(0, 1, cur, r) if not last_half else self.read_b(0, 0, nxt, r)
                if h4 == 1 and r < 4:
                    self.read_a(1, kh, cur, r)
                if h4 == 2 and r < 4:
                    self.read_a(0, 1, cur, r) if not last_half else self.read_a(0, 0, nxt, r)
                slot = 16 * (e - EB) + s if e >= EB else 16 * (NE - EB) + 16 * e + s
                if slot >= 2 and (slot - 2) % DMA_STRIDE == 0 and (slot - 2) // DMA_STRIDE < 16:
                    pc = (slot - 2) // DMA_STRIDE
                    assert (pc < 8) == (e >= EB)
                    self.request(pc, cur if e >= EB else nxt)
                self.drain_side_work(t, e, s)
                if self.ntail or self.mtail:
                    if e == 2 and s in (2, 6):
                        self.tail_request((s - 2) // 4, nxt)
                    if e in (0, 4) and s == 10:
                        self.tail_reads(e // 4, cur)       # (waited for by the next eighth's counter wait)
                    if e in (1, 5) and s == 15:
                        self.tail_mfma()
        self.advance()

    def loop(self):
        # set-up: working descriptors, byte offsets, counter; the first fragments of the tile in stage 0
        self.e(f"s_mov_b32 s{S_DA}, %[a_lo]")
        self.e(f"s_mov_b32 s{S_DA + 1}, %[a_hi]")
        self.e(f"s_mov_b32 s{S_DA + 3}, %[flags]")
        self.e(f"s_mov_b32 s{S_DB + 3}, %[flags]")
        if self.nt:
            self.e(f"s_mov_b32 s{S_DB}, %[b_lo]")
            self.e(f"s_mov_b32 s{S_DB + 1}, %[b_hi]")
        else:
            self.e(f"s_mov_b32 s{S_BASE}, %[b_lo]")
            self.e(f"s_mov_b32 s{S_BASE + 1}, %[b_hi]")
            self.e(f"s_mov_b32 s{S_REM}, %[b_rem_lo]")
            self.e(f"s_mov_b32 s{S_REM + 1}, %[b_rem_hi]")
        if self.mtail:
            # (the ragged rows' first request, in front of step 0's barrier, goes through A's descriptor: its length word,
            # otherwise first written behind that barrier, stands for the tile at k_late)
            self.e("s_cmp_lt_u32 %[k_late], %[k_end]")
            self.e(f"s_cselect_b32 s{S_DA + 2}, %[a_bytes], 0")
        self.e(f"s_lshl_b32 s{S_OE}, %[k_early], 1")
        self.e(f"s_lshl_b32 s{S_OL}, %[k_late], 1")
        self.e(f"s_mov_b32 s{S_KT}, 0")
        for r in range(4):
            self.read_a(0, 0, 0, r)
        for r in range(self.nbr):
            self.read_b(0, 0, 0, r)
        if self.drain:
            # the first DRAIN_STEPS steps, unrolled, with the previous tile's stores woven in (the caller guarantees
            # nk >= DRAIN_STEPS); then the steady loop for what is left
            self.e(f"s_mov_b32 s{S_DC}, %[c_lo]")
            self.e(f"s_mov_b32 s{S_DC + 1}, %[c_hi]")
            self.e(f"s_mov_b32 s{S_DC + 2}, %[c_bytes]")
            self.e(f"s_mov_b32 s{S_DC + 3}, %[flags]")
            for t in range(DRAIN_STEPS):
                self.step(t & 1, t)
            self.e(f"s_mov_b32 s{S_KT}, {DRAIN_STEPS}")
            self.e(f"s_cmp_ge_u32 s{S_KT}, %[nk]")
            self.e("s_cbranch_scc1 L_kloop_end_%=")
        self.e("L_kloop_top_%=:")
        self.step(0)
        self.e(f"s_add_u32 s{S_KT}, s{S_KT}, 1")
        self.e(f"s_cmp_ge_u32 s{S_KT}, %[nk]")
        self.e("s_cbranch_scc1 L_kloop_end_%=")          # an odd number of steps: out after the last real one
        self.step(1)
        self.e(f"s_add_u32 s{S_KT}, s{S_KT}, 1")
        self.e(f"s_cmp_lt_u32 s{S_KT}, %[nk]")
        self.e("s_cbranch_scc1 L_kloop_top_%=")
        self.e("L_kloop_end_%=:")


def function(nt, drain=False, ntail=False, mtail=False):
    em = Emitter(nt, drain, ntail, mtail)
    em.loop()
    name = ("kloop_asm_nt" if nt else "kloop_asm_nn") + ("_drain" if drain else "") + ("_ntail" if ntail else "") + ("_mtail" if mtail else "")
    nb_rd = 2 if nt else 8
    out = []
    out.append(f"// {'B stored N x K' if nt else 'B stored K x N (row-major)'}: {sum(l.startswith('v_mfma') for l in em.lines)} matrix instructions per trip")
    params = ["floatx4 (&acc)[8][8]", "const uint32_t (&a_rd)[2]", f"const uint32_t (&b_rd)[{8}]", "const uint32_t (&a_vo)[8]", "const uint32_t (&b_vo)[8]", "uint32_t a_step, uint32_t b_step",
              "uint32_t a_lo, uint32_t a_hi, uint32_t a_bytes, uint32_t b_lo, uint32_t b_hi, uint32_t b_bytes",
              "uint32_t b_rem_lo, uint32_t b_rem_hi, uint32_t b_step_lo, uint32_t b_step_hi",
              "uint32_t flags, uint32_t lds_a, uint32_t lds_b, uint32_t& k_early, uint32_t& k_late, uint32_t k_end, uint32_t nk"]
    if drain:
        params += ["const u32x4 (&ct)[32]", "uint32_t c_vo", "uint32_t c_lo, uint32_t c_hi, uint32_t c_bytes, uint32_t c_row_bytes"]
    if ntail or mtail:    # (x_rdt: address registers of the fragment read from the whole tile's stage, A's or B's)
        params += ["floatx4& acc_t", "const uint32_t (&x_rdt)[2]", "const uint32_t (&t_rd)[2]", "const uint32_t (&t_vo)[2]", "uint32_t lds_t"]
    out.append(f"__device__ __forceinline__ void {name}({', '.join(params)}) {{")
    out.append("    asm volatile(")
    for l in em.lines:
        out.append(f'        "{l}\\n\\t"')
    outs = [f'[c{i}{j}] "+a"(acc[{i}][{j}])' for i in range(8) for j in range(8)]
    outs += ['[k_early] "+s"(k_early)', '[k_late] "+s"(k_late)']
    ins = [f'[a_rd{k}] "v"(a_rd[{k}])' for k in range(2)] + [f'[b_rd{k}] "v"(b_rd[{k}])' for k in range(nb_rd)]
    if COMPACT:   # offsets of the representative pieces only: 0, 1 of a K-contiguous tile; 0, 1, 4, 5 of a row-major B
        ins += [f'[a_vo{k}] "v"(a_vo[{k}])' for k in range(2)]
        ins += [f'[b_vo{k}] "v"(b_vo[{k}])' for k in range(2)] if nt else [f'[b_vo{q}] "v"(b_vo[{k}])' for q, k in enumerate((0, 1, 4, 5))]
        ins += ['[a_step] "s"(a_step)', '[b_step] "s"(b_step)']
    else:
        ins += [f'[a_vo{k}] "v"(a_vo[{k}])' for k in range(8)] + [f'[b_vo{k}] "v"(b_vo[{k}])' for k in range(8)]
    ins += ['[a_lo] "s"(a_lo)', '[a_hi] "s"(a_hi)', '[a_bytes] "s"(a_bytes)', '[b_lo] "s"(b_lo)', '[b_hi] "s"(b_hi)', '[flags] "s"(flags)',
            '[lds_a] "s"(lds_a)', '[lds_b] "s"(lds_b)', '[k_end] "s"(k_end)', '[nk] "s"(nk)']
    if nt:
        ins += ['[b_bytes] "s"(b_bytes)']
    else:
        ins += ['[b_rem_lo] "s"(b_rem_lo)', '[b_rem_hi] "s"(b_rem_hi)', '[b_step_lo] "s"(b_step_lo)', '[b_step_hi] "s"(b_step_hi)']
    clob = ['"memory"', '"scc"', '"m0"'] + [f'"v{r}"' for r in range(FA0, FB0 + 32)] + [f'"s{r}"' for r in range(SW, SW + 16)]
    if COMPACT:
        clob += [f'"v{VT0}"', f'"s{S_T2}"']
    if drain:
        ins += [f'"{{v[{CT0 + 4 * q}:{CT0 + 4 * q + 3}]}}"(ct[{q}])' for q in range(32)]
        ins += ['[c_vo] "v"(c_vo)', '[c_lo] "s"(c_lo)', '[c_hi] "s"(c_hi)', '[c_bytes] "s"(c_bytes)', '[c_row_bytes] "s"(c_row_bytes)']
        clob += [f'"s{r}"' for r in range(S_DC, S_DC + 4)]
    if ntail:
        outs += ['[ct] "+v"(acc_t)']
        ins += [f'[a_rdt{k}] "v"(x_rdt[{k}])' for k in range(2)] + [f'[t_rd{k}] "v"(t_rd[{k}])' for k in range(2 if nt else 1)]
    if mtail:
        outs += ['[ct] "+v"(acc_t)']
        ins += [f'[b_rdt{k}] "v"(x_rdt[{k}])' for k in range(2 if nt else 1)] + [f'[t_rd{k}] "v"(t_rd[{k}])' for k in range(2)]
    if ntail or mtail:
        ins += [f'[t_vo{k}] "v"(t_vo[{k}])' for k in range(2)] + ['[lds_t] "s"(lds_t)']
        clob += [f'"v{r}"' for r in range(FT_A, FT_B + 4)]
    out.append("        : " + ", ".join(outs))
    out.append("        : " + ", ".join(ins))
    out.append("        : " + ", ".join(clob) + ");")
    if not COMPACT:
        out.append("    (void)a_step; (void)b_step;")
    if nt:
        out.append("    (void)b_rem_lo; (void)b_rem_hi; (void)b_step_lo; (void)b_step_hi;")
    else:
        out.append("    (void)b_bytes;")
    out.append("}")
    return "\n".join(out)


def main():
    text = ["// GENERATED by gen_kloop.py -- do not edit.  The K loop of the 256 x 256 bf16 macro-tile kernel as one",
            "// inline-assembly statement with its own register assignment (see the generator for the register map).",
            "#pragma once", "", f"constexpr uint32_t KLOOP_DRAIN_STEPS = {DRAIN_STEPS};   // K steps a deferred C tile is stored over", "", function(True), "", function(False), ""]
    text += [function(True, ntail=True), "", function(False, ntail=True), "", function(True, mtail=True), "", function(False, mtail=True), ""]
    if DRAIN_STEPS:
        text += [function(True, True), "", function(False, True), ""]
    with open(sys.argv[1], "w") as f:
        f.write("\n".join(text))


if __name__ == "__main__":
    main()
