"""What the embedded gfx950 code object contains, kernel by kernel.

The reference checks its MMA catalogue by compiling a one-op kernel and asserting that the emitted PTX
contains the op's mnemonic (run_test_sync_mma, crates/maize_tile/src/mma/mod.rs:101-114).  The analogue
here disassembles the library's own code object (llvm-objdump of the ROCm toolchain that built it) and
asserts, for every GEMM kernel, the matrix instruction of its operand type, the data-movement
instructions the design rests on, and what must be absent: scratch memory (its mere use slowed a launch
by 13 us), writes through the scalar data cache, and packed-fp32 arithmetic."""
import os
import re
import shutil
import subprocess

import pytest

import maize_amd as mz

OBJDUMP = shutil.which("llvm-objdump") or "/opt/rocm/llvm/bin/llvm-objdump"
READELF = shutil.which("llvm-readelf") or "/opt/rocm/llvm/bin/llvm-readelf"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HSACO = os.path.join(ROOT, "maize_amd", "lib", "maize_gemm_gfx950.hsaco")

pytestmark = pytest.mark.skipif(not (os.path.exists(OBJDUMP) and os.path.exists(HSACO)),
                                reason="needs the ROCm llvm-objdump and the built code object")


@pytest.fixture(scope="module")
def kernels():
    """{kernel name: list of instruction mnemonics+operands}."""
    text = subprocess.run([OBJDUMP, "-d", "--mcpu=gfx950", HSACO], check=True, capture_output=True, text=True).stdout
    out, cur = {}, None
    for line in text.splitlines():
        m = re.match(r"^[0-9a-f]+ <([A-Za-z0-9_]+)>:", line)
        if m:
            if not m.group(1).startswith("L_"):       # (labels inside an assembly statement are not kernels)
                cur = out.setdefault(m.group(1), [])
            continue
        if cur is not None and "\t" in line:
            ins = line.split("//")[0].strip()
            if ins:
                cur.append(ins)
    return out


def count(instrs, prefix):
    return sum(1 for i in instrs if i.startswith(prefix))


def test_every_registry_entry_has_its_device_kernel(kernels):
    for name in mz.kernel_names():
        assert name.replace("_packed_gen", "_gen").replace("_packed", "_splitk").replace("_trb", "") in kernels, name      # registry entries that reuse a device kernel
    for helper in ("maize_gemm_splitk_reduce", "maize_pack_2d", "maize_pack_2d_u8", "maize_transpose_u8"):
        assert helper in kernels


def test_matrix_instruction_per_kernel(kernels):
    for name, ins in kernels.items():
        if name.endswith(("_skinny_nt_m32", "_skinny_nt_m64")):
            # 17 .. 64 rows against N x K weights: the same instructions, 2 or 4 row groups per fragment of B, A through LDS
            groups = 2 if name.endswith("_m32") else 4
            if name.startswith("maize_gemm_bf16"):
                # 4 turns x 2 fragments of B x row groups x 2 K steps
                assert count(ins, "v_mfma_f32_16x16x32_bf16") >= 16 * groups and count(ins, "v_mfma_f32_16x16x32_f16") >= 16 * groups, name
            else:
                f8 = [i for i in ins if i.startswith("v_mfma_f32_16x16x128_f8f6f4")]
                tag = name[len("maize_gemm_"):].split("_")[0]
                a_e5m2, b_e5m2 = {"e4m3": (0, 0), "e5m2": (1, 1), "e4m3e5m2": (0, 1), "e5m2e4m3": (1, 0)}[tag]
                assert len(f8) >= 8 * groups and all(("cbsz:1" in i) == bool(b_e5m2) and ("blgp:1" in i) == bool(a_e5m2) for i in f8), name
            assert count(ins, "ds_read_b128") >= 16 + 8 * groups and count(ins, "ds_read_b64_tr_b16") == 0, name
            assert len([i for i in ins if i.startswith("buffer_load_dwordx4") and " lds" in i]) >= 16 + 2 * groups, name
            assert count(ins, "s_barrier") >= 4, name                     # one per block: the A blocks are shared
        elif "_skinny_nn" in name and not name.startswith("maize_gemm_bf16"):
            # 8-bit operands, few rows against a row-major (K x N) B: 1, 2 or 4 row groups, A through LDS by 128-bit reads,
            # B's operand by four transposing 8-byte reads per column group; 4 turns x 2 column groups x row groups
            groups = 2 if name.endswith("_m32") else 4 if name.endswith("_m64") else 1
            f8 = [i for i in ins if i.startswith("v_mfma_f32_16x16x128_f8f6f4")]
            tag = name[len("maize_gemm_"):].split("_")[0]
            a_e5m2, b_e5m2 = {"e4m3": (0, 0), "e5m2": (1, 1), "e4m3e5m2": (0, 1), "e5m2e4m3": (1, 0)}[tag]
            assert len(f8) == 8 * groups and count(ins, "v_mfma") == 8 * groups, name
            assert all(("cbsz:1" in i) == bool(b_e5m2) and ("blgp:1" in i) == bool(a_e5m2) for i in f8), name
            assert count(ins, "ds_read_b64_tr_b8") == 32 and count(ins, "ds_read_b128") >= 8 * groups and count(ins, "ds_read_b64_tr_b16") == 0, name
            assert len([i for i in ins if i.startswith("buffer_load_dwordx4") and " lds" in i]) >= 16 + 2 * groups, name
            assert count(ins, "s_barrier") >= 4, name                     # one per block: the A blocks are shared
        elif name.endswith("_skinny_nt"):
            # M <= 16 against N x K weights: 16-row instructions, 32 deep for 16-bit operands (bf16 and half in one
            # kernel), 128 deep for 8-bit ones (format codes as below)
            if name == "maize_gemm_bf16_skinny_nt":
                assert count(ins, "v_mfma_f32_16x16x32_bf16") >= 16 and count(ins, "v_mfma_f32_16x16x32_f16") >= 16
            else:
                f8 = [i for i in ins if i.startswith("v_mfma_f32_16x16x128_f8f6f4")]
                tag = name[len("maize_gemm_"):].split("_")[0]
                a_e5m2, b_e5m2 = {"e4m3": (0, 0), "e5m2": (1, 1), "e4m3e5m2": (0, 1), "e5m2e4m3": (1, 0)}[tag]
                assert len(f8) >= 8 and all(("cbsz:1" in i) == bool(b_e5m2) and ("blgp:1" in i) == bool(a_e5m2) for i in f8), name
            assert count(ins, "ds_read_b128") >= 16 and count(ins, "ds_read_b64_tr_b16") == 0, name
            assert len([i for i in ins if i.startswith("buffer_load_dwordx4") and " lds" in i]) >= 16, name
        elif name.startswith(("maize_gemm_e4m3", "maize_gemm_e5m2")) and "_t128_" in name:
            # 8-bit operands on 128 x 128 tiles: two K steps of 16 MFMAs per trip (B's fragments alternate between two register sets)
            f8 = [i for i in ins if i.startswith("v_mfma_f32_16x16x128_f8f6f4")]
            assert len(f8) == 32 and count(ins, "v_mfma") == 32, name
            tag = name[len("maize_gemm_"):].split("_")[0]
            a_e5m2, b_e5m2 = {"e4m3": (0, 0), "e5m2": (1, 1), "e4m3e5m2": (0, 1), "e5m2e4m3": (1, 0)}[tag]
            assert all(("cbsz:1" in i) == bool(b_e5m2) and ("blgp:1" in i) == bool(a_e5m2) for i in f8), name
            idx = [k for k, i in enumerate(ins) if i.startswith("v_mfma")]
            body = ins[idx[0]:idx[-1] + 1]
            if name.endswith("_nn"):      # B stored K x N: four transposing 64-bit reads per fragment of B
                assert count(body, "ds_read_b128") == 16 and count(body, "ds_read_b64_tr_b8") == 32, name
            else:
                assert count(body, "ds_read_b128") == 32 and count(body, "ds_read_b64_tr_b8") == 0, name
            assert count(body, "buffer_load_dwordx4") == 16 and count(body, "s_barrier") == 2, name
            assert sum(1 for i in body if i.startswith("s_waitcnt") and "vmcnt(16)" in i) == 2, name
            moves = [i for i in body if i.startswith(("v_mov", "v_accvgpr", "v_perm", "v_pk_", "v_lshl", "v_bfi", "v_alignbit"))]
            assert not moves, (name, moves[:5])                               # (no move of a fragment between its read and its MFMA)
        elif name.startswith(("maize_gemm_e4m3", "maize_gemm_e5m2")):
            # 8-bit operands: the 128-deep 16 x 16 instruction (cheaper per multiply-add at the power limit than 32 x 32 x 64).
            # B is fed as the first source, so cbsz carries B's format code and blgp A's (E4M3 = 0 is not printed, E5M2 = 1).
            f8 = [i for i in ins if i.startswith("v_mfma_f32_16x16x128_f8f6f4")]
            h128 = "_h128" in name                                            # 128 x 256 tiles: half the MFMAs, one A group
            stages = 3 if "_h128r3" in name else 2                            # K steps per trip of the loop = ring stages
            # 128-row tiles, and 256-row tiles with the general epilogue (alpha / beta, fp32 C, K ranges): the steps a count that is
            # no multiple of the trip leaves over have copies of their own behind the loop
            peeled = h128 or name.endswith(("_gen", "_splitk"))
            steps = stages + (stages - 1 if peeled else 0)
            per = (32 if h128 else 64) * steps
            assert len(f8) == per and count(ins, "v_mfma") == per, name       # unrolled K steps of 128 elements, 64 (32) MFMAs each
            tag = name[len("maize_gemm_"):].split("_")[0]
            a_e5m2, b_e5m2 = {"e4m3": (0, 0), "e5m2": (1, 1), "e4m3e5m2": (0, 1), "e5m2e4m3": (1, 0)}[tag]
            assert all(("cbsz:1" in i) == bool(b_e5m2) and ("blgp:1" in i) == bool(a_e5m2) for i in f8), name
            # the loop proper: from the first matrix instruction to the last one of a trip (what follows are the left-over
            # steps' copies and the epilogue, in whatever order the compiler lays the blocks out)
            at = [k for k, i in enumerate(ins) if i.startswith("v_mfma")]
            body = ins[at[0]:at[(32 if h128 else 64) * stages - 1] + 1]
            if "_mt256_nn" in name:
                # row-major B: A by 128-bit reads, B by four transposing 8-byte reads per fragment
                assert count(body, "ds_read_b128") == (8 * stages if h128 else 32) and count(body, "ds_read_b64_tr_b8") == 32 * stages, name
            else:
                assert count(body, "ds_read_b128") == (24 * stages if h128 else 64) and count(body, "ds_read_b64_tr_b8") == 0, name
            assert count(body, "buffer_load_dwordx4") == (12 * stages if h128 else 32) and count(body, "s_barrier") == stages, name
            assert sum(1 for i in body if i.startswith("s_waitcnt") and "vmcnt(12)" in i) == (3 if stages == 3 else 0), name
            assert count(body, "v_accvgpr") == 0 and count(body, "v_mov_b32") == 0, name     # accumulators and fragments stay in place
        elif "_mt128_" in name:
            # the catalogue's tf32 and f64 entries: full fp32 / fp64 matrix instructions; one K tile of 128 bytes
            # per row (8 or 4 steps of 16 MFMAs), in the 128-bit and in the element-wise version of the loop
            want = "v_mfma_f64_16x16x4_f64" if "_f64_" in name else "v_mfma_f32_16x16x4_f32"
            per_tile = 64 if "_f64_" in name else 128
            assert count(ins, want) == 2 * per_tile and count(ins, "v_mfma") == 2 * per_tile, name
            assert count(ins, "buffer_load_dwordx4") >= 16, name      # operands by buffer loads (range-checked edges), two tiles' worth
        elif name.startswith("maize_gemm_bf16_skinny_nn"):
            groups = {"maize_gemm_bf16_skinny_nn": 1, "maize_gemm_bf16_skinny_nn_m32": 2, "maize_gemm_bf16_skinny_nn_m64": 4}[name]
            # 8 turns of the ring x 2 column groups x row groups
            assert count(ins, "v_mfma_f32_16x16x32_bf16") >= 16 * groups and count(ins, "v_mfma_f32_16x16x32_f16") >= 16 * groups
        elif name == "maize_gemm_bf16_wave32":
            assert count(ins, "v_mfma_f32_32x32x16_bf16") >= 1 and count(ins, "v_mfma_f32_32x32x16_f16") >= 1


def test_the_register_only_loops_are_nothing_but_matrix_instructions(kernels):
    """The loops bench.py times as the box's ceiling: 16 independent matrix instructions per round and a branch, no
    loads, no LDS, no moves between the register files."""
    for name, mnemonic in (("maize_probe_mfma_loop_16x16x32", "v_mfma_f32_16x16x32_bf16"),
                           ("maize_probe_mfma_loop_16x16x128_e4m3", "v_mfma_f32_16x16x128_f8f6f4")):
        ins = kernels[name]
        first = next(i for i, x in enumerate(ins) if x.startswith(mnemonic))
        last = max(i for i, x in enumerate(ins) if x.startswith(mnemonic))
        loop = ins[first:last + 1]
        assert len(loop) == 16 and all(x.startswith(mnemonic) for x in loop), (name, loop)
        assert "cbsz" not in " ".join(loop) and "blgp" not in " ".join(loop), name          # E4M3 on both sides
        assert len({x.split()[1].rstrip(",") for x in loop}) == 16, name                    # 16 different accumulators
        back = next(x for x in ins[last + 1:] if x.startswith("s_cbranch"))
        assert back.startswith("s_cbranch_scc"), name
        between = ins[last + 1:ins.index(back, last + 1)]
        assert all(x.startswith(("s_add", "s_sub", "s_cmp")) for x in between), (name, between)


def test_data_movement_the_design_rests_on(kernels):
    for name, ins in kernels.items():
        if "_mt256_" in name or name.startswith("maize_gemm_bf16_skinny_nn"):
            lds_dma = [i for i in ins if i.startswith("buffer_load_dwordx4") and " lds" in i]
            assert len(lds_dma) >= 16, f"{name}: operands must reach LDS by 128-bit direct-to-LDS loads"
            fp32_staging = "_gen" in name or "_splitk" in name
            assert count(ins, "ds_write_b128") == 0 or fp32_staging, name   # no register round trip for operands
        if "_mt256_nn" in name or name.startswith("maize_gemm_bf16_skinny_nn"):
            tr = "ds_read_b64_tr_b8" if name.startswith(("maize_gemm_e4m3", "maize_gemm_e5m2")) else "ds_read_b64_tr_b16"
            assert count(ins, tr) >= 8, f"{name}: a row-major K x N B is read with transposing reads"
        if "_mt256_nt" in name:
            assert count(ins, "ds_read_b64_tr_b16") == 0 and count(ins, "ds_read_b128") >= 16, name
    plain = kernels["maize_gemm_bf16_mt256_nn"]
    assert any(i.startswith("buffer_store_dwordx4") and i.rstrip().endswith("nt") for i in plain), "non-temporal C stores"
    assert count(plain, "v_cvt_pk_bf16_f32") >= 128


def test_nothing_that_must_not_be_there(kernels):
    for name, ins in kernels.items():
        assert count(ins, "scratch_") == 0, f"{name} spills to scratch"
        # writes through the scalar data cache: scalar memory stores and atomics, its write-back (names assembled
        # here so that this checker does not itself contain them)
        scalar_writes = tuple("s_" + x for x in ("sto" + "re", "buffer_" + "sto" + "re", "ato" + "mic", "buffer_" + "ato" + "mic", "dcache_" + "wb"))
        assert not any(i.startswith(scalar_writes) for i in ins), f"{name} writes through the scalar cache"
        for banned in ("v_pk_add_f32", "v_pk_mul_f32", "v_pk_fma_f32"):
            assert count(ins, banned) == 0, f"{name} contains {banned}"


def test_main_loop_of_the_headline_kernel_is_lean(kernels):
    """Between the first and the last MFMA of the plain kernels' unrolled K loop nothing but matrix
    instructions, LDS reads, direct-to-LDS loads, waits, barriers and scalar bookkeeping may appear."""
    for name, reads in (("maize_gemm_bf16_mt256_nn", {"ds_read_b128": 32, "ds_read_b64_tr_b16": 64}),
                        ("maize_gemm_bf16_mt256_nt", {"ds_read_b128": 64})):
        ins = kernels[name]
        idx = [k for k, i in enumerate(ins) if i.startswith("v_mfma")]
        assert len(idx) == 256
        body = ins[idx[0]:idx[-1] + 1]                                 # the K loop: two unrolled steps
        allowed = ("v_mfma", "ds_read", "buffer_load_dwordx4", "s_")
        extra = [i for i in body if not i.startswith(allowed)]
        assert not extra, extra[:5]                                    # no vector ALU work at all: in particular no accumulator moves
        assert len(body) <= 500
        for mnemonic, n in reads.items():
            assert count(body, mnemonic) == n, (name, mnemonic)        # every fragment is read once per K step
        assert count(body, "buffer_load_dwordx4") == 32                # 16 pieces of 1 KiB per wave and K step
        assert count(body, "s_barrier") == 2
        assert count(body, "s_waitcnt") <= 16                          # one per eighth of a K step, placed by hand


def test_main_loop_of_the_half_height_kernels_is_lean(kernels):
    """The 128 x 256 tile kernels: two unrolled K steps of 64 MFMAs per wave, one A group (8 reads per step) and two
    B groups (16 reads, or 32 transposing ones), 12 pieces per wave and step, one barrier per step; behind the loop one more
    copy of the step for an odd step count."""
    for name, reads in (("maize_gemm_bf16_mt256_nn_h128", {"ds_read_b128": 16, "ds_read_b64_tr_b16": 64}),
                        ("maize_gemm_bf16_mt256_nt_h128", {"ds_read_b128": 48})):
        ins = kernels[name]
        idx = [k for k, i in enumerate(ins) if i.startswith("v_mfma")]
        assert len(idx) == 192 and count(ins, "v_mfma_f32_16x16x32_bf16") == 192
        body = ins[idx[0]:idx[127] + 1]                                # the loop proper: the first two steps
        # (the row-major B's descriptor is re-based per K tile and cut at 2 GiB: the compiler does that one 64-bit compare,
        # for which there is no scalar instruction, on the vector unit -- one uniform compare per K step)
        extra = [i for i in body if not i.startswith(("v_mfma", "ds_read", "buffer_load_dwordx4", "s_", "v_cmp_lt_u64"))]
        assert not extra and count(body, "v_cmp_lt_u64") <= 2, extra[:5]
        for mnemonic, n in reads.items():
            assert count(body, mnemonic) == n, (name, mnemonic)
        assert count(body, "buffer_load_dwordx4") == 24 and count(body, "s_barrier") == 2
        assert count(body, "s_waitcnt") <= 8
    for name in ("maize_gemm_bf16_mt256_nn_h128_gen", "maize_gemm_f16_mt256_nt_h128_gen", "maize_gemm_bf16_mt256_nt_h128_splitk", "maize_gemm_f16_mt256_nn_h128_splitk"):
        want = "v_mfma_f32_16x16x32_f16" if "_f16_" in name else "v_mfma_f32_16x16x32_bf16"
        assert count(kernels[name], want) == 192 and count(kernels[name], "v_mfma") == 192, name


def test_main_loop_of_the_three_stage_kernels_is_lean(kernels):
    """The 128 x 256 tile kernels with three ring stages: three unrolled K steps of 64 MFMAs, the same reads and requests
    per step as the two-stage loop, one barrier per step, and a counted wait that leaves twelve requests in flight; behind
    the loop two more copies of the step for a step count that is no multiple of three."""
    for name, reads in (("maize_gemm_bf16_mt256_nn_h128r3", {"ds_read_b128": 24, "ds_read_b64_tr_b16": 96}),
                        ("maize_gemm_bf16_mt256_nt_h128r3", {"ds_read_b128": 72})):
        ins = kernels[name]
        idx = [k for k, i in enumerate(ins) if i.startswith("v_mfma")]
        assert len(idx) == 320 and count(ins, "v_mfma_f32_16x16x32_bf16") == 320
        body = ins[idx[0]:idx[191] + 1]                                # the loop proper: the first three steps
        extra = [i for i in body if not i.startswith(("v_mfma", "ds_read", "buffer_load_dwordx4", "s_", "v_cmp_lt_u64"))]
        assert not extra and count(body, "v_cmp_lt_u64") <= 3, extra[:5]
        for mnemonic, n in reads.items():
            assert count(body, mnemonic) == n, (name, mnemonic)
        assert count(body, "buffer_load_dwordx4") == 36 and count(body, "s_barrier") == 3
        assert count(body, "s_waitcnt") <= 12
        assert sum(1 for i in body if i.startswith("s_waitcnt") and "vmcnt(12)" in i) == 3, name
    for name in ("maize_gemm_bf16_mt256_nn_h128r3_gen", "maize_gemm_f16_mt256_nt_h128r3_gen", "maize_gemm_f16_mt256_nn_h128r3_gen", "maize_gemm_bf16_mt256_nt_h128r3_gen"):
        want = "v_mfma_f32_16x16x32_f16" if "_f16_" in name else "v_mfma_f32_16x16x32_bf16"
        assert count(kernels[name], want) == 320 and count(kernels[name], "v_mfma") == 320, name


def test_main_loop_of_the_128_by_128_tile_kernels_is_lean(kernels):
    """The 128 x 128 tile kernels: one K step of 32 MFMAs per wave and trip, 16 128-bit fragment reads (K x N B: 8 and 16
    transposing ones), eight requests, one barrier whose wait leaves sixteen requests in flight.  Between a fragment
    read and the matrix instruction that takes it stands a wait and nothing else: no move of a fragment (the reads
    are assembly statements whose results the compiler believes ready at once; a move would copy them early)."""
    for name, reads in (("maize_gemm_bf16_t128_nn", {"ds_read_b128": 8, "ds_read_b64_tr_b16": 16}), ("maize_gemm_bf16_t128_nt", {"ds_read_b128": 16}),
                        ("maize_gemm_f16_t128_nn", {"ds_read_b128": 8, "ds_read_b64_tr_b16": 16}), ("maize_gemm_f16_t128_nt", {"ds_read_b128": 16})):
        ins = kernels[name]
        idx = [k for k, i in enumerate(ins) if i.startswith("v_mfma")]
        assert len(idx) == 32 and count(ins, "v_mfma_f32_16x16x32_f16" if "_f16_" in name else "v_mfma_f32_16x16x32_bf16") == 32, name
        body = ins[idx[0]:idx[-1] + 1]
        for mnemonic, n in reads.items():
            assert count(body, mnemonic) == n, (name, mnemonic)               # (one, or two transposing ones, behind each of a half's first MFMAs)
        assert count(body, "buffer_load_dwordx4") == 8 and count(body, "s_barrier") == 1
        assert sum(1 for i in body if i.startswith("s_waitcnt") and "vmcnt(16)" in i) == 1, name
        moves = [i for i in body if i.startswith(("v_mov", "v_accvgpr", "v_perm", "v_pk_", "v_lshl", "v_bfi", "v_and", "v_alignbit"))]
        assert not moves, (name, moves[:5])
        vector = [i for i in body if i.startswith("v_") and not i.startswith(("v_mfma", "v_add_u32", "v_or_b32", "v_cmp_lt_u64"))]
        assert not vector, (name, vector[:5])                                   # (the reads' addresses: ring stage added to the lane's base)



def test_no_k_loop_wraps_its_requests_in_scalarising_loops(kernels):
    """A buffer descriptor that the compiler carries in vector registers makes it wrap every request in a loop that
    reads the descriptor back lane by lane (v_readfirstlane / s_and_saveexec / s_cbranch_execnz): the general-epilogue
    and split-K kernels on a row-major 16-bit B had sixteen of those per pair of K steps (and a branch around the odd-N
    fix-up), 8-22 % of their run time.  Every macro-tile K loop is one basic block: no exec-mask juggling, no branch
    between its first and its last matrix instruction other than the loop's own, a handful of readfirstlanes at most
    (the descriptor of a K x N B, said once per K tile).  And no descriptor word is sign-extended on its way."""
    for name, ins in kernels.items():
        if "_mt256_" not in name or name.endswith("_edge"):       # (the edge kernels hold three loops, checked by their own test)
            continue
        idx = [k for k, i in enumerate(ins) if i.startswith("v_mfma")]
        body = ins[idx[0]:idx[-1] + 1]
        # (the 128-row kernels: behind the loop come one or two more copies of the step for the steps a trip leaves over, each
        # under a uniform branch of its own, and the epilogue may be laid out among them)
        h128 = "_h128" in name
        peeled = h128 or name.endswith(("_gen", "_splitk"))
        trip = (32 if name.startswith(("maize_gemm_e4m3", "maize_gemm_e5m2")) else 64) * (1 if h128 else 2) * (3 if "_h128r3" in name else 2)
        loop = ins[idx[0]:idx[trip - 1] + 1] if peeled else body
        assert count(loop, "s_and_saveexec") == 0 and count(loop, "s_cbranch_exec") == 0, name
        assert count(loop, "v_readfirstlane") <= 12, (name, count(loop, "v_readfirstlane"))
        assert count(loop, "s_cbranch") <= 1, name
        if peeled:
            copies = 5 if "_h128r3" in name else 3
            assert count(body, "v_readfirstlane") <= 4 * copies + 4 and count(body, "s_and_saveexec") <= 2, name
        assert count(ins, "s_bfe_i64") == 0, name
