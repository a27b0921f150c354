"""The LDS index maps the kernels are compiled from (maize_amd/csrc/kernels/maps.hpp), checked on the host.

The reference proves its tile/fragment maps by emulating them on the CPU (SmemTile / MatrixFragment index
arithmetic, crates/maize_tile/src/smem/smem_tile.rs and crates/maize_tile/src/reg/mod.rs); here the maps are
constexpr functions shared by device and host, and tests/cpu/check_maps.cpp enumerates them: every
direct-to-LDS piece deposits each (row, chunk) of a tile exactly once where the fragment reads expect it, the
transposing reads hand every lane the operand element the matrix instruction wants, and every wave-wide LDS
access of the K loops and of the epilogue is free of bank conflicts.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs a host C++ compiler")
def test_lds_maps_by_enumeration(tmp_path):
    exe = tmp_path / "check_maps"
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-Werror",
                    "-I", os.path.join(ROOT, "maize_amd", "csrc", "kernels"),
                    "-o", str(exe), os.path.join(ROOT, "tests", "cpu", "check_maps.cpp")], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all LDS maps check out" in r.stdout
    assert r.stdout.count("ok  ") == 11


def test_kernels_use_the_shared_maps():
    # the kernels must not carry private copies of the swizzles the checker proves
    for name in ("gemm_mt256.hpp", "gemm_skinny.hpp", "gemm_skinny_nt.hpp"):
        src = open(os.path.join(ROOT, "maize_amd", "csrc", "kernels", name)).read()
        assert '#include "maps.hpp"' in src
        assert "maps::" in src
