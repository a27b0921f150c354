"""The no-allocation entry point under HIP graph capture (maize_amd/csrc/graph_replay.cpp, a C++ caller linked against
the library and the HIP runtime): a chain of six products -- five of which pass partial tiles and ticket counters through
the fixed per-GPU scratch array -- is captured once on the caller's stream and replayed with new inputs, eager launches
of the same chain in between.  Every replay must equal the eager results of the same inputs bit for bit."""
import json
import os
import subprocess
import sys

import pytest

import maize_amd as mz

pytestmark = pytest.mark.gpu
EXE = os.path.join(os.path.dirname(mz.LIB_PATH), "maize_graph_replay")


def test_noalloc_chain_replayed_from_a_graph():
    assert os.path.exists(EXE), f"{EXE} is missing: run make -C maize_amd/csrc"
    print("graph capture: maize_graph_replay 6", flush=True)
    sys.stdout.flush()
    out = subprocess.run([EXE, "6"], capture_output=True, text=True, timeout=240)
    assert out.returncode == 0, out.stderr + out.stdout
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    print(rec, flush=True)
    assert rec["mismatches"] == 0 and rec["rounds"] == 6
    assert rec["products"] == 6 and rec["with_scratch"] >= 5
    # one kernel node per launch: the split-K chain is two launches (first pass + reduce pass), nothing else is recorded
    assert rec["products"] <= rec["graph_nodes"] <= rec["products"] + 2
    families = " ".join(rec["kernels"])
    for part in ("skinny_nn", "skinny_nt", "skinny_nn_m64", "h128_splitk", "_edge"):
        assert part in families, (part, families)
