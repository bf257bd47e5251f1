"""CPU: host-side logic of the package that needs no device."""
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from tscale_amd.attention import alibi_layer_schedule

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("wide", [1024, 4096])
def test_layer_schedule_matches_the_oracle(wide):
    # the oracle's schedule is itself pinned against the reference-built InitModelDescr
    for depth in list(range(1, 41)) + [64, 96]:
        w, s = orc.init_alibi(depth, wide)
        got = alibi_layer_schedule(depth, wide)
        assert [g[0] for g in got] == w.tolist(), depth
        assert np.allclose([g[1] for g in got], s), depth


def test_layer_schedule_of_the_documented_models():
    # 12 layers: one pair of width-1 layers, then 5 x (64 with slope 0.5, wide)
    sched = alibi_layer_schedule(12, 1024)
    assert sched[:2] == [(1, 0.0), (1, 0.0)] and sched[2:4] == [(64, 0.5), (1024, 0.0)] and len(sched) == 12
    # 24 layers: two leading pairs of width 1, ten alternating pairs
    sched = alibi_layer_schedule(24, 2048)
    assert [w for w, _ in sched].count(1) == 4 and [w for w, _ in sched].count(64) == 10 and len(sched) == 24


def test_prefill_workgroup_mapping_visits_every_head_and_tile_once(tmp_path):
    """tests/cpp/test_wg_map.cpp walks the launch mapping of tscale_amd/csrc/wg_map.h (the code the kernel runs) over
    ~1500 launch shapes on the CPU, divisors of 1 (one query tile, one sequence, one unit per group) included."""
    import subprocess
    exe = tmp_path / "test_wg_map"
    subprocess.run(["g++", "-O2", "-std=c++17", "-o", str(exe), os.path.join(ROOT, "tests", "cpp", "test_wg_map.cpp")], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    assert r.stdout.startswith("OK")
