"""Every tile shape and block order the library can be told to use gives the layer step the default ones give.

The defaults are picked for speed; the others stay reachable through environment overrides (tuning runs) and
through shapes that rule the default out, so they are held to the same results: each configuration runs the
layer step of two shapes in a child process (the overrides are read once per process) and is compared with
this process's default run, tensor by tensor."""

import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parents[1]

CONFIGURATIONS = {
    "ring blocks everywhere": dict(MTS_TILE_GATEUP="1", MTS_TILE_DOWN="1", MTS_TILE_DY1="1", MTS_TILE_DX="1",
                                   MTS_NO_JOINT_BWD="1"),
    "staged kernels, separate launches": dict(MTS_TILE_GATEUP="0", MTS_TILE_DOWN="0", MTS_TILE_DY1="0", MTS_TILE_DX="0",
                                              MTS_TILE_DW1="0", MTS_TILE_DW2="0", MTS_NO_JOINT_BWD="1", MTS_NO_OVERLAP="1"),
    "specialised waves for dY1, round-robin tiles": dict(MTS_TILE_DY1="2", MTS_XCD_RANGES="0", MTS_NO_TILE_ORDER="1"),
    "four stages of 32-wide k-tiles, separate launches": dict(MTS_TILE_GATEUP="2", MTS_TILE_DOWN="2", MTS_TILE_DX="2",
                                                              MTS_TILE_DW1="2", MTS_TILE_DW2="2", MTS_NO_JOINT_BWD="1"),
    "64-wide k-tiles for dX and the weight gradients on their own, every tile whole": dict(MTS_NO_JOINT_BWD="1",
                                                                                           MTS_NO_TAIL_SPLIT="1"),
    "router projection on the vector pipe": dict(MTS_NO_MFMA_ROUTER="1"),
    "gate/up and down as two launches": dict(MTS_NO_JOINT_FWD="1"),
    "gate/up and down as one launch, every down tile whole": dict(MTS_FWD_JOINT_TAIL="0"),
    "gate/up and down as one launch, every down tile cut in two": dict(MTS_FWD_JOINT_TAIL="1000"),
    "ranges per XCD, plain order, tail launches apart": dict(MTS_XCD_RANGES="1", MTS_NO_TILE_ORDER="1",
                                                             MTS_NO_TAIL_IN_JOINT="1"),
}


@pytest.fixture(scope="module")
def default_run():
    sys.path.insert(0, str(ROOT / "tests"))
    import tile_choice_child as child

    results = {}
    for shape in child.SHAPES:
        results.update(child.layer_step(shape))
    return results


@pytest.mark.parametrize("name", list(CONFIGURATIONS))
def test_tile_choice_gives_the_default_results(name, default_run, tmp_path):
    print(f"tile choices: {name}", flush=True)
    env = dict(os.environ)
    env.update(CONFIGURATIONS[name])
    target = tmp_path / "step.npz"
    run = subprocess.run([sys.executable, str(ROOT / "tests" / "tile_choice_child.py"), str(target)], env=env,
                         capture_output=True, text=True, timeout=300, cwd=str(ROOT))
    assert run.returncode == 0, run.stderr[-2000:]
    got = np.load(target)
    assert set(got.files) == set(default_run)
    for key, want in default_run.items():
        # the same products summed in fp32; the order of the sums may differ between tile shapes (row chunks of
        # the weight gradients), the 16-bit rounding of the results does not hide more than one step of it
        scale = float(np.abs(want).max()) or 1.0
        assert float(np.abs(got[key] - want).max()) <= 1e-2 * scale, (name, key)
        assert float(np.linalg.norm(got[key] - want)) <= 2e-3 * float(np.linalg.norm(want)) + 1e-12, (name, key)
