"""The C-ABI library loads and exports every symbol the public header declares (no GPU needed)."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", name) for name in ("mts_moe.h", "mts_probe.h")]


def test_every_public_header_is_covered():
    assert sorted(os.listdir(os.path.join(ROOT, "include"))) == sorted(os.path.basename(h) for h in HEADERS)


def _declared():
    text = "".join(open(h).read() for h in HEADERS)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mts_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    for must in ("mts_router_fwd", "mts_router_bwd", "mts_moe_route", "mts_moe_fwd_gateup_swiglu", "mts_moe_fwd_down", "mts_moe_fwd_gateup_down",
                 "mts_moe_combine", "mts_moe_bwd_dy1", "mts_moe_bwd_dx", "mts_moe_bwd_dw1", "mts_moe_bwd_dw2",
                 "mts_moe_bwd_joint"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from minitrain_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = _lib.load()
    for name in _declared():
        assert hasattr(lib, name), f"{name} is declared in include/ but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes prototype"
    assert lib.mts_version() == 4
    assert lib.mts_error_string(0) == b"ok"
    # argument checks run on the host before any launch: safe without a GPU
    assert lib.mts_router_fwd(None, 4, 8, 2, 1, None, None, None, None, None, None, None, None, None, 0, None, 0, None) == -1
    assert lib.mts_moe_route_workspace_bytes(24576, 2, 8) == 192 * 8 * 4
    assert lib.mts_moe_ds_partials(1024) > 0


def test_contract_violations_are_reported_before_any_launch():
    """Argument checks of the newer entry points run on the host: every call here returns a negative
    MTS_ERR_* code without touching a GPU."""
    from minitrain_amd import _lib

    lib = _lib.load()
    NULL, SHAPE, WORKSPACE = -1, -2, -4
    fake = 4096   # any non-null, 16-byte aligned value: nothing is dereferenced before the checks fail
    # gate/up + down as one launch: required pointers, the shapes it exists for, workspace size
    BF16, F32 = 0, 1
    assert lib.mts_moe_fwd_joint_supported(BF16, 768, 1024) == 1
    assert lib.mts_moe_fwd_joint_supported(BF16, 768, 1000) == 0      # I not a multiple of 64
    assert lib.mts_moe_fwd_joint_supported(BF16, 4096, 14336) == 0    # an expert's W1 beyond an L2: the two launches
    assert lib.mts_moe_fwd_joint_supported(F32, 768, 1024) == 0
    need = lib.mts_moe_fwd_joint_workspace_bytes(49152, 8)
    assert need % 16 == 0 and need >= (2 * (49152 // 256 + 7) + 1) * 4
    args = lambda **kw: [kw.get(k, v) for k, v in dict(x=fake, w1=fake, w2=fake, x_gather=fake, expert_start=fake, weights=fake,
                                                         s_scatter=fake, T=24576, K=2, E=8, H=768, I=1024, act=BF16, pre=fake,
                                                         post=fake, y=fake, ws=fake, ws_bytes=need, stream=None).items()]
    assert lib.mts_moe_fwd_gateup_down(*args(ws=None)) == NULL
    assert lib.mts_moe_fwd_gateup_down(*args(w2=None)) == NULL
    assert lib.mts_moe_fwd_gateup_down(*args(s_scatter=None)) == NULL     # the routing weight needs the row -> entry map
    assert lib.mts_moe_fwd_gateup_down(*args(I=1000)) == SHAPE
    assert lib.mts_moe_fwd_gateup_down(*args(ws_bytes=need - 16)) == WORKSPACE
    assert lib.mts_moe_fwd_gateup_down(*args(act=F32)) == -3
    assert lib.mts_moe_fwd_gateup_down(*args(y=fake + 4)) == -5
    # capacity mask: required pointers, expert limit, workspace size
    assert lib.mts_moe_capacity_mask(None, fake, 8, 2, 4, 3, fake, None, fake, fake, 1 << 20, None) == NULL
    assert lib.mts_moe_capacity_mask(fake, fake, 8, 2, 4096, 3, fake, None, fake, fake, 1 << 20, None) == SHAPE
    assert lib.mts_moe_capacity_mask(fake, fake, 8, 2, 4, 3, fake, None, fake, fake, 16, None) == WORKSPACE
    assert lib.mts_moe_capacity_workspace_bytes(24576, 2, 8) >= 4 * 49152 * 4
    # weight layout of the backward GEMMs
    assert lib.mts_moe_bwd_weights_as_stored(_lib.MTS_BF16, 768, 1024) == 1
    assert lib.mts_moe_bwd_weights_as_stored(_lib.MTS_F16, 768, 1024) == 1
    assert lib.mts_moe_bwd_weights_as_stored(_lib.MTS_F32, 768, 1024) == 0      # fp32 path reads transposed copies
    assert lib.mts_moe_bwd_weights_as_stored(_lib.MTS_BF16, 72, 40) == 0        # no whole 64-wide k-tiles
    assert lib.mts_moe_bwd_dx(fake, fake, 1, fake, 512, 4, 64, 128, _lib.MTS_F32, fake, None) == SHAPE
    assert lib.mts_moe_bwd_dx(fake, fake, 1, fake, 512, 4, 72, 40, _lib.MTS_BF16, fake, None) == SHAPE
    # row-chunk workspace of the weight-gradient GEMMs: 2E slots of 256x256 fp32 tiles
    assert lib.mts_moe_bwd_dw_workspace_bytes(1, 8, 768, 1024) == 2 * 8 * (8 * 3) * 256 * 256 * 4
    assert lib.mts_moe_bwd_dw_workspace_bytes(2, 8, 768, 1024) == 2 * 8 * (3 * 4) * 256 * 256 * 4
    assert lib.mts_moe_bwd_dw1(fake, fake, fake, fake, 256, 2, 4, 64, 128, _lib.MTS_BF16, _lib.MTS_BF16, fake, fake, 16,
                               None) == WORKSPACE
    # dW1 + dW2 + dX + dS as one launch: 16-bit activations with whole 64-wide k-tiles of 2I only
    assert lib.mts_moe_bwd_joint_supported(_lib.MTS_BF16, 768, 1024) == 1
    assert lib.mts_moe_bwd_joint_supported(_lib.MTS_F16, 64, 128) == 1
    assert lib.mts_moe_bwd_joint_supported(_lib.MTS_F32, 768, 1024) == 0
    assert lib.mts_moe_bwd_joint_supported(_lib.MTS_BF16, 72, 40) == 0
    joint = lambda *a: lib.mts_moe_bwd_joint(*a)
    ok_args = [fake] * 9 + [256, 2, 4, 64, 128, _lib.MTS_BF16, _lib.MTS_BF16, fake, fake, fake, fake, None, 0, None, 0, None, None]
    assert joint(*([None] + ok_args[1:])) == NULL
    assert joint(*(ok_args[:14] + [_lib.MTS_F32] + ok_args[15:])) == -3                      # activations must be 16-bit
    assert joint(*(ok_args[:12] + [72, 40] + ok_args[14:])) == SHAPE                          # 2I = 80 has no whole k-tile
    assert joint(*(ok_args[:20] + [fake, 16] + ok_args[22:])) == WORKSPACE
    # without d_w2 the joint launch leaves dW2 to a call of its own: weighted_act and the second workspace may be absent
    # too (the next check that fails is the unsupported width, not a missing pointer)
    no_dw2 = ok_args[:1] + [None] + ok_args[2:12] + [72, 40] + ok_args[14:18] + [None] + ok_args[19:]
    assert joint(*no_dw2) == SHAPE
    # the schedule of the joint launch covers up to 32 experts; dO*W2 refuses to write one beyond that
    assert lib.mts_moe_bwd_schedule_bytes(8) == 4096 and lib.mts_moe_bwd_schedule_bytes(32) == 4096
    assert lib.mts_moe_bwd_schedule_bytes(33) == 0 and lib.mts_moe_bwd_schedule_bytes(0) == 0
    assert lib.mts_moe_bwd_schedule(None, 1024, 8, fake, None) == NULL
    assert lib.mts_moe_bwd_schedule(fake, 1024, 33, fake, None) == SHAPE
    assert lib.mts_moe_bwd_schedule(fake, 1024, 8, fake + 4, None) == -5
    assert lib.mts_moe_bwd_dy1(fake, fake, 1, fake, fake, fake, fake, fake, 256, 2, 40, 64, 128, _lib.MTS_BF16, fake, None, fake,
                               fake, None) == SHAPE
    # the MFMA rate probe: sink pointer, launch size, sink size
    assert lib.mts_probe_mfma_sink_bytes(512) == 512 * 256 * 4
    assert lib.mts_probe_mfma_rate(1, 512, 100, None, 1 << 20, None, None) == NULL
    assert lib.mts_probe_mfma_rate(1, 0, 100, fake, 1 << 20, None, None) == SHAPE
    assert lib.mts_probe_mfma_rate(1, 512, 100, fake, 16, None, None) == WORKSPACE
    # unknown element type
    assert lib.mts_moe_combine(fake, None, None, fake, 8, 2, 64, 7, fake, None) == -3


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from minitrain_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.MtsError):
        _lib.load()


def test_cpu_tensors_are_rejected_not_served_by_a_fallback():
    import torch

    from minitrain_amd.model.ops import get_ops_backend

    ops = get_ops_backend("hip")
    with pytest.raises(RuntimeError):
        ops.router_postprocess(torch.zeros(4, 8), 2, normalize=True)
    with pytest.raises(RuntimeError):
        ops.fused_moe(torch.zeros(4, 8, dtype=torch.bfloat16), torch.zeros(2, 16, 8, dtype=torch.bfloat16),
                      torch.zeros(2, 8, 8, dtype=torch.bfloat16), torch.zeros(4, 1, dtype=torch.int32),
                      torch.zeros(4, 1, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        get_ops_backend("triton")


def test_bench_refuses_more_than_one_gpu_and_a_missing_gpu():
    """bench.py measures one GPU: `--gpus 2` (or a multi-rank launch) exits with a message, and without
    a GPU it exits instead of timing a CPU path."""
    import subprocess
    import sys
    from pathlib import Path

    bench = str(Path(__file__).resolve().parents[1] / "bench.py")
    two = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert two.returncode == 2 and "one GPU" in two.stderr and two.stdout.strip() == ""
    import torch

    if not torch.cuda.is_available():
        one = subprocess.run([sys.executable, bench, "--steps", "1", "--warmup", "0"], capture_output=True, text=True,
                             timeout=300)
        assert one.returncode == 2 and "needs a GPU" in one.stderr and one.stdout.strip() == ""


def test_bench_names_a_committed_file_for_its_counter_derived_traffic():
    """`roofline.traffic` in the bench line is not measured live: the line names the file that holds the
    counter runs it comes from, and every stage with such a figure appears in that file."""
    import sys

    sys.path.insert(0, ROOT)
    import bench

    path = os.path.join(ROOT, bench.TRAFFIC_SOURCE)
    assert os.path.isfile(path)
    text = open(path).read()
    assert "FETCH_SIZE" in text and "WRITE_SIZE" in text
    for stage in bench.MEASURED_TRAFFIC_BYTES:
        assert stage in text, stage
