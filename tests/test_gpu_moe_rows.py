"""The operator benchmark rows in the reference's schema (benchmarks/operators/measurement.py:25-38,
485-496; moe_runner.py:53,176-193) and the decoder training step at its real size (config 5)."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

TIMING = ("fwd_p50_ms", "fwd_p95_ms", "bwd_p50_ms", "bwd_p95_ms", "full_p50_ms", "full_p95_ms")
MEMORY = ("fwd_peak_mem_mb", "bwd_peak_mem_mb", "full_peak_mem_mb")
PARITY = ("max_abs", "max_rel", "relative_l2", "cosine_similarity")


@pytest.mark.parametrize("tokens,zipf,capacity_factor", [(2048, False, None), (4096, True, 1.0)])
def test_operator_rows_schema_and_acceptance(tokens, zipf, capacity_factor):
    print(f"moe rows tokens={tokens} zipf={zipf} capacity_factor={capacity_factor}", flush=True)
    from minitrain_amd.benchmarks.moe_rows import operator_rows

    rows = operator_rows("layer", tokens, iters=3, warmup=1, seed=1, with_torch=True, zipf=zipf,
                         capacity_factor=capacity_factor)
    by = {r["provider"]: r for r in rows}
    assert set(by) >= {"hip", "torch"}
    for r in rows:
        assert r["op"] == "fused_moe" and r["size"] == tokens and r["dtype"] == "bf16" and r["timer"] == "cuda_events"
        for key in TIMING + MEMORY:
            assert key in r and math.isfinite(r[key]) and r[key] >= 0, (r["provider"], key)
        assert r["fwd_p50_ms"] > 0 and r["full_p50_ms"] >= r["fwd_p50_ms"] * 0.5
    hip = by["hip"]
    for side in ("fwd", "bwd"):
        for key in PARITY:
            assert f"{side}_{key}" in hip
        # the reference's gate for this operator (moe_runner.py:176-193)
        assert hip[f"{side}_relative_l2"] <= 1e-2 and hip[f"{side}_cosine_similarity"] >= 0.9999, hip
        assert hip[f"{side}_correct"] is True
    for m in ("fwd", "bwd", "full"):
        assert hip[f"{m}_speedup"] > 0 and by["torch"][f"{m}_speedup"] == 1.0
    if capacity_factor is not None:
        assert "hip_zero_weight" in by and 0.0 < hip["dropped_route_fraction"] < 1.0
        assert hip["capacity"] == max(4, math.ceil(capacity_factor * tokens * 2 / 8))
        assert all(a <= hip["capacity"] for a in hip["accepted_per_expert"])


def test_decoder_step_at_the_real_size():
    """Config 5: 12 layers, 24 x 1024 tokens, 293 494 272 parameters, bf16 autocast over fp32 parameters,
    AdamW: one warm-up step and two timed ones on one batch; the loss is finite and falls, and the MoE
    blocks report their share of the step."""
    print("decoder step, 12 layers, 24x1024", flush=True)
    from minitrain_amd.train.bench_step import run

    rec = run(layers=12, batch=24, seq=1024, vocab=50257, steps=2, warmup=1, seed=4)
    assert rec["parameters"] == 293_494_272
    losses = rec["losses"]
    assert len(losses) == 3 and all(math.isfinite(v) for v in losses)
    assert losses[0] > math.log(50257) * 0.9            # an untrained model starts near the uniform entropy
    assert losses[-1] < losses[0]
    assert 0.0 < rec["moe_share_of_step"] < 1.0 and rec["moe_ms_per_step"] > 0
    assert rec["value"] > 0 and rec["config"]["layers"] == 12
    torch.cuda.empty_cache()


def test_mfma_rate_probe_reports_a_plausible_rate():
    """The register-only MFMA loop the benchmark line quotes as `mfma_sustained`: every thread's sum is
    finite, the reported FLOPs match the launch, and the rate lies between a fifth of the nominal bf16 peak
    and the peak itself (2.5 PFLOP/s); constant operands are not slower than toggling ones by more than noise."""
    print("mfma rate probe", flush=True)
    import sys
    from pathlib import Path

    sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
    import bench

    rec = bench.mfma_sustained(blocks=512, rounds=200, launches=12, lead=4)
    assert rec["peak"] == 2500.0 and rec["unit"] == "TFLOP/s"
    for key in ("random_operands_tflops", "constant_operands_tflops"):
        assert 500.0 < rec[key] <= 2500.0, rec
    assert rec["constant_operands_tflops"] >= 0.9 * rec["random_operands_tflops"], rec
    from minitrain_amd import _lib

    lib = _lib.load()
    sink = torch.full((64 * 256,), float("nan"), device="cuda")
    assert lib.mts_probe_mfma_rate(1, 64, 4, sink.data_ptr(), sink.numel() * 4, None, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert torch.isfinite(sink).all() and sink.abs().max() > 0


def test_bench_line_carries_the_contract():
    """`python bench.py` prints one JSON line with the metric of the baseline, the roofline of the dominant
    kernel (algorithmic bytes beside the counter-derived traffic and the file that holds the counter runs)
    and the CPU baseline; the fractions follow from the figures in the line."""
    print("bench line", flush=True)
    import json
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    run = subprocess.run([sys.executable, str(root / "bench.py"), "--steps", "3", "--warmup", "1"], capture_output=True,
                         text=True, timeout=600, cwd=str(root))
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [l for l in run.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 3 and rec["warmup"] == 1 and rec["unit"] == "tokens/s"
    assert rec["dtype"] == "bf16" and rec["data"] == "synthetic" and rec["vs_baseline"] is None
    assert rec["config"]["workload"] == "moe_layer_24x1024_d768_e8_top2_ff1024_bf16" and "model" not in rec["config"]
    assert math.isclose(rec["value"], 24576 / (rec["ms_per_step"] * 1e-3), rel_tol=1e-3)
    roof = rec["roofline"]
    assert roof["bound"] in ("hbm", "mfma") and roof["unit"] in ("GB/s", "TFLOP/s")
    assert math.isclose(roof["frac"], roof["achieved"] / roof["peak"], rel_tol=1e-3)
    assert roof["bound"] == ("mfma" if roof["intensity_flop_per_byte"] >= roof["ridge_flop_per_byte"] else "hbm")
    assert roof["traffic"] >= roof["algorithmic_bytes"] > 0 and roof["traffic_source"].startswith("profiles/")
    assert roof["avg_ms"] < rec["ms_per_step"]
    for stage in rec["kernels"]:
        assert stage["bound"] == ("mfma" if stage["intensity_flop_per_byte"] >= roof["ridge_flop_per_byte"] else "hbm"), stage
        assert 0 < stage["frac_mfma"] < 1 and 0 < stage["frac_hbm"] < 1
    assert sum(s["avg_ms"] for s in rec["kernels"]) < 1.25 * rec["ms_per_step"]
    cpu = rec["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "tokens/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    assert rec["value"] > 20 * cpu["value"]
    assert 0.3 < rec["mfma_sustained"]["frac_of_peak"] < 1.0
    # the other workloads of the benchmark contract
    cfg = rec["configs"]
    assert set(cfg) == {"layer_24x1024_protocol_only", "layer_24x1024_graph_replay", "layer_96x1024", "layer_24x1024_zipf_ties",
                        "decoder_12layer_24x1024"}
    for name, row in cfg.items():
        assert row["tokens_per_s"] > 0 and row["ms_per_step"] > 0 and row["peak_hbm_allocated_mb"] > 0, name
    proto = cfg["layer_24x1024_protocol_only"]
    assert proto["tokens"] == 24576 and proto["ms_per_step"] >= 0.97 * rec["ms_per_step"]   # the hooks only take work away
    replay = cfg["layer_24x1024_graph_replay"]
    assert replay["tokens"] == 24576 and 0.9 * rec["ms_per_step"] < replay["ms_per_step"] < 1.05 * rec["ms_per_step"]   # the same kernels
    assert cfg["layer_96x1024"]["tokens"] == 98304 and cfg["layer_96x1024"]["peak_hbm_allocated_mb"] > cfg["layer_96x1024"]["resident_inputs_mb"]
    skew = cfg["layer_24x1024_zipf_ties"]
    assert 0.33 < skew["top_expert_share"] < 0.5 and skew["tied_tokens"] == 246
    dec = cfg["decoder_12layer_24x1024"]
    assert dec["parameters"] == 293494272 and 0.02 < dec["moe_share_of_step"] < 0.6
