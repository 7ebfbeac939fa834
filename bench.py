#!/usr/bin/env python3
"""MoE-layer forward+backward benchmark on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: fp32 router
GEMM -> router post-process -> fused top-2 MoE, then the full backward (dX,
dRouter, dW1, dW2).  The workload is the 293M-class layer shape: 24 x 1024
tokens, d_model 768, 8 experts, top-2, expert d_ff 1024, bf16 tensors with fp32
accumulation, seed 1, all inputs resident in HBM before the timed region.

One JSON line is printed.  Besides the whole-layer tokens/s it carries
  * ``kernels``: every kernel stage timed on its own with HIP events on the stream
    it is launched on, with its algorithmic FLOPs or bytes and roofline fraction;
  * ``roofline``: the same figures for the stage that takes the most time;
  * ``gemm_roofline`` / ``combine_roofline``: all expert GEMMs together against the
    dense bf16 MFMA peak, and the combine kernels against peak HBM bandwidth;
  * ``configs``: the other benchmark workloads, each a short run of its own: the headline layer through the
    unchanged two-method operator protocol (no extension hooks), the 98304-token batch with its peak
    allocation, Zipf-imbalanced routing with exact ties, and the 12-layer decoder's training step with the
    MoE share of it;
  * ``cpu_baseline``: the CPU restatement of the reference's PyTorch path timed on
    the host cores of the same box on a bounded sample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "mini-train-sys_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import numpy as np
import torch
import torch.nn.functional as F

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

RIDGE_FLOP_PER_BYTE = PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9)   # 312.5: below it a kernel is HBM-bound

# HBM-side bytes per launch (fetch + write) of the GEMM and combine stages at this workload.  They come
# from two rocprofv3 counter runs (FETCH_SIZE, then WRITE_SIZE; FETCH_SIZE scaled by 2.0 and WRITE_SIZE by
# 1.0 against a plain copy kernel of known size) and are NOT measured live: `traffic_source` in the bench
# line names the file that holds the runs' commands and tables.
TRAFFIC_SOURCE = "profiles/moe_layer_24x1024_hbm_traffic.txt"
MEASURED_TRAFFIC_BYTES = {
    "fwd_gateup_down": 772.7e6,   # gate/up and down as one launch; as two launches: 546.9 and 224.1
    "fwd_gateup_swiglu": 546.9e6, "fwd_down": 224.1e6, "bwd_dy1": 538.8e6,
    "bwd_joint": 1248.1e6,   # the joint launch (1083.0) and the launch of partial sums with the dX combine behind it (165.1)
    "combine": 114.7e6,
}

# the forward GEMMs as the layer node issues them: one launch unless the comparison switch asks for two
JOINT_FWD = os.environ.get("MTS_NO_JOINT_FWD", "0") in ("", "0")

WORKLOAD = dict(name="moe_layer_24x1024_d768_e8_top2_ff1024_bf16", seed=1, T=24576, H=768, E=8, K=2, I=1024)


def make_inputs(seed, T, H, E, I):
    """x, W_r, gate_up_proj, down_proj, G drawn in that order from a Philox stream."""
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.standard_normal((T, H), dtype=np.float32)
    w_r = rng.standard_normal((E, H), dtype=np.float32) * np.float32(0.02)
    w1 = rng.standard_normal((E, 2 * I, H), dtype=np.float32) * np.float32(0.02)
    w2 = rng.standard_normal((E, H, I), dtype=np.float32) * np.float32(0.02)
    g = rng.standard_normal((T, H), dtype=np.float32)
    return tuple(torch.from_numpy(a) for a in (x, w_r, w1, w2, g))


class Layer:
    """The layer as the MoE block runs it, with leaves that collect gradients.

    ``protocol_only``: the step goes through the two methods of the reference's operator protocol alone
    (`router_postprocess`, `fused_moe`) with `F.linear` for the logits, `torch.bincount` for the route counts
    and autograd's own sum of the two gradients of `x`, i.e. what an unmodified `minitrain/model` MoE block
    costs (minitrain/model/moe_router.py:63-144, blocks.py:86-102); none of the backend's extension hooks
    (`moe_layer`, `router_logits`, the counts and casts inside the post-process) is used.
    ``logit_transform``: applied to the logits before the post-process (the imbalanced-routing workload);
    it takes the layer off the one-node path, which forms the logits itself."""

    def __init__(self, ops, x, w_r, w1, w2, g, K, protocol_only=False, logit_transform=None):
        self.ops, self.K = ops, K
        self.protocol_only, self.logit_transform = protocol_only, logit_transform
        self.x = x.cuda().bfloat16().requires_grad_(True)
        self.w_r = w_r.cuda().requires_grad_(True)
        self.w1 = w1.cuda().bfloat16().requires_grad_(True)
        self.w2 = w2.cuda().bfloat16().requires_grad_(True)
        self.g = g.cuda().bfloat16()
        self.E = w_r.shape[0]
        self.seed_aux = torch.tensor(0.01, device="cuda")    # router_aux_loss_coef (minitrain/model/config.py:20)
        self.seed_z = torch.tensor(0.001, device="cuda")     # router_z_loss_coef (config.py:21)

    def hook(self, name):
        return None if self.protocol_only else getattr(self.ops, name, None)

    def step(self):
        for t in (self.x, self.w_r, self.w1, self.w2):
            t.grad = None
        # as the MoE block does: a backend that offers the whole layer as one node is asked first
        layer = self.hook("moe_layer") if self.logit_transform is None else None
        whole = layer(self.x, self.w_r, self.w1, self.w2, self.K, normalize=True) if layer is not None else None
        if whole is not None:
            out, aux, z_loss = whole[:3]
            torch.autograd.backward([out, aux, z_loss], [self.g, self.seed_aux, self.seed_z])
            return out
        fused = self.hook("router_logits")
        logits = fused(self.x, self.w_r) if fused is not None else None
        if logits is None:
            logits = F.linear(self.x.float(), self.w_r)
        if self.logit_transform is not None:
            logits = self.logit_transform(logits)
        # as the router module does: the backend may hand back the weights in the activation dtype itself
        extra = {"weights_dtype": self.x.dtype} if self.hook("casts_router_weights") else {}
        route = self.ops.router_postprocess(logits, self.K, normalize=True, **extra)
        aux = None if self.protocol_only else getattr(route, "load_balance_loss", None)
        if aux is None:
            counts = torch.bincount(route.expert_indices.flatten().long(), minlength=self.E)
            aux = self.E * torch.sum(counts.float() / route.expert_indices.numel() * route.probability_per_expert)
        weights = None if self.protocol_only else getattr(route, "expert_weights_cast", None)
        if weights is None:
            weights = route.expert_weights.to(self.x.dtype)
        self.last_indices = route.expert_indices
        out = self.ops.fused_moe(self.x, self.w1, self.w2, route.expert_indices, weights)
        # loss = sum(out * G) + 0.01 * aux + 0.001 * z: its gradient enters as the three seeds G, 0.01 and
        # 0.001, so the scalar itself (a few 5 us element-wise launches on 0-dim tensors) is not formed
        torch.autograd.backward([out, aux, route.z_loss], [self.g, self.seed_aux, self.seed_z])
        return out


def settle(layer, seconds=0.4, at_least=30):
    """Untimed steps until the clocks have settled: the first steps after an idle period run 5-15 % slower
    on this chip, however few warm-up steps the caller asks for.  Returns the number of steps run."""
    n, t_end = 0, time.perf_counter() + seconds
    while n < at_least or time.perf_counter() < t_end:
        layer.step()
        n += 1
        if n % 10 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    return n


def time_layer(layer, steps, warmup):
    for _ in range(warmup):
        layer.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        layer.step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def check_forward_status():
    """The joint gate/up + down launches of the steps so far all ran through (their outputs would be invalid otherwise)."""
    from minitrain_amd.kernels.hip.fused_moe import joint_forward_status

    status = joint_forward_status()
    if status != 0:
        raise RuntimeError(f"the joint gate/up + down launch reported status {status}")


def stage_breakdown(layer, steps):
    """Launch every stage of the layer step through the C ABI, in the order the layer node issues them,
    with HIP events (recorded on the launching stream) around each call.

    Every stage carries its algorithmic FLOPs and its algorithmic bytes (what one launch must read and
    write once); the binding roofline follows from their ratio against the ridge of the chip."""
    from minitrain_amd import _lib

    lib = _lib.load()
    w = WORKLOAD
    T, H, E, K, I = w["T"], w["H"], w["E"], w["K"], w["I"]
    TK = T * K
    dev = layer.x.device
    bf = dict(dtype=torch.bfloat16, device=dev)
    f32, i32 = dict(dtype=torch.float32, device=dev), dict(dtype=torch.int32, device=dev)
    x, w_r, w1, w2, g = layer.x.detach(), layer.w_r.detach(), layer.w1.detach(), layer.w2.detach(), layer.g
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    B = _lib.MTS_BF16
    esz = 2
    # head outputs
    logits, r_w, r_i, r_wa = torch.empty(T, E, **f32), torch.empty(T, K, **f32), torch.empty(T, K, **i32), torch.empty(T, K, **bf)
    r_stats = torch.empty(2 * E + 10, **f32)
    cnt, es = torch.empty(E, **i32), torch.empty(E + 1, **i32)
    ss, sr, xg = torch.empty(TK, **i32), torch.empty(TK, **i32), torch.empty(TK, **i32)
    hws = torch.empty(lib.mts_moe_head_workspace_bytes(T, K, E), dtype=torch.uint8, device=dev)
    # expert path
    pre, post, y, out = torch.empty(TK, 2 * I, **bf), torch.empty(TK, I, **bf), torch.empty(TK, H, **bf), torch.empty(T, H, **bf)
    dpre, dxe, dx = torch.empty(TK, 2 * I, **bf), torch.empty(TK, H, **bf), torch.empty(T, H, **bf)
    npart = lib.mts_moe_ds_partials(I)
    dsp = torch.empty(TK, npart, **f32)
    dwts = torch.empty(T, K, **bf)
    dw1, dw2 = torch.empty_like(w1), torch.empty_like(w2)
    dws1 = torch.empty(lib.mts_moe_bwd_dw_workspace_bytes(1, E, H, I), dtype=torch.uint8, device=dev)
    dws2 = torch.empty(lib.mts_moe_bwd_dw_workspace_bytes(2, E, H, I), dtype=torch.uint8, device=dev)
    # router backward
    gp, gz = torch.randn(E, device=dev), torch.ones((), device=dev)
    bws = torch.empty(lib.mts_moe_head_bwd_workspace_bytes(T, H, E), dtype=torch.uint8, device=dev)
    dx_r, dw_r = torch.empty(T, H, **bf), torch.empty_like(w_r)
    sched = torch.empty(lib.mts_moe_bwd_schedule_bytes(E) // 4, **i32)   # written by the dO*W2 launch, read by the joint one

    status_words = []
    unit = 2.0 * TK * H * I                  # FLOPs of one [TK,H] x [H,I] product
    w1_b, w2_b = E * 2 * I * H * esz, E * H * I * esz
    rows_h, rows_i = TK * H * esz, TK * I * esz
    if JOINT_FWD and lib.mts_moe_fwd_joint_supported(B, H, I):
        # gate/up and down in one launch, as the layer node issues them: post_act is written once and read inside the launch
        jws = torch.zeros(lib.mts_moe_fwd_joint_workspace_bytes(TK, E) // 4, **i32)
        status_words.append(jws)
        fwd_gemm_stages = [
            ("fwd_gateup_down", 3 * unit, rows_h + w1_b + 3 * rows_i + TK * (4 + 4 + esz) + w2_b + rows_h,
             lambda: lib.mts_moe_fwd_gateup_down(p(x), p(w1), p(w2), p(xg), p(es), p(r_wa), p(ss), T, K, E, H, I, B, p(pre), p(post),
                                                 p(y), p(jws), jws.numel() * 4, st)),
        ]
    else:
        fwd_gemm_stages = [
            ("fwd_gateup_swiglu", 2 * unit, rows_h + w1_b + 3 * rows_i + TK * (4 + 4 + esz),
             lambda: lib.mts_moe_fwd_gateup_swiglu(p(x), p(w1), p(xg), p(es), p(r_wa), p(ss), T, K, E, H, I, B, p(pre), p(post), st)),
            ("fwd_down", unit, rows_i + w2_b + rows_h, lambda: lib.mts_moe_fwd_down(p(post), p(w2), p(es), TK, E, H, I, B, p(y), st)),
        ]
    stages = [
        # name, FLOPs, algorithmic bytes, call
        ("head_fwd", 2.0 * T * H * E, T * H * esz + E * H * 4 + T * E * 4 + T * K * (4 + 4 + esz) + TK * 4 * 4,
         lambda: lib.mts_moe_head_fwd(p(x), p(w_r), T, H, E, K, 1, B, p(logits), p(r_w), p(r_i), p(r_wa), p(r_stats),
                                      p(r_stats) + 4 * E, p(r_stats) + 4 * E + 4, p(cnt), p(r_stats) + 4 * E + 8,
                                      p(r_stats) + 4 * E + 12, p(es), p(ss), p(sr), p(xg), p(hws), hws.numel(), st)),
        *fwd_gemm_stages,
        ("combine", 1.0 * TK * H, rows_h + T * H * esz + TK * 4,
         lambda: lib.mts_moe_combine(p(y), None, None, p(sr), T, K, H, B, p(out), st)),
        ("bwd_dy1", unit, rows_h + w2_b + 2 * rows_i + 2 * rows_i + TK * npart * 4 + TK * (4 + 4 + esz),
         lambda: lib.mts_moe_bwd_dy1(p(g), p(w2), 1, p(pre), p(r_wa), p(xg), p(ss), p(es), T, K, E, H, I, B, p(dpre), None, p(dsp), p(sched), st)),
        # dW1, dW2, dX, the dS reduction and the router's backward (its blocks trail the dX tiles): one launch, plus
        # one small launch for the chunk sum, the dW_r partial sum and the dX combine, as the layer node issues them
        ("bwd_joint", 5 * unit + 4.0 * T * H * E + 1.0 * TK * H,
         2 * (2 * rows_i) + 2 * rows_h + rows_i + w1_b + rows_h + w1_b + w2_b + 2 * TK * npart * 4
         + 2 * T * H * esz + T * E * 4 + T * K * (4 + 4) + 2 * E * H * 4
         + rows_h + 2 * T * H * esz + TK * 4,
         lambda: lib.mts_moe_bwd_joint_router(p(g), p(post), p(dpre), p(x), p(w1), p(xg), p(es), p(sr), p(dsp), T, K, E, H, I, B, B,
                                              p(dxe), p(dw1), p(dw2), p(dwts), p(dws1), dws1.numel(), p(dws2), dws2.numel(),
                                              p(w_r), p(logits), p(r_w), p(r_i), p(cnt), p(gp), p(gz), p(gz), 1, p(dx_r), p(dx), p(dw_r),
                                              p(bws), bws.numel(), p(sched), st)),
    ]
    # One stage is bracketed per pass over the whole sequence, so the other stages of that pass run
    # back to back as they do in the layer step and the chip is in the state it has there.
    elapsed = [[] for _ in stages]
    for j in range(len(stages)):
        for it in range(1 + steps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for i, (name, _, _, fn) in enumerate(stages):
                if i == j:
                    e0.record()
                rc = fn()
                if i == j:
                    e1.record()
                if rc != 0:
                    raise RuntimeError(f"{name} returned {rc}")
            if it:
                elapsed[j].append((e0, e1))
    torch.cuda.synchronize()
    for words in status_words:
        if int(words[0]) != 0:
            raise RuntimeError(f"the joint gate/up + down launch reported status {int(words[0])}")
    rows = []
    for j, (name, flops, nbytes, _) in enumerate(stages):
        ms = float(np.mean([a.elapsed_time(b) for a, b in elapsed[j]]))
        intensity = flops / nbytes
        bound = "mfma" if intensity >= RIDGE_FLOP_PER_BYTE else "hbm"
        tflops, gbs = flops / (ms * 1e-3) / 1e12, nbytes / (ms * 1e-3) / 1e9
        row = dict(stage=name, bound=bound, avg_ms=round(ms, 4), flops=flops, algorithmic_bytes=int(nbytes),
                   intensity_flop_per_byte=round(intensity, 1), tflops=round(tflops, 2), frac_mfma=round(tflops / PEAK_BF16_TFLOPS, 4),
                   gbs=round(gbs, 1), frac_hbm=round(gbs / PEAK_HBM_GBS, 4))
        if bound == "mfma":
            row.update(achieved=row["tflops"], peak=PEAK_BF16_TFLOPS, unit="TFLOP/s", frac=row["frac_mfma"])
        else:
            row.update(achieved=row["gbs"], peak=PEAK_HBM_GBS, unit="GB/s", frac=row["frac_hbm"])
        rows.append(row)
    return rows


def mfma_sustained(blocks=512, rounds=1000, launches=40, lead=10):
    """What the matrix pipes sustain on registers alone (no LDS, no memory): the library's probe kernel
    (two blocks of four waves per CU), launched back to back for ~100 ms and timed with events on the
    launching stream over the launches behind the first `lead` ones, so that the clocks are where the
    power governor leaves them under continuous load.  The rate on pseudo-random registers is the ceiling
    the GEMM figures are read against; the nominal peak stays the denominator of every `frac`."""
    import ctypes

    from minitrain_amd import _lib

    lib = _lib.load()
    sink = torch.empty(lib.mts_probe_mfma_sink_bytes(blocks), dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    flops = ctypes.c_double(0.0)
    out = {}
    for name, random_operands in (("random_operands", 1), ("constant_operands", 0)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for it in range(launches):
            if it == lead:
                e0.record()
            rc = lib.mts_probe_mfma_rate(random_operands, blocks, rounds, sink.data_ptr(), sink.numel(), ctypes.addressof(flops), st)
            if rc != 0:
                raise RuntimeError(f"mts_probe_mfma_rate returned {rc}")
        e1.record()
        torch.cuda.synchronize()
        out[name + "_tflops"] = round(flops.value * (launches - lead) / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)
    out.update(peak=PEAK_BF16_TFLOPS, unit="TFLOP/s", frac_of_peak=round(out["random_operands_tflops"] / PEAK_BF16_TFLOPS, 4),
               kernel=f"register-only bf16 32x32x16 MFMA loop, {blocks} blocks of 4 waves (two per CU), {launches} launches back to back, "
                      f"the last {launches - lead} timed")
    return out


def zipf_ties_transform(T, E, seed, s=1.2, tie_fraction=0.01):
    """The imbalanced-routing workload: log p_e is added to the logits, p_e ~ rank^-s over the experts, and on a
    seeded `tie_fraction` of the tokens two or three logits are overwritten with one value above the row's
    maximum (exact ties for rank 1/2, for rank 2/3 behind a clear winner, and three-way, in turn)."""
    rank = np.arange(1, E + 1, dtype=np.float64) ** (-s)
    bias = torch.from_numpy(np.log(rank / rank.sum()).astype(np.float32)).cuda()
    rng = np.random.Generator(np.random.Philox(seed + 1000))
    rows = rng.choice(T, size=max(1, int(round(tie_fraction * T))), replace=False)
    mask = np.zeros((T, E), dtype=bool)
    lift = np.zeros((T, E), dtype=np.float32)
    for j, t in enumerate(rows):
        cols = rng.choice(E, size=3, replace=False)
        kind = j % 3
        picked = cols[:2] if kind == 0 else cols
        mask[t, picked] = True
        lift[t, picked] = 1.0
        if kind == 1:
            lift[t, cols[0]] = 2.0
    mask, lift = torch.from_numpy(mask).cuda(), torch.from_numpy(lift).cuda()

    def transform(logits):
        biased = logits + bias
        top = biased.detach().amax(dim=1, keepdim=True)
        return torch.where(mask, top + lift, biased)

    transform.tied_tokens = int(len(rows))
    return transform


class Replayed:
    """A layer's step captured into a graph once (forward and backward on the layer's own buffers); `step` replays it."""

    def __init__(self, layer):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                layer.step()
        torch.cuda.current_stream().wait_stream(side)
        self.layer, self.graph = layer, torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            layer.step()

    def step(self):
        self.graph.replay()


def run_config(ops, seed, T, steps, warmup, **layer_kwargs):
    """tokens/s and peak allocation of one more workload of the same layer shape."""
    w = WORKLOAD
    replayed = layer_kwargs.pop("replayed", False)
    transform = layer_kwargs.pop("transform_factory", None)
    if transform is not None:
        layer_kwargs["logit_transform"] = transform(T, w["E"], seed)
    layer = Layer(ops, *make_inputs(seed, T, w["H"], w["E"], w["I"]), w["K"], **layer_kwargs)
    torch.cuda.synchronize()
    resident = torch.cuda.memory_allocated()
    runner = Replayed(layer) if replayed else layer   # (captured before the clocks are settled: a capture leaves the GPU idle)
    settle(runner, seconds=0.2, at_least=10)
    torch.cuda.reset_peak_memory_stats()
    sec = time_layer(runner, steps, warmup)
    check_forward_status()
    rec = {"tokens": T, "seed": seed, "ms_per_step": round(sec * 1e3, 4), "tokens_per_s": round(T / sec, 1),
           "layer_gemm_tflops": round(18.0 * T * w["K"] * w["H"] * w["I"] / sec / 1e12, 2),
           "peak_hbm_allocated_mb": round(torch.cuda.max_memory_allocated() / 2**20, 1),
           "resident_inputs_mb": round(resident / 2**20, 1)}
    idx = getattr(layer, "last_indices", None)
    if idx is not None and transform is not None:
        counts = torch.bincount(idx.flatten().long(), minlength=w["E"]).float()
        rec["top_expert_share"] = round(float(counts.max() / counts.sum()), 4)
        rec["tied_tokens"] = layer.logit_transform.tied_tokens
    del layer
    torch.cuda.empty_cache()
    return rec


def other_configs(ops, steps, warmup):
    """The benchmark workloads besides the headline one, each a short run of its own: the headline layer through
    the unchanged operator protocol, the headline step replayed from a graph, the 98304-token batch with its peak allocation, imbalanced routing with
    exact ties, and the 12-layer decoder's training step with the MoE share of it."""
    w = WORKLOAD
    out = {}
    out["layer_24x1024_protocol_only"] = dict(
        run_config(ops, w["seed"], w["T"], steps, warmup, protocol_only=True),
        path="F.linear + OpsBackend.router_postprocess + torch.bincount + OpsBackend.fused_moe, autograd sums dx; no extension hooks")
    out["layer_24x1024_graph_replay"] = dict(
        run_config(ops, w["seed"], w["T"], steps, warmup, replayed=True),
        path="the headline step (one autograd node, forward and backward) captured into a graph once and replayed")
    out["layer_96x1024"] = dict(run_config(ops, 2, 98304, max(3, steps // 2), max(1, warmup // 2)), path="one autograd node (as the headline)")
    out["layer_24x1024_zipf_ties"] = dict(
        run_config(ops, 3, w["T"], steps, warmup, transform_factory=zipf_ties_transform),
        path="router_logits hook + bias and ties (torch) + router_postprocess + fused_moe")
    from minitrain_amd.train.bench_step import run as decoder_step

    rec = decoder_step(steps=5, warmup=4)
    out["decoder_12layer_24x1024"] = {
        "tokens_per_s": round(rec["value"], 1), "ms_per_step": round(rec["ms_per_step"], 3),
        "moe_ms_per_step": round(rec["moe_ms_per_step"], 3), "moe_share_of_step": round(rec["moe_share_of_step"], 4),
        "parameters": rec["parameters"], "peak_hbm_allocated_mb": round(rec["peak_allocated_gib"] * 1024, 1),
        "ms_per_step_mean": round(rec["ms_per_step_mean"], 3), "timing": "median of the timed steps (each ends with the host reading the loss)",
        "steps": 5, "warmup": 4, "dtype": "bf16 autocast, fp32 parameters, AdamW", "seed": 4}
    torch.cuda.empty_cache()
    return out


def cpu_baseline(budget_s=20.0):
    """The oracle's restatement of the reference's PyTorch path (input-dtype arithmetic,
    autograd backward) on the host cores, on the first ``sample`` tokens of the workload."""
    from oracle import moe_oracle as O

    w = WORKLOAD
    sample = w["T"]
    x, w_r, w1, w2, g = O.make_inputs(w["seed"], w["T"], w["H"], w["E"], w["I"])
    x, g = x[:sample].bfloat16(), g[:sample].bfloat16()
    w1, w2 = w1.bfloat16(), w2.bfloat16()

    def step():
        leaves = [t.clone().requires_grad_(True) for t in (x, w_r, w1, w2)]
        hidden, r = O.moe_feed_forward(leaves[0], leaves[1], leaves[2], leaves[3], w["K"])
        loss = (hidden.float() * g.float()).sum() + 0.01 * r.auxiliary_loss + 0.001 * r.z_loss
        loss.backward()

    step()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 10 and (time.perf_counter() < t_end or len(times) < 3):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    p50 = float(np.median(times))
    return dict(value=round(sample / p50, 1), unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{sample} of {w['T']} tokens of the same workload, bf16 tensors, fwd+bwd, p50 of {len(times)} runs",
                host_cpus=os.cpu_count(), p50_s=round(p50, 4))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    ap.add_argument("--no-mfma-probe", action="store_true", help="skip the register-only MFMA rate probe")
    ap.add_argument("--no-configs", action="store_true", help="skip the workloads besides the headline one (`configs` in the line)")
    ap.add_argument("--no-settle", action="store_true", help="skip the untimed clock-settling steps before the warm-up")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB -> 256 MiB elementwise copy (the known-size kernel that "
                         "FETCH_SIZE / WRITE_SIZE counter runs are scaled by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU fallback for the hip backend)", file=sys.stderr)
        sys.exit(2)

    from minitrain_amd.model.ops import get_ops_backend

    w = WORKLOAD
    ops = get_ops_backend("hip")
    layer = Layer(ops, *make_inputs(w["seed"], w["T"], w["H"], w["E"], w["I"]), w["K"])
    settled = 0 if args.no_settle else settle(layer)
    sec = time_layer(layer, args.steps, args.warmup)
    check_forward_status()
    tokens_per_s = w["T"] / sec
    gemm_flops = 18.0 * w["T"] * w["K"] * w["H"] * w["I"]

    result = {
        "metric": "MoE layer fwd+bwd tokens/s (24x1024, bf16)",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_steps": settled,
        "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": w["name"], "tokens": w["T"], "d_model": w["H"], "experts": w["E"], "top_k": w["K"],
                   "d_ff": w["I"], "seed": w["seed"],
                   "step": "router projection + router post-process + routing metadata + fused MoE, fwd + full bwd",
                   "timing": "untimed clock-settling steps (settle_steps), then `warmup` untimed steps, then `steps` timed steps"},
        "layer_gemm_tflops": round(gemm_flops / sec / 1e12, 2),
    }
    if not args.no_breakdown:
        rows = stage_breakdown(layer, max(5, min(args.steps, 20)))
        result["kernels"] = rows
        dom = max(rows, key=lambda r: r["avg_ms"])
        traffic = MEASURED_TRAFFIC_BYTES.get(dom["stage"])
        result["roofline"] = {"kernel": dom["stage"], "bound": dom["bound"], "achieved": dom["achieved"], "peak": dom["peak"],
                              "unit": dom["unit"], "frac": dom["frac"], "avg_ms": dom["avg_ms"],
                              "algorithmic_flops": dom["flops"], "algorithmic_bytes": dom["algorithmic_bytes"],
                              "intensity_flop_per_byte": dom["intensity_flop_per_byte"], "ridge_flop_per_byte": RIDGE_FLOP_PER_BYTE,
                              "frac_mfma": dom["frac_mfma"], "frac_hbm": dom["frac_hbm"],
                              "traffic": traffic, "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                              "traffic_over_algorithmic": round(traffic / dom["algorithmic_bytes"], 3) if traffic else None}
        gemm_rows = [r for r in rows if r["stage"] in ("fwd_gateup_down", "fwd_gateup_swiglu", "fwd_down", "bwd_dy1", "bwd_joint")]
        g_ms = sum(r["avg_ms"] for r in gemm_rows)
        g_ach = sum(r["flops"] for r in gemm_rows) / (g_ms * 1e-3) / 1e12
        result["gemm_roofline"] = {"bound": "mfma", "achieved": round(g_ach, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                   "frac": round(g_ach / PEAK_BF16_TFLOPS, 4), "sum_ms": round(g_ms, 4)}
        c_rows = [r for r in rows if r["stage"] == "combine"]
        c_ms = sum(r["avg_ms"] for r in c_rows)
        c_ach = sum(r["algorithmic_bytes"] for r in c_rows) / (c_ms * 1e-3) / 1e9
        result["combine_roofline"] = {"bound": "hbm", "achieved": round(c_ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                      "frac": round(c_ach / PEAK_HBM_GBS, 4), "sum_ms": round(c_ms, 4)}
        result["kernel_sum_ms"] = round(sum(r["avg_ms"] for r in rows), 4)
    if not args.no_mfma_probe:
        result["mfma_sustained"] = mfma_sustained()
        if "gemm_roofline" in result:
            result["gemm_roofline"]["frac_of_sustained"] = round(
                result["gemm_roofline"]["achieved"] / result["mfma_sustained"]["random_operands_tflops"], 4)
    if args.copy_probe:
        src = torch.ones(64 * 2**20, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        result["copy_probe_bytes_each_way"] = src.numel() * 4
    if not args.no_configs:
        del layer
        torch.cuda.empty_cache()
        result["configs"] = other_configs(ops, max(5, min(args.steps, 20)), max(2, min(args.warmup, 5)))
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
