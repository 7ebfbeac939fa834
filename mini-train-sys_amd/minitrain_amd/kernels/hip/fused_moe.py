"""Fused top-k MoE (dispatch -> grouped SwiGLU experts -> weighted combine).

Counterpart of minitrain/kernels/triton/fused_moe.py:37-449: the support
predicate, the routing-metadata step, the autograd function and the module-level
entry point.  Every buffer is a torch tensor on the caller's device; kernels are
enqueued through the C ABI and nothing synchronises with the host.  The backward pass
forks two side streams from the current stream for kernels that do not depend on one
another and joins them before it returns.
"""

import functools
import warnings

import torch

from minitrain_amd import _lib
from minitrain_amd.kernels.hip.switches import SWITCHES

_MAX_EXPERTS = 65534   # MTS_MAX_MOE_EXPERTS
BLOCK_M_TOKEN = 64


def ensure_contiguous(fn):
    """Autograd-function decorator: every tensor argument reaches ``fn`` dense and row-major."""

    @functools.wraps(fn)
    def dense_call(ctx, *args):
        return fn(ctx, *(a.contiguous() if torch.is_tensor(a) else a for a in args))

    return dense_call


def expert_contract(x, gate_up_proj, down_proj):
    """``(holds, requirement)`` pairs for the activations and the expert parameters; the first one that
    does not hold is what an error message names."""
    tensors = (x, gate_up_proj, down_proj)
    if not all(torch.is_tensor(t) for t in tensors):
        return [(False, "x, gate_up_proj and down_proj are tensors")]
    shapes_ok = x.ndim == 2 and gate_up_proj.ndim == 3 and down_proj.ndim == 3
    if not shapes_ok:
        return [(False, "x is [T,H], gate_up_proj [E,2I,H] and down_proj [E,H,I]")]
    T, H = x.shape
    E, two_i, h_w = gate_up_proj.shape
    I = two_i // 2
    wide = x.dtype == torch.float32
    # expert parameters come in the activation dtype or as fp32 master weights; fp32 activations
    # take 16-bit parameters as well (widened once per call)
    param_dtypes = (torch.float32, torch.bfloat16, torch.float16) if wide else (x.dtype, torch.float32)
    return [
        (all(t.is_cuda for t in tensors) and len({t.device for t in tensors}) == 1, "all tensors on one GPU"),
        (x.dtype in (torch.bfloat16, torch.float16, torch.float32), "activations are bf16, fp16 or fp32"),
        (T > 0, "at least one token"),
        (0 < E <= _MAX_EXPERTS, f"between 1 and {_MAX_EXPERTS} experts"),
        (two_i % 2 == 0 and h_w == H and tuple(down_proj.shape) == (E, H, I),
         "gate_up_proj is [E,2I,H] and down_proj [E,H,I] for x [T,H]"),
        (gate_up_proj.dtype in param_dtypes and down_proj.dtype in param_dtypes,
         "expert parameters in the activation dtype or fp32 (any of fp32/bf16/fp16 under fp32 activations)"),
        # rows of x and of dO are gathered from anywhere through 32-bit offsets; the [T*K, ...] intermediates are
        # addressed tile by tile and may be larger
        (wide or (T * H * 2 < 2**31 and 2 * I * H * 2 < 2**31), "16-bit activations and one expert's weights smaller than 2 GiB each"),
    ]


def routing_contract(x, gate_up_proj, top_k_index, top_k_weights):
    if not (torch.is_tensor(top_k_index) and torch.is_tensor(top_k_weights)):
        return [(False, "top_k_index and top_k_weights are tensors")]
    if top_k_index.ndim != 2:
        return [(False, "top_k_index is [T,K]")]
    K = top_k_index.shape[1]
    return [
        (top_k_index.is_cuda and top_k_weights.is_cuda and top_k_index.device == x.device == top_k_weights.device,
         "routing tensors on the activations' GPU"),
        (top_k_weights.shape == top_k_index.shape and top_k_index.shape[0] == x.shape[0], "top_k_index and top_k_weights are [T,K]"),
        (0 < K <= min(gate_up_proj.shape[0], 32768), "1 <= K <= number of experts (at most 32768)"),
        (x.shape[0] * K < 2**31, "fewer than 2^31 routes"),
        (top_k_index.dtype == torch.int32, "int32 expert indices"),
        (top_k_weights.dtype == x.dtype, "routing weights in the activation dtype"),
    ]


def first_violation(pairs):
    for holds, requirement in pairs:
        if not holds:
            return requirement
    return None


def fused_moe_violation(x, gate_up_proj, down_proj, top_k_index, top_k_weights):
    """The first requirement of the operator's tensor contract that the arguments miss, or None."""
    missed = first_violation(expert_contract(x, gate_up_proj, down_proj))
    return missed if missed is not None else first_violation(routing_contract(x, gate_up_proj, top_k_index, top_k_weights))


def is_fused_moe_supported(x, gate_up_proj, down_proj, top_k_index, top_k_weights) -> bool:
    """Counterpart of the reference's predicate (minitrain/kernels/triton/fused_moe.py:37-71)."""
    return fused_moe_violation(x, gate_up_proj, down_proj, top_k_index, top_k_weights) is None


def compute_routing_metadata(topk_indices: torch.Tensor, E: int, block_m_token: int = BLOCK_M_TOKEN):
    """Counts, expert offsets, the stable expert-major permutation and the tile list.

    Returns the same eight tensors, in the same order, as the reference's
    ``compute_routing_metadata`` (minitrain/kernels/triton/fused_moe.py:74-154).
    """
    lib = _lib.load()
    topk_indices = topk_indices.contiguous()
    T, K = topk_indices.shape
    TK = T * K
    dev = topk_indices.device
    i32 = dict(dtype=torch.int32, device=dev)
    expert_token_count = torch.empty(E, **i32)
    expert_start_idx = torch.empty(E + 1, **i32)
    s_scatter_idx = torch.empty(TK, **i32)
    s_reverse_scatter_idx = torch.empty(TK, **i32)
    x_gather_idx = torch.empty(TK, **i32)
    max_m_tiles = min(TK, -(-TK // block_m_token) + E - 1)
    tile_row_start = torch.empty(max_m_tiles, **i32)
    tile_expert = torch.empty(max_m_tiles, **i32)
    tile_count = torch.empty(1, **i32)
    ws_bytes = lib.mts_moe_route_workspace_bytes(T, K, E)
    ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
    _lib.check(
        lib.mts_moe_route(
            topk_indices.data_ptr(), T, K, E, block_m_token, expert_token_count.data_ptr(),
            expert_start_idx.data_ptr(), s_scatter_idx.data_ptr(), s_reverse_scatter_idx.data_ptr(),
            x_gather_idx.data_ptr(), tile_row_start.data_ptr(), tile_expert.data_ptr(),
            tile_count.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_of(topk_indices),
        ),
        "mts_moe_route",
    )
    return (
        expert_token_count,
        expert_start_idx,
        x_gather_idx,
        s_scatter_idx,
        s_reverse_scatter_idx,
        tile_row_start,
        tile_expert,
        tile_count,
    )


def routing_for_experts(topk_indices: torch.Tensor, E: int):
    """``(expert_start, x_gather, s_scatter, s_reverse)``: what the operator itself needs of the routing
    metadata, in one int32 allocation (the tile list of the reference's kernels is not produced)."""
    lib = _lib.load()
    T, K = topk_indices.shape
    TK = T * K
    dev = topk_indices.device
    pad = -(-(2 * E + 1) // 4) * 4           # the per-row arrays start on 16-byte boundaries
    buf = torch.empty(pad + 3 * TK, dtype=torch.int32, device=dev)
    counts, expert_start = buf[:E], buf[E:2 * E + 1]
    s_scatter, s_reverse, x_gather = buf[pad:pad + TK], buf[pad + TK:pad + 2 * TK], buf[pad + 2 * TK:]
    ws_bytes = lib.mts_moe_route_workspace_bytes(T, K, E)
    ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
    _lib.check(
        lib.mts_moe_route(
            topk_indices.data_ptr(), T, K, E, BLOCK_M_TOKEN, counts.data_ptr(), expert_start.data_ptr(),
            s_scatter.data_ptr(), s_reverse.data_ptr(), x_gather.data_ptr(), None, None, None, ws.data_ptr(), ws_bytes,
            _lib.stream_of(topk_indices),
        ),
        "mts_moe_route",
    )
    return expert_start, x_gather, s_scatter, s_reverse


def expert_counts(topk_indices: torch.Tensor, E: int) -> torch.Tensor:
    """Routes per expert, int32 ``[E]``: the histogram pass of the routing metadata alone.

    Stands in for ``torch.bincount(expert_indices.flatten().long(), minlength=E)`` of the
    router module (minitrain/model/moe_router.py:82) without its host synchronisation.
    """
    lib = _lib.load()
    topk_indices = topk_indices.contiguous()
    if topk_indices.dtype != torch.int32 or topk_indices.ndim != 2 or not topk_indices.is_cuda:
        raise RuntimeError("hip expert_counts requires a 2D int32 index tensor on the GPU")
    T, K = topk_indices.shape
    dev = topk_indices.device
    out = torch.empty(2 * E + 1, dtype=torch.int32, device=dev)   # counts, then expert_start
    ws_bytes = lib.mts_moe_route_workspace_bytes(T, K, E)
    ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
    _lib.check(
        lib.mts_moe_route(
            topk_indices.data_ptr(), T, K, E, BLOCK_M_TOKEN, out.data_ptr(), out[E:].data_ptr(), None, None, None,
            None, None, None, ws.data_ptr(), ws_bytes, _lib.stream_of(topk_indices),
        ),
        "mts_moe_route",
    )
    return out[:E]


_SIDE_STREAMS: dict = {}


def _side_stream(device: torch.device, index: int) -> torch.cuda.Stream:
    key = (device.index if device.index is not None else torch.cuda.current_device(), index)
    s = _SIDE_STREAMS.get(key)
    if s is None:
        s = _SIDE_STREAMS[key] = torch.cuda.Stream(device=device)   # default priority
    return s


# The weight-gradient GEMMs cut the rows of an over-full expert into chunks when they are given a
# workspace for the chunk partials (skewed routing); beyond this size they run without one.
_DW_WORKSPACE_LIMIT = 512 * 2**20


_warned_shapes: set = set()


def _dw_workspace(lib, which: int, E: int, H: int, I: int, dtype: torch.dtype, device):
    nbytes = lib.mts_moe_bwd_dw_workspace_bytes(which, E, H, I) if dtype != torch.float32 else 0
    if nbytes > _DW_WORKSPACE_LIMIT and (E, H, I) not in _warned_shapes:
        # said once per shape: from here on an over-full expert is not cut into row chunks and the joint launch gets no
        # schedule, so skewed routing costs these widths more time than it has to (the results are the same)
        _warned_shapes.add((E, H, I))
        warnings.warn(f"hip fused MoE: the row-chunk workspace of the weight-gradient GEMMs for E={E}, H={H}, I={I} would take "
                      f"{nbytes / 2**20:.0f} MiB (limit {_DW_WORKSPACE_LIMIT / 2**20:.0f} MiB); running without it", RuntimeWarning,
                      stacklevel=3)
    if nbytes <= 0 or nbytes > _DW_WORKSPACE_LIMIT:
        return None, 0, 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return ws, ws.data_ptr(), nbytes


class _JointForwardWorkspace:
    """Counters of the launch that holds gate/up and down (``mts_moe_fwd_gateup_down``), one per device and stream.

    The launch needs them zero and leaves them zero, so the layers of a model that run one after the other on a stream
    share one buffer.  Word 0 is the launch's status: it stays zero unless a block gave up waiting for the rows it reads
    (or found them written on another XCD than its own); the outputs of that call are then invalid.  Nothing here
    waits for the GPU: every ``CHECK_EVERY`` calls the word is copied to pinned host memory, and the copy of an earlier
    call is looked at once its event has passed, so an error is raised a few calls late rather than never."""

    CHECK_EVERY = 16

    def __init__(self, device: torch.device):
        self.device = device
        self.buf = None
        self.host = None     # pinned word, allocated with the first copy (not while a graph is being captured)
        self.event = None
        self.calls = 0

    def get(self, nbytes: int) -> torch.Tensor:
        if self.buf is None or self.buf.numel() * 4 < nbytes:
            self.buf = torch.zeros((nbytes + 3) // 4, dtype=torch.int32, device=self.device)
        return self.buf

    def _raise(self, status: int):
        self.buf = None     # the counters of a failed launch are not trusted again
        raise RuntimeError(f"hip fused MoE: the joint gate/up + down launch reported status {status} "
                           "(1: a block gave up waiting for its rows, 2: rows written on another XCD); the outputs of "
                           "that call are invalid. MTS_NO_JOINT_FWD=1 runs the two GEMMs as launches of their own.")

    def before_launch(self):
        # (a stream that is being captured into a graph admits neither the query nor the copy: the word is then left
        # to joint_forward_status())
        if torch.cuda.is_current_stream_capturing():
            return
        if self.event is not None and self.event.query():
            self.event = None
            if int(self.host[0]) != 0:
                self._raise(int(self.host[0]))

    def after_launch(self):
        self.calls += 1
        if torch.cuda.is_current_stream_capturing():
            return
        if self.event is None and self.calls % self.CHECK_EVERY == 1:
            if self.host is None:
                self.host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
            self.host.copy_(self.buf[:1], non_blocking=True)
            self.event = torch.cuda.Event()
            self.event.record()

    def status(self) -> int:
        """The status word now (waits for the stream)."""
        return 0 if self.buf is None else int(self.buf[0].item())


_JOINT_FWD: dict = {}


def _joint_forward_workspace(device: torch.device) -> _JointForwardWorkspace:
    key = (device.index if device.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(device).cuda_stream)
    ws = _JOINT_FWD.get(key)
    if ws is None:
        ws = _JOINT_FWD[key] = _JointForwardWorkspace(device)
    return ws


def joint_forward_status(device=None) -> int:
    """Status of the joint gate/up + down launches on the current stream of ``device`` (0: all of them ran through).
    Synchronises; for tests, benchmarks and the points where a training loop reads a value back anyway."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    return _joint_forward_workspace(device).status()


def _stage(lib, w: torch.Tensor, transpose: bool, dtype: torch.dtype, stream: int | None = None) -> torch.Tensor:
    """Copy of an expert weight ``[E,R,C]`` in the activation dtype, optionally as ``[E,C,R]``."""
    if not transpose and w.dtype == dtype:
        return w
    E, R, C = w.shape
    out = torch.empty((E, C, R) if transpose else (E, R, C), dtype=dtype, device=w.device)
    _lib.check(
        lib.mts_moe_stage_weights(
            w.data_ptr(), _lib.dtype_code(w.dtype), out.data_ptr(), _lib.dtype_code(dtype), E, R, C, int(transpose),
            _lib.stream_of(w) if stream is None else stream,
        ),
        "mts_moe_stage_weights",
    )
    return out


class _Saved:
    """What the forward pass leaves for the backward pass (the tensors travel through
    ``ctx.save_for_backward``; the rest are plain attributes)."""

    __slots__ = ("dims", "staged", "weighted")


def moe_forward(x, gate_up_proj, down_proj, weights_flat, routing):
    """Gate/up + SwiGLU, down projection and combine for routes that are already sorted.

    ``routing`` = ``(expert_start, x_gather, s_scatter, s_reverse)``.  Returns the output, the tensors
    to save for :func:`moe_backward` and the non-tensor state."""
    lib = _lib.load()
    expert_start, x_gather, s_scatter, s_reverse = routing
    T, H = x.shape
    E = gate_up_proj.shape[0]
    I = gate_up_proj.shape[1] // 2
    TK = weights_flat.numel()
    K = TK // T
    dev = x.device
    act = _lib.dtype_code(x.dtype)
    stream = _lib.stream_of(x)

    if (gate_up_proj.dtype == down_proj.dtype == torch.float32 and x.dtype != torch.float32
            and gate_up_proj.numel() % 8 == 0 and down_proj.numel() % 8 == 0):
        # fp32 master weights: both casts in one launch (the backward pass reuses the copies)
        w1, w2 = torch.empty_like(gate_up_proj, dtype=x.dtype), torch.empty_like(down_proj, dtype=x.dtype)
        _lib.check(
            lib.mts_moe_cast_weights_pair(gate_up_proj.data_ptr(), w1.data_ptr(), gate_up_proj.numel(), down_proj.data_ptr(),
                                          w2.data_ptr(), down_proj.numel(), act, stream),
            "mts_moe_cast_weights_pair",
        )
    else:
        w1 = _stage(lib, gate_up_proj, False, x.dtype)
        w2 = _stage(lib, down_proj, False, x.dtype)
    pre_act = torch.empty(TK, 2 * I, dtype=x.dtype, device=dev)
    post_act = torch.empty(TK, I, dtype=x.dtype, device=dev)
    # The routing weight is applied where the activation is formed: post_act = s * silu(g) * u.  The
    # down projection then yields s * y, the combine is a plain sum, and post_act is at the same time
    # the `weighted_act` operand of the dW2 GEMM, so it is kept for the backward pass instead of being
    # written again there (TK * I elements held from forward to backward, and as many fewer written).
    weighted = SWITCHES.weighted_post
    y = torch.empty(TK, H, dtype=x.dtype, device=dev)
    if SWITCHES.joint_fwd and x.dtype != torch.float32 and lib.mts_moe_fwd_joint_supported(act, H, I):
        # one launch: the down tiles take the CUs as the gate/up tiles leave them
        jw = _joint_forward_workspace(dev)
        jw.before_launch()
        nbytes = lib.mts_moe_fwd_joint_workspace_bytes(TK, E)
        counters = jw.get(nbytes)
        _lib.check(
            lib.mts_moe_fwd_gateup_down(
                x.data_ptr(), w1.data_ptr(), w2.data_ptr(), x_gather.data_ptr(), expert_start.data_ptr(),
                weights_flat.data_ptr() if weighted else None, s_scatter.data_ptr() if weighted else None,
                T, K, E, H, I, act, pre_act.data_ptr(), post_act.data_ptr(), y.data_ptr(), counters.data_ptr(), nbytes, stream,
            ),
            "mts_moe_fwd_gateup_down",
        )
        jw.after_launch()
    else:
        _lib.check(
            lib.mts_moe_fwd_gateup_swiglu(
                x.data_ptr(), w1.data_ptr(), x_gather.data_ptr(), expert_start.data_ptr(),
                weights_flat.data_ptr() if weighted else None, s_scatter.data_ptr() if weighted else None,
                T, K, E, H, I, act, pre_act.data_ptr(), post_act.data_ptr(), stream,
            ),
            "mts_moe_fwd_gateup_swiglu",
        )
        _lib.check(
            lib.mts_moe_fwd_down(
                post_act.data_ptr(), w2.data_ptr(), expert_start.data_ptr(), TK, E, H, I, act, y.data_ptr(), stream
            ),
            "mts_moe_fwd_down",
        )
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    _lib.check(
        lib.mts_moe_combine(
            y.data_ptr(), None if weighted else weights_flat.data_ptr(), None, s_reverse.data_ptr(), T, K, H, act,
            out.data_ptr(), stream,
        ),
        "mts_moe_combine",
    )
    tensors = (x, gate_up_proj, down_proj, pre_act, weights_flat, expert_start, x_gather, s_scatter, s_reverse,
               *((post_act,) if weighted else ()))
    state = _Saved()
    state.dims = (T, K, E, H, I)
    state.weighted = weighted
    # fp32 parameters under a bf16 activation dtype: the backward GEMMs that read the weights as
    # stored reuse the casts made here (38 MB a layer at the 768/1024 shape) instead of repeating them
    keep = bool(lib.mts_moe_bwd_weights_as_stored(act, H, I))
    state.staged = (w1 if keep and w1 is not gate_up_proj else None, w2 if keep and w2 is not down_proj else None)
    return out, tensors, state


class RouterTail:
    """What the router's backward needs besides ``dS`` (saved router tensors and the gradients of the
    router's loss terms); ``moe_backward`` fills ``dx_r`` / ``dw_r`` when that backward ran inside the
    launch of the expert GEMMs' backward."""

    def __init__(self, router_weight, logits, weights, indices, counts, g_prob_mean, g_z_loss, g_load_balance, normalize):
        self.router_weight, self.logits, self.weights, self.indices, self.counts = router_weight, logits, weights, indices, counts
        self.g_prob_mean, self.g_z_loss, self.g_load_balance, self.normalize = g_prob_mean, g_z_loss, g_load_balance, normalize
        self.dx_r = self.dw_r = None


def moe_backward(tensors, state, dO, needs, x_addend=None, router_tail=None):
    """``(dx, dW1, dW2, dS)`` for ``needs = (x, W1, W2, S)``.

    ``x_addend``: called with ``dS`` (on the caller's stream) once it exists and before the dX combine;
    what it returns ([T,H], activation dtype, or None) is added to ``dx`` inside the combine kernel.
    It is how a caller that owns another path from ``x`` to the loss (the router) avoids a separate
    sum of the two gradients.  ``router_tail``: the router's side of that path; where the one-launch
    backward applies and the library can hold the router's backward in it, its outputs are stored in
    the object before ``x_addend`` is called."""
    lib = _lib.load()
    (x, gate_up_proj, down_proj, pre_act, weights_flat, expert_start, x_gather, s_scatter, s_reverse) = tensors[:9]
    T, K, E, H, I = state.dims
    TK = T * K
    dev = dO.device
    if dO.dtype != x.dtype:
        dO = dO.to(x.dtype)
    act = _lib.dtype_code(x.dtype)
    stream = _lib.stream_of(dO)
    need_x, need_w1, need_w2, need_s = needs

    # Kernels that do not depend on one another run side by side: the transposed copy of W1 (needed
    # by dX only) next to the dO*W2 GEMM, and then dW2, dW1 and dX, which depend only on what that
    # GEMM wrote; the two weight-gradient GEMMs have fewer tiles than the chip has CUs.  Two side
    # streams (default priority) are forked from and joined to the caller's stream with events;
    # everything they read stays referenced until the join has been enqueued.
    main = torch.cuda.current_stream(dev)
    overlap = SWITCHES.overlap
    side = [_side_stream(dev, 0), _side_stream(dev, 1)] if overlap else [main, main]

    def fork(*to):
        # one marker on the caller's stream, however many side streams wait for it
        if overlap:
            ev = torch.cuda.Event()
            ev.record(main)
            for s in to:
                s.wait_event(ev)

    def join(frm):
        if overlap:
            ev = torch.cuda.Event()
            ev.record(frm)
            main.wait_event(ev)

    # The ring kernels read the weights in their stored layout (bf16, whole 64-wide k-tiles);
    # other contracts get transposed copies, W1's made on a side stream next to the dO*W2 GEMM.
    as_stored = bool(lib.mts_moe_bwd_weights_as_stored(act, H, I))
    w1_bwd = None
    if need_x:
        if as_stored:
            # [E, 2I, H]: the parameter itself, or the forward pass's cast of an fp32 parameter
            w1_bwd = state.staged[0] if state.staged[0] is not None else _stage(lib, gate_up_proj, False, x.dtype)
        else:
            fork(side[0])
            w1_bwd = _stage(lib, gate_up_proj, True, x.dtype, side[0].cuda_stream)  # [E, H, 2I]
            w1t_ready = torch.cuda.Event() if overlap else None
            if overlap:
                w1t_ready.record(side[0])

    if as_stored and state.staged[1] is not None:
        w2_bwd = state.staged[1]
    else:
        w2_bwd = _stage(lib, down_proj, not as_stored, x.dtype)  # [E, H, I] as stored, else [E, I, H]
    d_pre_act = torch.empty(TK, 2 * I, dtype=x.dtype, device=dev)
    # s * silu(g) * u: the forward pass's post_act where it carries the routing weight, else written by dY1
    weighted_act = tensors[9] if state.weighted else torch.empty(TK, I, dtype=x.dtype, device=dev)
    n_part = lib.mts_moe_ds_partials(I)
    ds_part = torch.empty(TK, n_part, dtype=torch.float32, device=dev)
    # When every gradient is wanted, dW1, dW2, dX and the dS reduction go out as ONE launch whose block
    # order starts the long weight-gradient tiles first; no side stream is involved.  Which XCD runs which of
    # its units and dX tiles follows a table that the dO * W2 launch writes on the side (uneven routing).
    joint = (
        SWITCHES.joint_bwd and need_x and need_w1 and need_w2 and need_s and as_stored
        and gate_up_proj.dtype == down_proj.dtype and bool(lib.mts_moe_bwd_joint_supported(act, H, I))
    )
    ws1, ws1_ptr, ws1_bytes = _dw_workspace(lib, 1, E, H, I, x.dtype, dev) if need_w1 else (None, 0, 0)
    ws2, ws2_ptr, ws2_bytes = _dw_workspace(lib, 2, E, H, I, x.dtype, dev) if need_w2 else (None, 0, 0)
    schedule = None
    if joint and SWITCHES.joint_schedule and ws1 is not None and ws2 is not None:
        sched_bytes = lib.mts_moe_bwd_schedule_bytes(E)
        if sched_bytes > 0:
            schedule = torch.empty(sched_bytes // 4, dtype=torch.int32, device=dev)
    _lib.check(
        lib.mts_moe_bwd_dy1(
            dO.data_ptr(), w2_bwd.data_ptr(), int(as_stored), pre_act.data_ptr(), weights_flat.data_ptr(),
            x_gather.data_ptr(),
            s_scatter.data_ptr(), expert_start.data_ptr(), T, K, E, H, I, act, d_pre_act.data_ptr(),
            None if state.weighted else weighted_act.data_ptr(), ds_part.data_ptr(), _lib.ptr(schedule), stream,
        ),
        "mts_moe_bwd_dy1",
    )

    ddown_proj = None

    def combine_dx(dx_expanded, d_weights):
        addend = x_addend(d_weights) if x_addend is not None else None
        dx = torch.empty(T, H, dtype=x.dtype, device=dev)
        _lib.check(
            lib.mts_moe_combine(
                dx_expanded.data_ptr(), None, _lib.ptr(addend), s_reverse.data_ptr(), T, K, H, act, dx.data_ptr(), stream
            ),
            "mts_moe_combine",
        )
        return dx

    if joint:
        dgate_up_proj, ddown_proj = torch.empty_like(gate_up_proj), torch.empty_like(down_proj)
        d_weights = torch.empty(T, K, dtype=weights_flat.dtype, device=dev)
        dx_expanded = torch.empty(TK, H, dtype=x.dtype, device=dev)
        joint_args = (
            dO.data_ptr(), weighted_act.data_ptr(), d_pre_act.data_ptr(), x.data_ptr(), w1_bwd.data_ptr(),
            x_gather.data_ptr(), expert_start.data_ptr(), s_reverse.data_ptr(), ds_part.data_ptr(), T, K, E, H, I,
            act, _lib.dtype_code(gate_up_proj.dtype), dx_expanded.data_ptr(), dgate_up_proj.data_ptr(),
            ddown_proj.data_ptr(), d_weights.data_ptr(), ws1_ptr, ws1_bytes, ws2_ptr, ws2_bytes,
        )
        sched_ptr = _lib.ptr(schedule)
        rt = router_tail
        if rt is not None and SWITCHES.tail_in_joint and lib.mts_moe_bwd_joint_router_supported(act, T, H, I, E):
            # the router's backward as trailing blocks of the same launch: it needs nothing the launch writes
            dx_r, dw_r = torch.empty_like(x), torch.empty_like(rt.router_weight)
            dx = torch.empty_like(x) if SWITCHES.combine_in_tail else None
            rws_bytes = lib.mts_moe_head_bwd_workspace_bytes(T, H, E)
            rws = torch.empty(rws_bytes, dtype=torch.uint8, device=dev)
            _lib.check(
                lib.mts_moe_bwd_joint_router(
                    *joint_args, rt.router_weight.data_ptr(), rt.logits.data_ptr(), rt.weights.data_ptr(),
                    rt.indices.data_ptr(), _lib.ptr(rt.counts), _lib.ptr(rt.g_prob_mean), _lib.ptr(rt.g_z_loss),
                    _lib.ptr(rt.g_load_balance), int(rt.normalize), dx_r.data_ptr(), _lib.ptr(dx), dw_r.data_ptr(),
                    rws.data_ptr(), rws_bytes, sched_ptr, stream,
                ),
                "mts_moe_bwd_joint_router",
            )
            rt.dx_r, rt.dw_r = dx_r, dw_r
            if dx is None:
                return combine_dx(dx_expanded, d_weights), dgate_up_proj, ddown_proj, d_weights
            if x_addend is not None:
                x_addend(d_weights)   # lets the caller pick the router's outputs up; the combine has been launched
            return dx, dgate_up_proj, ddown_proj, d_weights
        _lib.check(lib.mts_moe_bwd_joint(*joint_args, sched_ptr, stream), "mts_moe_bwd_joint")
        return combine_dx(dx_expanded, d_weights), dgate_up_proj, ddown_proj, d_weights

    if need_w1 and need_w2:
        fork(side[0], side[1])
    elif need_w2:
        fork(side[0])
    elif need_w1:
        fork(side[1])
    # the routing-weight gradient is needed after the join only: it leads one of the side streams
    # (when there is one) so that dX follows the dO*W2 GEMM directly on the caller's stream; a caller
    # that takes it before the dX combine gets it on its own stream
    d_weights = None
    if need_s:
        ds_stream = stream if x_addend is not None else (
            side[0].cuda_stream if need_w2 else (side[1].cuda_stream if need_w1 else stream))
        d_weights = torch.empty(T, K, dtype=weights_flat.dtype, device=dev)
        _lib.check(
            lib.mts_moe_bwd_ds(
                ds_part.data_ptr(), s_reverse.data_ptr(), TK, I, act, d_weights.data_ptr(), ds_stream
            ),
            "mts_moe_bwd_ds",
        )

    if need_w2:
        ddown_proj = torch.empty_like(down_proj)
        _lib.check(
            lib.mts_moe_bwd_dw2(
                dO.data_ptr(), weighted_act.data_ptr(), x_gather.data_ptr(), expert_start.data_ptr(), T, K, E, H,
                I, act, _lib.dtype_code(down_proj.dtype), ddown_proj.data_ptr(), ws2_ptr, ws2_bytes,
                side[0].cuda_stream,
            ),
            "mts_moe_bwd_dw2",
        )

    dgate_up_proj = None
    if need_w1:
        dgate_up_proj = torch.empty_like(gate_up_proj)
        _lib.check(
            lib.mts_moe_bwd_dw1(
                d_pre_act.data_ptr(), x.data_ptr(), x_gather.data_ptr(), expert_start.data_ptr(), T, K, E, H, I,
                act, _lib.dtype_code(gate_up_proj.dtype), dgate_up_proj.data_ptr(), ws1_ptr, ws1_bytes,
                side[1].cuda_stream,
            ),
            "mts_moe_bwd_dw1",
        )

    dx = None
    if need_x:
        if overlap and not as_stored:
            main.wait_event(w1t_ready)
        dx_expanded = torch.empty(TK, H, dtype=x.dtype, device=dev)
        _lib.check(
            lib.mts_moe_bwd_dx(
                d_pre_act.data_ptr(), w1_bwd.data_ptr(), int(as_stored), expert_start.data_ptr(), TK, E, H, I,
                act, dx_expanded.data_ptr(), stream,
            ),
            "mts_moe_bwd_dx",
        )
        dx = combine_dx(dx_expanded, d_weights)

    if need_w2 or need_x:
        join(side[0])
    if need_w1:
        join(side[1])

    return dx, dgate_up_proj, ddown_proj, d_weights


class _FusedMoEFunction(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(ctx, x, gate_up_proj, down_proj, top_k_index, top_k_weights):
        T, K = top_k_index.shape
        E = gate_up_proj.shape[0]
        with torch.no_grad():
            routing = routing_for_experts(top_k_index, E)
        weights_flat = top_k_weights.flatten().contiguous()
        out, tensors, state = moe_forward(x, gate_up_proj, down_proj, weights_flat, routing)
        ctx.save_for_backward(*tensors)
        ctx.state = state
        ctx.mark_non_differentiable(top_k_index)
        ctx.set_materialize_grads(False)
        return out

    @staticmethod
    @ensure_contiguous
    def backward(ctx, dO):
        if dO is None:
            return None, None, None, None, None
        need_x, need_w1, need_w2, _, need_s = ctx.needs_input_grad
        dx, dw1, dw2, ds = moe_backward(ctx.saved_tensors, ctx.state, dO, (need_x, need_w1, need_w2, need_s))
        return dx, dw1, dw2, None, ds


def _width_granule(dtype: torch.dtype) -> int:
    """The kernels move 16 bytes per lane: rows must be a whole number of 16-byte chunks."""
    return 4 if dtype == torch.float32 else 8


def needs_padding(x, gate_up_proj) -> bool:
    g = _width_granule(x.dtype)
    return x.shape[1] % g != 0 or (x.dtype != torch.float32 and (gate_up_proj.shape[1] // 2) % g != 0)


def _padded_operands(x, gate_up_proj, down_proj):
    """Zero-padded copies whose widths are whole 16-byte chunks: H -> H8 everywhere, I -> I8 with the gate
    rows at 0.. and the up rows at I8...  Zero columns and rows contribute nothing to any product, so the
    operator's result on the padded operands, cut back to H columns, is the result on the originals; the
    copies are made with differentiable torch ops, so the gradients come back cut to size as well."""
    g = _width_granule(x.dtype)
    E, two_i, H = gate_up_proj.shape
    I = two_i // 2
    H8 = -(-H // g) * g
    I8 = I if x.dtype == torch.float32 else -(-I // g) * g
    pad = torch.nn.functional.pad
    gate, up = gate_up_proj[:, :I], gate_up_proj[:, I:]
    w1 = torch.cat([pad(gate, (0, H8 - H, 0, I8 - I)), pad(up, (0, H8 - H, 0, I8 - I))], dim=1)
    return pad(x, (0, H8 - H)), w1, pad(down_proj, (0, I8 - I, 0, H8 - H))


def fused_moe(x, gate_up_proj, down_proj, top_k_index, top_k_weights):
    missed = fused_moe_violation(x, gate_up_proj, down_proj, top_k_index, top_k_weights)
    if missed is not None:
        raise RuntimeError(f"Unsupported tensor contract for hip fused MoE: it requires {missed}")
    if needs_padding(x, gate_up_proj):
        # widths that are not whole 16-byte chunks (legal in the reference, minitrain/kernels/triton/fused_moe.py:55-70)
        H = x.shape[1]
        xp, w1p, w2p = _padded_operands(x, gate_up_proj, down_proj)
        return _FusedMoEFunction.apply(xp, w1p, w2p, top_k_index, top_k_weights)[:, :H]
    return _FusedMoEFunction.apply(x, gate_up_proj, down_proj, top_k_index, top_k_weights)
