"""ctypes binding of ``libmts_moe.so`` (declared in ``include/mts_moe.h``).

The library is loaded after torch so that its HIP symbols bind to the runtime
torch already brought into the process.  There is no fallback: a missing library
raises, and so does every non-zero return code.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch  # noqa: F401  (must be imported before the library is opened)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmts_moe.so")

MTS_BF16 = 0
MTS_F32 = 1
MTS_F16 = 2

_c = ctypes
_p = _c.c_void_p
_i = _c.c_int
_l = _c.c_int64

# name -> (restype, argtypes); one entry per declaration in include/mts_moe.h
SIGNATURES = {
    "mts_version": (_i, []),
    "mts_error_string": (_c.c_char_p, [_i]),
    "mts_router_workspace_bytes": (_l, [_l, _i]),
    "mts_router_fwd": (_i, [_p, _l, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _l, _p]),
    "mts_router_bwd": (_i, [_p, _p, _p, _p, _p, _i, _p, _p, _p, _p, _l, _i, _i, _i, _p, _p]),
    "mts_router_logits_fwd": (_i, [_p, _p, _l, _i, _i, _i, _p, _p]),
    "mts_router_logits_bwd_workspace_bytes": (_l, [_l, _i, _i]),
    "mts_router_logits_bwd": (_i, [_p, _p, _p, _l, _i, _i, _i, _p, _p, _p, _l, _p]),
    "mts_moe_route_workspace_bytes": (_l, [_l, _i, _i]),
    "mts_moe_route": (_i, [_p, _l, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _p, _l, _p]),
    "mts_moe_route_static": (_i, [_p, _l, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _p]),
    "mts_moe_capacity_workspace_bytes": (_l, [_l, _i, _i]),
    "mts_moe_capacity_mask": (_i, [_p, _p, _l, _i, _i, _l, _p, _p, _p, _p, _l, _p]),
    "mts_moe_stage_weights": (_i, [_p, _i, _p, _i, _i, _l, _l, _i, _p]),
    "mts_moe_cast_weights_pair": (_i, [_p, _p, _l, _p, _p, _l, _i, _p]),
    "mts_moe_fwd_gateup_swiglu": (_i, [_p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _p, _p]),
    "mts_moe_fwd_down": (_i, [_p, _p, _p, _l, _i, _i, _i, _i, _p, _p]),
    "mts_moe_fwd_joint_supported": (_i, [_i, _i, _i]),
    "mts_moe_fwd_joint_workspace_bytes": (_l, [_l, _i]),
    "mts_moe_fwd_gateup_down": (_i, [_p] * 7 + [_l, _i, _i, _i, _i, _i, _p, _p, _p, _p, _l, _p]),
    "mts_moe_combine": (_i, [_p, _p, _p, _p, _l, _i, _i, _i, _p, _p]),
    "mts_moe_head_workspace_bytes": (_l, [_l, _i, _i]),
    "mts_moe_head_fwd": (_i, [_p, _p, _l, _i, _i, _i, _i, _i] + [_p] * 14 + [_p, _l, _p]),
    "mts_moe_head_bwd_workspace_bytes": (_l, [_l, _i, _i]),
    "mts_moe_head_bwd": (_i, [_p] * 11 + [_l, _i, _i, _i, _i, _i, _p, _p, _p, _l, _p]),
    "mts_moe_ds_partials": (_i, [_i]),
    "mts_probe_mfma_sink_bytes": (_l, [_i]),
    "mts_probe_mfma_rate": (_i, [_i, _i, _i, _p, _l, _p, _p]),
    "mts_moe_bwd_weights_as_stored": (_i, [_i, _i, _i]),
    "mts_moe_bwd_dy1": (_i, [_p, _p, _i, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p]),
    "mts_moe_bwd_schedule_bytes": (_l, [_i]),
    "mts_moe_bwd_schedule": (_i, [_p, _l, _i, _p, _p]),
    "mts_moe_bwd_ds": (_i, [_p, _p, _l, _i, _i, _p, _p]),
    "mts_moe_bwd_dx": (_i, [_p, _p, _i, _p, _l, _i, _i, _i, _i, _p, _p]),
    "mts_moe_bwd_dw_workspace_bytes": (_l, [_i, _i, _i, _i]),
    "mts_moe_bwd_dw2": (_i, [_p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _i, _p, _p, _l, _p]),
    "mts_moe_bwd_dw1": (_i, [_p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _i, _p, _p, _l, _p]),
    "mts_moe_bwd_joint_supported": (_i, [_i, _i, _i]),
    "mts_moe_bwd_joint": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p, _l, _p, _l, _p, _p]),
    "mts_moe_bwd_joint_router_supported": (_i, [_i, _l, _i, _i, _i]),
    "mts_moe_bwd_joint_router": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p, _l, _p, _l]
                                 + [_p] * 8 + [_i, _p, _p, _p, _p, _l, _p, _p]),
}

_lib = None
_lock = threading.Lock()


class MtsError(RuntimeError):
    pass


def load():
    """Open the library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise MtsError(
                    f"{LIB_PATH} is missing: build it with `python -m minitrain_amd.build` "
                    "(there is no fallback for the hip backend)"
                )
            lib = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().mts_error_string(code).decode()
        raise MtsError(f"{what} failed: {msg} (code {code})")


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def stream_of(t) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def dtype_code(dt) -> int:
    if dt == torch.bfloat16:
        return MTS_BF16
    if dt == torch.float32:
        return MTS_F32
    if dt == torch.float16:
        return MTS_F16
    raise MtsError(f"unsupported dtype {dt}")
