"""MI355X-native `hip` operator backend for the fused top-k MoE layer.

Host-side mirror of the reference's operator interface for this one path:
``model/ops.py`` (the ``OpsBackend`` contract and ``get_ops_backend``),
``kernels/hip`` (the backend whose ``router_postprocess`` and ``fused_moe`` run
hand-written gfx950 kernels through a C ABI) and ``model/moe_router.py`` /
``model/blocks.py`` (the MoE block that calls them).
"""

__all__ = ["__version__"]
__version__ = "0.1.0"
