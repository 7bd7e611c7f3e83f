"""faith_amd -- MI355X (gfx950) kernels for forward linear-bound propagation.

    from faith_amd import Bounds, ops

The HIP library is loaded on first use of `Bounds`, `ops` or `c_bound`; it is
built in-tree with `python -m faith_amd.build`.  There is no CPU fallback.
"""
import importlib

__all__ = ["Bounds", "CompactBounds", "BoundsMaker", "ConvBounds", "ops", "c_bound", "workloads"]


def __getattr__(name):
    if name in ("Bounds", "CompactBounds", "BoundsMaker", "ConvBounds"):
        return getattr(importlib.import_module(".bounds", __name__), name)
    if name in ("ops", "c_bound", "workloads", "build"):
        return importlib.import_module("." + name, __name__)
    raise AttributeError(name)
