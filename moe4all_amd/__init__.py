"""MI355X (gfx950) backend for the routed-expert MoE FFN path of the MoE4All engine.

The product is ``libinfr_hip.so`` (hand-written HIP kernels behind the C ABI declared in
``include/infr_hip.h``).  This package is a thin ctypes view of that ABI with the names of
the reference's Rust interface (``Backend``, ``Buffer``, ``Plan``, ``Bindings``, ``Graph``,
``Op``), so tests read like the reference's own one-op parity harness
(crates/infr-testkit/src/lib.rs:170-201).  No computation happens in Python and there is no
CPU fallback: without the library or without a gfx950 device, construction raises.
"""
from .backend import (  # noqa: F401
    Activation,
    Backend,
    BackendError,
    Bindings,
    Buffer,
    BufferUsage,
    DType,
    Graph,
    MoeGating,
    Plan,
    TensorDesc,
    TensorKind,
    Unsupported,
    build_library,
    library_path,
    load_library,
    run_graph,
)

__all__ = [
    "Activation", "Backend", "BackendError", "Bindings", "Buffer", "BufferUsage", "DType", "Graph",
    "MoeGating", "Plan", "TensorDesc", "TensorKind", "Unsupported", "build_library", "library_path",
    "load_library", "run_graph",
]
