"""einsummable_amd: MI355X (gfx950) kernel manager for einsummable apply nodes.

The product is the C-ABI shared library ``libes_km.so`` (``include/es_km.h``).  This module
is the thin ctypes loader used by the tests, the smoke test and the benchmark; it mirrors
the reference's ``kernel_manager_t`` members (build / workspace_size / call / touch /
constant_fill / lowerTri_fill, src/engine/gpu/gpu_kernel_manager.h:274-321) and adds
nothing of its own: every call goes straight to the library and fails loudly when the
library is missing.
"""
from .km import (  # noqa: F401
    ApplyGraph,
    C64,
    F16,
    F32,
    F64,
    Einsummable,
    KernelManager,
    KmError,
    NodeCallback,
    StreamPool,
    WorkspacePool,
    Touch,
    TouchBatch,
    codegen_source,
    lib_path,
    load_library,
    memgraph_describe,
    merge_adjacent_dims,
    scalarop_roundtrip,
    scalarop_simplify,
)
