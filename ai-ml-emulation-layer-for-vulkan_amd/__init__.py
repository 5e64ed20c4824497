"""MI355X-native execution backend for TOSA 1.0 data-graph operators.

The product is two shared libraries under csrc/: libmlel_hip.so (hand-written gfx950 kernels behind the C ABI
of include/mlel_hip.h) and libmlel_graph.so (the host-side operator surface: GraphPipeline, memory planner,
graph front-end).  The Python in this package is a thin ctypes harness over those libraries; it performs no
arithmetic and has no CPU fallback.

The directory name contains hyphens, so import it with
    importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd")
"""
from . import abi  # noqa: F401
