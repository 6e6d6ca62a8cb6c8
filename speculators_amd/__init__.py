"""MI355X-native draft-model training hot path (EAGLE3 / DFlash forward +
backward) behind the plug-in points of vllm-project/speculators.

The compute lives in ``libspx_hip.so`` (hand-written gfx950 HIP kernels behind
a C ABI, declared in ``include/spx.h``); this package is the host side: ctypes
bindings, autograd wrappers, and mirrors of the reference's attention-function
and loss-function registries and of its draft-model ``forward`` API.
"""

__version__ = "0.1.0"
