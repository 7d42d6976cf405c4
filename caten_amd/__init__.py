"""caten_amd: an MI355X (gfx950) `:HIP` execution backend for Caten's BYOC interface.

The product is libcaten_hip.so (C ABI in include/caten_hip.h): a HIP runtime
(caching allocator, hipRTC, module launch) plus hand-written CDNA4 kernels for
the fused items of a GPT-2 / Llama shaped batch-1 decode.  This package is the
host-side mirror of Caten's backend interface over that ABI.
"""
from . import _lib  # noqa: F401
from ._lib import HipError  # noqa: F401
from .backend import define_backend, get_backend_buffer, get_backend_runtime, get_backend_renderer  # noqa: F401
from .backend import get_buffer_type, get_runtime_type, jit_mode_p  # noqa: F401
from .buffer import AbstractBuffer, HipBuffer, make_buffer  # noqa: F401
from .runtime import GraphRuntime, HipRuntime, Node, CompiledKernel  # noqa: F401
from .renderer import HipRenderer  # noqa: F401
