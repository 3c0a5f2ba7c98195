"""MI355X (gfx950) backend for strix-halo-vulkan's language-model token loop.

The product is the C-ABI library libshv_hip.so (include/shv_hip.h); this package holds its HIP
sources (csrc/), the in-tree build (build.py) and a thin ctypes binding (hip_api) used by the
tests and the benchmark.  There is no CPU fallback: loading fails loudly when the library has not
been built, and every op fails when no gfx950 device is present.
"""
from . import gguf_api, hip_api, llm_api, sample_api, text_api  # noqa: F401
from .hip_api import Context, ShvError, lib_path, load  # noqa: F401
