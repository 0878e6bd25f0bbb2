"""MI355X-native int4 GPT-2 inference path for async_gpu: Python binding of libagpu_hip.so.

The directory name carries a hyphen, so import it through `load_package()` of the
repository's __graft_entry__.py (or importlib) under the module name `async_gpu_amd`.
The compute lives in the HIP library; this package only binds its C ABI (ctypes) and
mirrors the reference's `nn` surface for tests and the benchmark.  There is no CPU
fallback: every operator raises if the library is missing.
"""
from . import _lib  # noqa: F401
from ._lib import AgpuError, Context, lib_path, library_available  # noqa: F401
