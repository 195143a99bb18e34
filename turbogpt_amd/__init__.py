"""MI355X-native training-step hot path of TurboGPT: HIP kernels + engine behind a C ABI.

The package is a thin ctypes loader; all compute lives in libturbogpt.so (built by
``python -m turbogpt_amd.build``).  Loading fails loudly when the library is missing.
"""
from .bridge import library, library_path  # noqa: F401
