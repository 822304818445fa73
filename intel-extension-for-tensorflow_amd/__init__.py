"""MI355X-native INT8 quantized-inference kernels behind ITEX's op interface.

The product is native: `lib/libitexhip.so` (HIP kernels + C ABI, include/itexhip.h) and
`lib/libitex_amd.so` (the TensorFlow PluggableDevice kernel plugin exporting TF_InitKernel).
This Python package only binds the C ABI with ctypes for tests and benchmarks; it holds no
arithmetic and no fallback: if the native library is missing, importing `itexhip` raises.

The directory name is not a Python identifier; load it with `load_package()` from
`__graft_entry__.py` or import `itexhip` after putting this directory on sys.path.
"""
from . import itexhip  # noqa: F401
