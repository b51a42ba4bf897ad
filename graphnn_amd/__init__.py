"""graphnn_amd — MI355X (gfx950) backend for graphnn's structure2vec mean-field forward.

The product is the HIP library graphnn_amd/lib/libgnnhip.so behind the C ABI of
include/gnnhip.h.  This package only loads it (ctypes) and offers thin helpers
that pass torch device pointers through; torch is used for device memory and
streams, never for the arithmetic.
"""
from ._lib import load_library, library_path, GnnHipError  # noqa: F401
