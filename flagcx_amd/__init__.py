"""MI355X (gfx950) local reduce / chunk-copy kernels behind FlagCX's enums.

The product is flagcx_amd/lib/libflagcx_amd.so (C ABI, include/flagcx_amd.h).
`flagcx_amd.local` is a thin ctypes binding used by the tests and the benchmark;
it raises if the library has not been built - there is no fallback path.
"""
from .local import (  # noqa: F401
    DataType, RedOp, Result, FlagcxError, lib, lib_path,
)
