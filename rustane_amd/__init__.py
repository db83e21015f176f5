"""rustane_amd: an MI355X (gfx950) decode backend for rustane behind the reference's decode API.

The product is the C-ABI library `libhipdecode.so` (include/hip_decode.h) and the host engine
above it (`librustane_engine.so`: DecodeContext / InferenceSession / samplers).  This package is
the ctypes view of both, used by the tests and the benchmark.
"""
from .hipdec import HipDecodeModel, HipDecodeError, Config, WeightDtype, KvDtype  # noqa: F401
