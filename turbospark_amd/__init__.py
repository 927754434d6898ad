"""MI355X-native speculative-decoding verify step (target forward over the drafted rows,
acceptance, KV rollback) behind the reference's draft/verify/accept producer interface.

The compute lives in libtsverify.so (hand-written HIP for gfx950, C ABI in include/tsverify.h);
this package is the thin host-side mirror of that interface.  There is no CPU fallback: if
the library is missing, importing `turbospark_amd.ffi` raises.
"""
from .ffi import F32, F16, Q8_0, Q4_K, Q6_K, BF16, MXFP4, TsvError, lib, shaping  # noqa: F401
from .producer import HipVerifier, MtpHead, RoundResult  # noqa: F401
from . import synth  # noqa: F401
