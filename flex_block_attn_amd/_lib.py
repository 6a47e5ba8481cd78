"""ctypes binding of libfba_gfx950.so (the C ABI declared in include/fba.h).

There is no CPU or PyTorch fallback: if the library has not been built, or a call fails, an exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# FBA_LIBRARY points the loader at another build of the same ABI (an instrumented or experimental one)
LIB_PATH = os.environ.get("FBA_LIBRARY") or os.path.join(_HERE, "csrc", "libfba_gfx950.so")

FBA_OK = 0
FBA_ERR_INVALID = 1
FBA_ERR_UNSUPPORTED = 2
FBA_ERR_HIP = 3

_c_i32 = ctypes.c_int32
_c_i64 = ctypes.c_int64
_c_ptr = ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/fba.h one to one
SIGNATURES = {
    "fba_version": (_c_i32, []),
    "fba_last_error": (ctypes.c_char_p, []),
    "fba_mask_compact": (_c_i32, [_c_ptr, _c_i64, _c_i32, _c_i32, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "fba_split_workspace_bytes": (_c_i64, []),
    "fba_fwd": (_c_i32, [_c_ptr] * 7 + [_c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_bwd": (_c_i32, [_c_ptr] * 14 + [_c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_probe_mfma": (_c_i32, [_c_ptr, _c_ptr, _c_i32, _c_i32, _c_ptr]),
    "fba_probe_read": (_c_i32, [_c_ptr, _c_i64, _c_ptr, _c_i32, _c_ptr]),
    "fba_pair_slots": (_c_i32, [_c_ptr] * 4 + [_c_i64, _c_i32, _c_i32, _c_ptr, _c_ptr, _c_ptr]),
    "fba_bwd_handover": (_c_i32, [_c_ptr] * 8 + [_c_i64] + [_c_ptr] * 9 + [_c_i64, _c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_bwd_dkdv_handover": (_c_i32, [_c_ptr] * 8 + [_c_i64] + [_c_ptr] * 3 + [_c_i64, _c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_bwd_dq_from_ds": (_c_i32, [_c_ptr] * 2 + [_c_i64] + [_c_ptr] * 5 + [_c_i64, _c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_tile_slots": (_c_i32, [_c_ptr, _c_ptr, _c_i64, _c_i32, _c_i32, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "fba_bwd_tiled_handover": (_c_i32, [_c_ptr] * 8 + [_c_i64] + [_c_ptr] * 10 + [_c_i64, _c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_bwd_noalloc": (_c_i32, [_c_ptr] * 13 + [_c_i64] + [_c_i32] * 8 + [_c_ptr]),
    "fba_tile_lists": (_c_i32, [_c_ptr, _c_i64, _c_i32, _c_i32, _c_i32, _c_i32, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "fba_block_mean": (_c_i32, [_c_ptr, _c_ptr, _c_i64, _c_i32, _c_i32, _c_i32, _c_ptr]),
    "fba_ssta_mask": (_c_i32, [_c_ptr, _c_ptr, _c_ptr, _c_ptr] + [_c_i32] * 10 + [_c_ptr]),
    "fba_tile_permute": (_c_i32, [_c_ptr, _c_ptr, _c_i64] + [_c_i32] * 8 + [_c_ptr]),
    "fba_fwd_tiled": (_c_i32, [_c_ptr] * 7 + [_c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_bwd_tiled": (_c_i32, [_c_ptr] * 14 + [_c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_bwd_stats": (_c_i32, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i32, _c_ptr]),
    "fba_bwd_dq": (_c_i32, [_c_ptr] * 8 + [_c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
    "fba_bwd_dkdv": (_c_i32, [_c_ptr] * 9 + [_c_i64] + [_c_i32] * 8 + [_c_ptr, _c_i64, _c_ptr]),
}

# fba_version() of the library these signatures describe (include/fba.h; bumped whenever an argument list changes)
ABI_VERSION = 2003

_lib = None


class FbaError(RuntimeError):
    """A call into libfba_gfx950.so returned an error code."""

    def __init__(self, code, message):
        super().__init__(f"libfba_gfx950 error {code}: {message}")
        self.code = code
        self.message = message


def load():
    """Load the shared library (once) and declare every entry point. Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m flex_block_attn_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.fba_version.restype = _c_i32
    lib.fba_version.argtypes = []
    if lib.fba_version() != ABI_VERSION:  # argument lists below belong to exactly this version
        raise ImportError(
            f"{LIB_PATH} reports version {lib.fba_version()}, this package binds version {ABI_VERSION}: "
            "rebuild it with `python -m flex_block_attn_amd.build`."
        )
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code):
    if code != FBA_OK:
        raise FbaError(code, load().fba_last_error().decode("utf-8", "replace"))


def call(name, *args):
    """Call an entry point and raise FbaError on a non-zero return."""
    check(getattr(load(), name)(*args))
