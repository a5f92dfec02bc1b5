"""ctypes binding of libmuon_amd.so (the C ABI declared in include/muon_amd.h).

The library is built in-tree by `python -m muon_amd.build` (or `__graft_entry__.build()`); there
is no fallback implementation: if it is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# MUON_AMD_LIBRARY: path of another build of the library (for comparing builds side by side)
LIB_PATH = os.environ.get("MUON_AMD_LIBRARY") or os.path.join(_HERE, "libmuon_amd.so")

ABI_VERSION = 3
ROUND_REFERENCE = 1
ROUND_FUSED = 0
NORM_UNIT = 2
GEMM_ROWSUM = 4
GEMM_Q_KMAJOR = 8
AOL_SYMMETRIC = 0
AOL_ROWS_ONLY = 1
SRC_F32 = 0
SRC_BF16 = 1

# numpy mirrors of the C structs (align=True reproduces the C layout; sizes are checked against
# the library's own sizeof at load time).
MAT_DESC = np.dtype(
    [("grad", "<u8"), ("momentum", "<u8"), ("param", "<u8"), ("out", "<u8"), ("u", "<u8"),
     ("direct", "<u8"), ("transp", "<u8"), ("result", "<u8"), ("partials", "<u8"),
     ("denom", "<u8"), ("rows", "<i4"), ("cols", "<i4"), ("rows_p", "<i4"), ("cols_p", "<i4"),
     ("ld_direct", "<i4"), ("ld_transp", "<i4"), ("src_dtype", "<i4"), ("scale", "<f4"), ("part_begin", "<i4"), ("part_end", "<i4")],
    align=True)
GEMM_DESC = np.dtype(
    [("P", "<u8"), ("Q", "<u8"), ("D", "<u8"), ("C", "<u8"), ("CT", "<u8"), ("C2", "<u8"),
     ("C2T", "<u8"), ("ldp", "<i4"), ("ldq", "<i4"), ("ldd", "<i4"), ("ldc", "<i4"),
     ("ldct", "<i4"), ("K", "<i4"), ("rows", "<i4"), ("colsn", "<i4"),
     ("rowsum", "<u8"), ("ld_rowsum", "<i4"), ("q_kmajor", "<i4")],
    align=True)
TILE_JOB = np.dtype([("desc", "<i4"), ("i0", "<i4"), ("j0", "<i4"), ("diag", "<i4"), ("k0", "<i4"),
                     ("k1", "<i4"), ("part_base", "<i4"), ("split", "<i4")], align=True)
ADAM_DESC = np.dtype(
    [("param", "<u8"), ("grad", "<u8"), ("exp_avg", "<u8"), ("exp_avg_sq", "<u8"),
     ("update", "<u8"), ("numel", "<i8"), ("dtype", "<i4"), ("reserved", "<i4")],
    align=True)

AOL_DESC = np.dtype(
    [("xr", "<u8"), ("xc", "<u8"), ("gram", "<u8"), ("rvec", "<u8"), ("rowsum", "<u8"),
     ("m_p", "<i4"), ("n_p", "<i4"), ("ld_n", "<i4"), ("ld_m", "<i4"), ("ld_rowsum", "<i4"), ("reserved", "<i4")],
    align=True)

_c_int = ctypes.c_int
_c_float = ctypes.c_float
_vp = ctypes.c_void_p

# name -> (restype, argtypes); every symbol include/muon_amd.h declares.
SIGNATURES = {
    "muon_amd_abi_version": (_c_int, []),
    "muon_amd_last_error": (ctypes.c_char_p, []),
    "muon_amd_init": (_c_int, []),
    "muon_amd_sizeof_mat_desc": (ctypes.c_size_t, []),
    "muon_amd_sizeof_gemm_desc": (ctypes.c_size_t, []),
    "muon_amd_sizeof_tile_job": (ctypes.c_size_t, []),
    "muon_amd_sizeof_adam_desc": (ctypes.c_size_t, []),
    "muon_amd_sizeof_aol_desc": (ctypes.c_size_t, []),
    "muon_amd_aol_rows_per_block": (_c_int, []),
    "muon_amd_validate_aol": (_c_int, [_vp, _c_int, _vp, _vp]),
    "muon_amd_aol_rowsum": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _vp]),
    "muon_amd_aol_rowsum_finalize": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _vp]),
    "muon_amd_aol_rescale": (_c_int, [_vp, _vp, _c_int, _c_int, _c_int, _vp]),
    "muon_amd_elementwise_block_elems": (_c_int, []),
    "muon_amd_normalize_tile": (_c_int, []),
    "muon_amd_gemm_tile_rows": (_c_int, [_c_int]),
    "muon_amd_gemm_tile_cols": (_c_int, [_c_int]),
    "muon_amd_validate_gemm": (_c_int, [_vp, _c_int, _vp, _c_int, _c_int, _c_int]),
    "muon_amd_validate_mats": (_c_int, [_vp, _c_int, _vp, _vp, _c_int]),
    "muon_amd_momentum": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _c_float, _c_int, _c_int, _vp, _vp]),
    "muon_amd_norm_finalize": (_c_int, [_vp, _c_int, _c_float, _c_int, _vp]),
    "muon_amd_normalize": (_c_int, [_vp, _vp, _c_int, _c_int, _vp]),
    "muon_amd_ns_gemm": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _c_float, _c_float, _c_int, _vp, _vp, _vp]),
    "muon_amd_ns_gemm_apply": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _c_float, _c_int, _vp, _c_float, _c_float, _vp, _vp]),
    "muon_amd_noalloc_max_split_slots": (_c_int, []),
    "muon_amd_ns_gemm_noalloc": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _c_float, _c_float, _c_int, _c_int, _vp]),
    "muon_amd_apply": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _c_float, _vp, _vp]),
    "muon_amd_adam": (_c_int, [_vp, _vp, _c_int, _c_int, _c_float, _c_float, _c_float, _c_float,
                               _c_float, _c_float, _c_float, _vp, _vp]),
}


class MuonAmdError(RuntimeError):
    pass


_lib = None


def load():
    """Load libmuon_amd.so once; raise if it is missing or its ABI does not match."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MuonAmdError(
            f"{LIB_PATH} is missing: build it with `python -m muon_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.muon_amd_abi_version() != ABI_VERSION:
        raise MuonAmdError(f"ABI mismatch: library {lib.muon_amd_abi_version()}, binding {ABI_VERSION}")
    for dt, fn in ((MAT_DESC, lib.muon_amd_sizeof_mat_desc), (GEMM_DESC, lib.muon_amd_sizeof_gemm_desc),
                   (TILE_JOB, lib.muon_amd_sizeof_tile_job), (ADAM_DESC, lib.muon_amd_sizeof_adam_desc),
                   (AOL_DESC, lib.muon_amd_sizeof_aol_desc)):
        if dt.itemsize != fn():
            raise MuonAmdError(f"struct layout mismatch: binding {dt.itemsize} bytes, library {fn()}")
    _lib = lib
    return lib


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        msg = load().muon_amd_last_error().decode("utf-8", "replace")
        raise MuonAmdError(f"{what or 'libmuon_amd'} failed (code {rc}): {msg}")


def host_ptr(arr: np.ndarray) -> int:
    assert arr.flags["C_CONTIGUOUS"]
    return arr.ctypes.data
