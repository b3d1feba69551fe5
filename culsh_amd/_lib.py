"""
Loader and ctypes prototypes for libculsh_amd.so (the C ABI declared in
include/culsh_amd.h).

The library is built in-tree by `make -C culsh_amd/csrc` (or `__graft_entry__.build()`).
There is no fallback: if the shared object is missing or cannot be loaded, importing
anything that computes raises, because a CPU substitute would silently change what is
being measured.
"""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libculsh_amd.so")

# culsh_status
OK, ERR_INVALID, ERR_HIP, ERR_NOMEM, ERR_LIMIT, ERR_INTERNAL = range(6)
# culsh_kind
KIND_CORE, KIND_RPLSH, KIND_PSLSH, KIND_MINHASH = range(4)
# culsh_array
ARR_CANDIDATE_INDICES, ARR_BUCKET_SIGNATURES, ARR_BUCKET_CANDIDATE_OFFSETS, ARR_TABLE_BUCKET_OFFSETS = 0, 1, 2, 3
ARR_PROJECTION, ARR_BIAS, ARR_HASH_A, ARR_HASH_B = 4, 5, 6, 7
ARR_QUERY_INDICES, ARR_QUERY_COUNTS, ARR_QUERY_OFFSETS = 16, 17, 18


class IndexMeta(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("n_total_candidates", C.c_int32),
        ("n_total_buckets", C.c_int32),
        ("n_hash_tables", C.c_int32),
        ("n_hashes", C.c_int32),
        ("sig_nbytes", C.c_int32),
        ("n_features", C.c_int32),
        ("is_double", C.c_int32),
        ("window_size", C.c_int32),
        ("seed", C.c_uint64),
        ("size_bytes", C.c_uint64),
    ]


class CandidatesMeta(C.Structure):
    _fields_ = [
        ("n_queries", C.c_int32),
        ("n_total_candidates", C.c_uint64),
        ("is_empty", C.c_int32),
    ]


_P = C.c_void_p
_I = C.c_int
_U64 = C.c_uint64
_PP = C.POINTER(C.c_void_p)

# name -> argtypes (every function returns culsh_status unless listed in _SPECIAL)
PROTOTYPES = {
    "culsh_ctx_create": [_I, _PP],
    "culsh_ctx_synchronize": [_P],
    "culsh_profile_enable": [_P, _I],
    "culsh_profile_reset": [_P],
    "culsh_profile_filter": [_P, C.c_char_p],
    "culsh_profile_get": [_P, _I, C.POINTER(C.c_char_p), C.POINTER(C.c_double), C.POINTER(C.c_int64)],
    "culsh_generate_projection_f32": [_U64, _I, _I, _P],
    "culsh_generate_projection_f64": [_U64, _I, _I, _P],
    "culsh_generate_pslsh_params_f32": [_U64, _I, _I, _I, _P, _P],
    "culsh_generate_pslsh_params_f64": [_U64, _I, _I, _I, _P, _P],
    "culsh_generate_minhash_params": [_U64, _I, _P, _P],
    "culsh_generate_minhash_params_mod": [_U64, _I, C.c_uint32, _P, _P],
    "culsh_ctx_set_minhash_prime": [_P, C.c_uint32],
    "culsh_ctx_get_minhash_prime": [_P, C.POINTER(C.c_uint32)],
    "culsh_index_minhash_prime": [_P, C.POINTER(C.c_uint32)],
    "culsh_rplsh_fit_f32": [_P, _P, _I, _I, _I, _I, _U64, _P, _PP],
    "culsh_rplsh_fit_f64": [_P, _P, _I, _I, _I, _I, _U64, _P, _PP],
    "culsh_rplsh_query_f32": [_P, _P, _I, _P, _I, _PP],
    "culsh_rplsh_query_f64": [_P, _P, _I, _P, _I, _PP],
    "culsh_rplsh_fit_query_f32": [_P, _P, _I, _I, _I, _I, _U64, _P, _PP],
    "culsh_rplsh_fit_query_f64": [_P, _P, _I, _I, _I, _I, _U64, _P, _PP],
    "culsh_pslsh_fit_f32": [_P, _P, _I, _I, _I, _I, _I, _U64, _P, _P, _PP],
    "culsh_pslsh_fit_f64": [_P, _P, _I, _I, _I, _I, _I, _U64, _P, _P, _PP],
    "culsh_pslsh_query_f32": [_P, _P, _I, _P, _I, _PP],
    "culsh_pslsh_query_f64": [_P, _P, _I, _P, _I, _PP],
    "culsh_pslsh_fit_query_f32": [_P, _P, _I, _I, _I, _I, _I, _U64, _P, _P, _PP],
    "culsh_pslsh_fit_query_f64": [_P, _P, _I, _I, _I, _I, _I, _U64, _P, _P, _PP],
    "culsh_minhash_fit": [_P, _P, _P, _I, _I, _I, _I, _U64, _P, _P, _PP],
    "culsh_minhash_query": [_P, _P, _P, _I, _P, _PP],
    "culsh_minhash_fit_query": [_P, _P, _P, _I, _I, _I, _I, _U64, _P, _P, _PP],
    "culsh_rplsh_hash_f32": [_P, _P, _P, _I, _I, _I, _I, _P],
    "culsh_rplsh_hash_f64": [_P, _P, _P, _I, _I, _I, _I, _P],
    "culsh_pslsh_hash_f32": [_P, _P, _P, _P, _I, _I, _I, _I, _P],
    "culsh_pslsh_hash_f64": [_P, _P, _P, _P, _I, _I, _I, _I, _P],
    "culsh_minhash_compute": [_P, _P, _P, _P, _P, _I, _I, _I, _P],
    "culsh_core_fit_index": [_P, _P, _I, _I, _I, _I, _P, _PP],
    "culsh_core_query_index": [_P, _P, _I, _I, _P, _PP],
    "culsh_core_find_matching_buckets": [_P, _P, _I, _I, _P, _P],
    "culsh_core_find_matching_buckets_static": [_P, _P, _I, _I, _P, _P],
    "culsh_core_query_from_matched_buckets": [_P, _P, _I, _P, _PP],
    "culsh_core_fit_query": [_P, _P, _I, _I, _I, _I, _PP],
    "culsh_index_get_meta": [_P, C.POINTER(IndexMeta)],
    "culsh_debug_arena_state": [_P, C.POINTER(C.c_uint64)],
    "culsh_index_key_form": [_P, C.POINTER(C.c_int32), C.POINTER(C.c_int32)],
    "culsh_index_array_info": [_P, _I, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)],
    "culsh_index_copy_array": [_P, _P, _I, _P, _U64, _I],
    "culsh_index_load": [_P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _U64, _PP],
    "culsh_candidates_get_meta": [_P, C.POINTER(CandidatesMeta)],
    "culsh_candidates_copy_array": [_P, _P, _I, _P, _U64, _I],
    "culsh_candidates_merge": [_P, _PP, _P],
}
# name -> (restype, argtypes)
_SPECIAL = {
    "culsh_last_error": (C.c_char_p, []),
    "culsh_version": (C.c_char_p, []),
    "culsh_debug_allocation_calls": (C.c_uint64, []),
    "culsh_ctx_destroy": (None, [_P]),
    "culsh_memory_trim": (None, []),
    "culsh_ctx_stream": (_P, [_P]),
    "culsh_profile_count": (C.c_int, [_P]),
    "culsh_index_free": (None, [_P]),
    "culsh_candidates_free": (None, [_P]),
    "culsh_candidates_device_ptr": (_P, [_P, _I]),
}
ALL_SYMBOLS = sorted(list(PROTOTYPES) + list(_SPECIAL))

_lib = None


def load() -> C.CDLL:
    """Loads libculsh_amd.so once and attaches the prototypes. Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(hipcc, --offload-arch=gfx950). There is no CPU fallback.")
    # A process can hold one HIP runtime.  PyTorch-ROCm ships its own libamdhip64 (same
    # soname as the system one): importing torch first makes the loader resolve this
    # library's dependency to that already-loaded runtime instead of opening a second one,
    # which would leave whichever runtime initialises last without any visible GPU.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = argtypes
    for name, (restype, argtypes) in _SPECIAL.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error() -> str:
    msg = load().culsh_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(status: int) -> None:
    """Maps a culsh_status to the exception the reference binding raises for it:
    RuntimeError for device/runtime failures and dtype mismatches
    (python/csrc/common/cuda_utils.cuh:11-25, bindings.cu:58-60), MemoryError for
    allocation failures (the reference exits the process there, core/utils.cuh:10-18)."""
    if status == OK:
        return
    msg = last_error()
    if status == ERR_NOMEM:
        raise MemoryError(msg)
    raise RuntimeError(msg)
