"""ctypes binding of libdistill_hip.so (the C ABI declared in include/distill_hip.h).

The library is the only compute path: if it is missing this module raises on
first use -- there is no PyTorch or CPU fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdistill_hip.so")

# dtype / kind codes of include/distill_hip.h
DL_F32, DL_BF16, DL_F16 = 0, 1, 2
DL_I32, DL_I64 = 0, 1
DL_FKL, DL_RKL, DL_JSD = 0, 1, 2
DL_MAX_TOPK = 2048
DL_MAX_TEACHERS = 8
DL_MAX_HOST_CONVOS = 64
DL_TOPK_UNIQUE_IDS = 1
DL_TOPK_NO_WAIT = 2
DL_TOPK_FINE_PARTS = 4
DL_TOPK_PARTS_SHIFT = 8
DL_STATIC_SCRATCH_BYTES = 4 << 20

_P = c_void_p
_SIGNATURES = {
    "dl_abi_version": (c_int, []),
    "dl_status_string": (c_char_p, [c_int]),
    "dl_div_topk": (c_int, [c_int, _P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int, _P, c_int, c_int, c_int64, _P,
                            c_float, c_float, c_float, _P, _P, c_int64, _P, c_int64, c_int, _P]),
    "dl_div_topk_workspace_bytes": (c_int64, [c_int, c_int, c_int64, c_int64]),
    "dl_div_topk_static": (c_int, [c_int, _P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int, _P, c_int, c_int, c_int64, _P,
                                   c_float, c_float, c_float, _P, _P, c_int64, c_int, _P]),
    "dl_div_dense": (c_int, [c_int, _P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int, c_int64, c_int64,
                             c_float, c_float, c_float, _P, _P, c_int64, _P]),
    "dl_div_dense_ws": (c_int, [c_int, _P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int, c_int64, c_int64,
                                c_float, c_float, c_float, _P, _P, c_int64, _P, c_int64, c_int, _P]),
    "dl_div_dense_workspace_bytes": (c_int64, [c_int, c_int, c_int, c_int64, c_int64]),
    "dl_rowstats_topk": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int, c_int, c_int64, c_float,
                                 _P, _P, _P]),
    "dl_rowcoef_grad_topk": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int, c_int, c_int64, c_float,
                                     _P, _P, _P, _P, c_int64, _P]),
    "dl_fkl_multi_teacher": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int, _P, _P, c_int, c_int, c_int, c_int64,
                                     _P, _P, c_int64, c_float, c_float, _P, _P, c_int64, _P, c_int64, c_int, _P]),
    "dl_fkl_multi_teacher_workspace_bytes": (c_int64, [c_int, c_int64, c_int64, c_int, c_int, c_int64, c_int]),
    "dl_merge_remap_topk": (c_int, [c_int, _P, _P, c_int, c_int, c_int, _P, c_int64, _P, c_int64, c_int64,
                                    _P, _P, _P, _P]),
    "dl_merge_topk_pair": (c_int, [_P, _P, c_int64, _P, _P, c_int64, c_int, c_int, c_int, c_int64, _P, _P, _P]),
    "dl_trie_longest_prefix_map": (c_int, [_P, _P, c_int64, _P, _P, c_int64, _P, _P]),
    "dl_csr_from_map": (c_int, [_P, c_int64, c_int64, _P, _P, _P]),
    "dl_marginal_plan_build": (c_int, [_P, c_int64, c_int64, _P, _P, _P, c_int64, _P, _P, c_int64, _P, _P]),
    "dl_marginalise_map": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int64, _P, _P, c_int, _P, c_int, c_int, _P,
                                   c_int64, c_int, _P]),
    "dl_marginalise_csr": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int64, _P, c_int64, c_int, _P]),
    "dl_gather_columns": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int64, _P, c_int64, _P]),
    "dl_expand_columns": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int64, _P, c_int64, _P]),
    "dl_rkl_marginalised": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int, c_int64, c_int64, c_int64, _P,
                                    _P, _P, c_int, _P, c_int, c_int, c_float, c_float, c_float, _P, _P, c_int64, _P]),
    "dl_rkl_marginalised_compact": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, _P, c_int64, _P, _P, c_int, c_int64,
                                            c_int64, c_int64, _P, _P, _P, c_int, _P, c_int, c_int, c_float, c_float, c_float,
                                            _P, _P, c_int64, _P]),
    "dl_composite_forward": (c_int, [_P, _P, _P, c_int, c_float, _P, c_int, c_int, _P, _P, c_int, _P, _P, _P, c_int, c_int,
                                     c_int64, c_float, _P, _P, _P, _P]),
    "dl_composite_backward": (c_int, [_P, _P, _P, c_int, c_float, _P, c_int, c_int, _P, c_int, c_int, c_int64, _P, _P, _P, _P,
                                      _P, _P]),
    "dl_composite_forward_fused": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int64, c_float, _P, c_int, c_float, _P, c_int, c_int,
                                           _P, _P, c_int, _P, _P, _P, c_int, c_int, c_float, _P, _P, _P, _P, _P, _P]),
    "dl_composite_backward_fused": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int64, c_float, _P, c_int, c_float, _P, c_int, c_int,
                                            _P, c_int, c_int, _P, _P, _P, _P, _P, _P, c_int64, _P]),
    "dl_teacher_topk": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int64, c_int, _P, c_int, _P, c_int, _P, c_int64, _P]),
    "dl_teacher_topk_workspace_bytes": (c_int64, [c_int, c_int64, c_int64, c_int]),
    "dl_reduce_sum": (c_int, [_P, c_int64, c_float, _P, _P]),
    "dl_copy16": (c_int, [_P, _P, c_int64, _P]),
    "dl_copy_rows": (c_int, [_P, _P, c_int64, c_int64, c_int, c_int, c_int, _P]),
}

_lib = None


class DistillLibraryError(RuntimeError):
    pass


def exported_symbols() -> list[str]:
    return sorted(_SIGNATURES)


def load() -> ctypes.CDLL:
    """Load the shared library once and attach the argument types."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise DistillLibraryError(
            f"{LIB_PATH} is missing: build it with `python llm-distillery_amd/build.py` "
            "(hipcc, gfx950). There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    """Translate a dl_status into the Python error the caller sees."""
    if status != 0:
        msg = load().dl_status_string(status).decode()
        raise RuntimeError(f"{what}: {msg} (dl_status {status})")
