"""ctypes binding of libtplr_hip.so (C ABI in include/tplr_hip.h).

The library is the product: there is no fallback.  If it is missing or a symbol cannot
be resolved, loading raises and every codec call fails.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TPLR_HIP_LIB selects another build of the same library (e.g. an instrumented one)
LIB_PATH = os.environ.get("TPLR_HIP_LIB") or os.path.join(_HERE, "libtplr_hip.so")

TPLR_E_BADARG, TPLR_E_ODD, TPLR_E_SHAPE, TPLR_E_TOOMANY, TPLR_E_WORKSPACE = -1, -2, -3, -4, -5
TPLR_MAX_PEERS = 128
TPLR_MAX_ROW = 4096
TPLR_MAX_K = 128
REDUCE_MEAN, REDUCE_SUM = 0, 1

_vp, _i64, _i32 = C.c_void_p, C.c_int64, C.c_int

# name -> (restype, argtypes); must list every function declared in include/tplr_hip.h
SIGNATURES = {
    "tplr_version": (_i32, []),
    "tplr_status_string": (C.c_char_p, [_i32]),
    "tplr_pack12": (_i32, [_vp, _i64, _vp, _vp, _vp]),
    "tplr_unpack12": (_i32, [_vp, _i64, _vp, _vp]),
    "tplr_pack12_host": (_i32, [_vp, _i64, _vp, _vp]),
    "tplr_unpack12_host": (_i32, [_vp, _i64, _vp]),
    "tplr_gather_host": (_i32, [_vp, _vp, _i64, _vp, _i32]),
    "tplr_dct2d_fwd": (_i32, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "tplr_dct2d_inv": (_i32, [_vp, _i64, _i64, _vp, _i64, _vp]),
    "tplr_dct1d": (_i32, [_vp, _i64, _i32, _vp, _vp]),
    "tplr_dct2d_dense": (_i32, [_vp, _i64, _i64, _i32, _i32, _vp, _vp, _i32, _i32, _vp, _vp]),
    "tplr_topk_pack": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp]),
    "tplr_encode_topk_pack": (_i32, [_vp, _i64, _i64, _i64, _i32, _i32, _vp, _vp, _vp]),
    "tplr_encode_topk_pack_batch": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp]),
    "tplr_encode_rows_batch": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp]),
    "tplr_decode_aggregate_batch": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp]),
    "tplr_decode_aggregate_stats_batch": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _vp]),
    "tplr_code_sumsq": (_i32, [_vp, _i32, _i32, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp]),
    "tplr_decode_aggregate_codes_batch": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _i32, _vp, _vp]),
    "tplr_decode_aggregate_codes_stats_batch": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _i32, _vp, _vp, _vp]),
    "tplr_segment_sumsq": (_i32, [_vp, _i32, _i32, _vp, _i32, _i32, _vp, _vp]),
    "tplr_clip_scales_batch": (_i32, [_vp, _i32, _i32, _i32, _vp, _vp, _vp]),
    "tplr_row_sumsq": (_i32, [_vp, _i32, _i32, _i64, _vp, _vp]),
    "tplr_clip_scales_rows": (_i32, [_vp, _i32, _vp, _i32, _i32, _vp, _vp, _vp, _vp]),
    "tplr_decode_aggregate": (_i32, [_vp, _vp, _vp, _i32, _i32, _i64, _i64, _i32, _i32, _i32, _vp, _i64, _vp, _vp]),
    "tplr_scatter_rows": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp, _vp, _vp]),
    "tplr_flat_update": (_i32, [_vp, _vp, _i64, C.c_float, _i32, _vp]),
    "tplr_aggregate_rows": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _i64, _i32, _vp, _vp, _vp]),
    "tplr_decode_rows_batch": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _i32, _i32, _vp, _vp]),
    "tplr_peer_sumsq": (_i32, [_vp, _i32, _i64, _i32, _vp, _vp]),
    "tplr_clip_scales": (_i32, [_vp, _i32, _i32, _vp, _vp, _vp]),
    "tplr_calib_encode": (_i32, [_vp, _i32, _i64, _vp]),
    "tplr_calib_copy": (_i32, [_vp, _vp, _i64, _vp]),
    "tplr_calib_fill": (_i32, [_vp, _i64, _i32, _vp]),
    "tplr_debug_fill_lds": (_i32, [_i32, _vp]),
    "tplr_calib_aggregate": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp, _i32, _i64, _vp]),
    "tplr_ef_encode_topk_pack_batch": (_i32, [_vp, _vp, _i32, _i64, C.c_float, _i32, _i32, _vp, _vp, _vp]),
    "tplr_ef_subtract_batch": (_i32, [_vp, _vp, _i32, _vp, _i32, _i64, _i32, _vp]),
    "tplr_apply_decoded_batch": (_i32, [_vp, _vp, _vp, _i32, _vp, _i32, _i64, _i32, _vp, _vp]),
    "tplr_outer_step_codes_batch": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _vp, _vp, _vp, _vp]),
    "tplr_outer_step_batch": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _vp, _vp, _vp, _vp]),
    "tplr_ef_step_batch": (_i32, [_vp, _vp, _i32, _i64, C.c_float, _i32, _vp, _vp, _vp]),
    "tplr_ef_subtract_own_batch": (_i32, [_vp, _vp, _vp, _i32, _vp, _i32, _i64, _vp]),
    "tplr_dequantize_batch": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _vp, _vp]),
    "tplr_dequantize_peers": (_i32, [_vp, _i32, _i64, _vp, _vp, _i32, _vp, _vp]),
    "tplr_quantize_batch": (_i32, [_vp, _i32, _vp, _i32, _i32, C.c_float, _i32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "tplr_tensor_rnorm": (_i32, [_vp, _vp, _i32, C.c_float, _vp, _vp]),
    "tplr_scale_batch": (_i32, [_vp, _i32, _i64, _vp, _vp]),
    "tplr_aggregate_sumsq_batch": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _vp, _vp]),
    "tplr_tensor_rnorm_scales": (_i32, [_vp, _vp, _i32, _i32, C.c_float, C.c_float, _vp, _vp, _vp]),
    "tplr_static_work_bytes": (_i64, []),
    "tplr_quantize_batch_static": (_i32, [_vp, _i32, _vp, _i32, _i32, C.c_float, _i32, _vp, _vp, _vp, _vp, _vp]),
    "tplr_index_stats_batch": (_i32, [_vp, _i32, _i32, _vp, _i32, _i64, _vp, _vp, _vp, _vp]),
}

_lib = None


class TplrHipError(RuntimeError):
    """A libtplr_hip call returned a non-zero status."""


def load():
    """Load libtplr_hip.so once and bind every entry point."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc --offload-arch=gfx950).  templar_amd has no other code path."
            )
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().tplr_status_string(status).decode()
        raise TplrHipError(f"{what}: {msg} (status {status})")
