"""numpy face of liborc.so (oracle/tplr_oracle.c).  Test infrastructure only.

Each function names the reference routine it restates (src/tplr/compress.py, tplr 2.1.28).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liborc.so")


def build(force: bool = False) -> str:
    """Compile tplr_oracle.c with gcc (seconds).  Building the checker is not using it."""
    src = os.path.join(_HERE, "tplr_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(
            ["gcc", "-O2", "-fPIC", "-std=c11", "-ffp-contract=off", "-shared", src, "-o", _LIB_PATH, "-lm"]
        )
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        i64, i32, p = C.c_int64, C.c_int, C.c_void_p
        L.orc_pack12.argtypes = [p, i64, p, p]
        L.orc_unpack12.argtypes = [p, i64, p]
        L.orc_divisors.argtypes = [i64, p, i32]
        L.orc_smaller_split.argtypes = [i64, i64]
        L.orc_smaller_split.restype = i64
        L.orc_dct_basis.argtypes = [i32, p]
        L.orc_encode2d.argtypes = [p, i64, i64, i32, i32, i32, p]
        L.orc_decode2d.argtypes = [p, i64, i64, i32, i32, i32, p]
        L.orc_dct1d.argtypes = [p, i64, i32, i32, p]
        L.orc_clamp_topk.argtypes = [i64, i64]
        L.orc_topk_rows.argtypes = [p, i64, i64, i32, p, p]
        L.orc_scatter_rows.argtypes = [p, p, i64, i64, i64, i32, p]
        L.orc_clip_scales.argtypes = [p, i32, p]
        L.orc_clip_scales.restype = C.c_float
        L.orc_norm2.argtypes = [p, i64]
        L.orc_norm2.restype = C.c_float
        L.orc_batch_scatter.argtypes = [p, p, p, i32, i64, i32, i64, i32, i32, p]
        L.orc_quantize.argtypes = [p, i64, i32, C.c_float, p, p, p]
        L.orc_quantize.restype = C.c_float
        L.orc_dequantize.argtypes = [p, i64, p, C.c_float, p]
        _lib = L
    return _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# ---------------------------------------------------------------- pack / unpack (:51-142)
def pack12(indices) -> np.ndarray:
    idx = _c(indices, np.int64).reshape(-1)
    out = np.zeros(idx.size // 2 * 3, dtype=np.uint8)
    bad = C.c_int64(0)
    rc = lib().orc_pack12(_ptr(idx), idx.size, _ptr(out), C.byref(bad))
    if rc == 1:
        raise ValueError(f"Index {bad.value} exceeds 12-bit limit (4095)")
    if rc == 2:
        raise ValueError(f"Number of indices must be even, got {idx.size}")
    return out


def unpack12(packed, values_shape) -> np.ndarray:
    n = int(np.prod(values_shape, dtype=np.int64)) if len(values_shape) else 1
    if n == 0:
        return np.zeros(values_shape, dtype=np.int64)
    if n % 2:
        raise ValueError(f"Number of indices must be even, got {n}")
    pk = _c(packed, np.uint8).reshape(-1)
    if pk.size < n // 2 * 3:
        raise ValueError("packed buffer too short")
    out = np.zeros(n, dtype=np.int64)
    lib().orc_unpack12(_ptr(pk), n, _ptr(out))
    return out.reshape(values_shape)


# ---------------------------------------------------------------- divisor rule (:791-872)
def divisors(n: int) -> list[int]:
    buf = np.zeros(4096, dtype=np.int64)
    cnt = lib().orc_divisors(n, _ptr(buf), 4096)
    return buf[:cnt].tolist()


def smaller_split(n: int, close_to: int) -> int:
    return int(lib().orc_smaller_split(n, close_to))


# ---------------------------------------------------------------- transforms (:186-292, :710-788)
def dct_basis(n: int) -> np.ndarray:
    f = np.zeros((n, n), dtype=np.float64)
    lib().orc_dct_basis(n, _ptr(f))
    return f


def encode2d(x, h: int = 64, w: int = 64, use_dct: bool = True) -> np.ndarray:
    x = _c(x, np.float32)
    R, Cc = x.shape
    out = np.zeros((R // h, Cc // w, h, w), dtype=np.float32)
    lib().orc_encode2d(_ptr(x), R, Cc, h, w, int(use_dct), _ptr(out))
    return out


def decode2d(coef, use_dct: bool = True) -> np.ndarray:
    coef = _c(coef, np.float32)
    Y, X, h, w = coef.shape
    out = np.zeros((Y * h, X * w), dtype=np.float32)
    lib().orc_decode2d(_ptr(coef), Y * h, X * w, h, w, int(use_dct), _ptr(out))
    return out


def dct1d(rows, inverse: bool = False) -> np.ndarray:
    rows = _c(rows, np.float32)
    n_vec, w = rows.shape
    out = np.zeros_like(rows)
    lib().orc_dct1d(_ptr(rows), n_vec, w, int(inverse), _ptr(out))
    return out


# ---------------------------------------------------------------- top-k (:352-412)
def clamp_topk(last_dim: int, topk: int) -> int:
    return int(lib().orc_clamp_topk(last_dim, topk))


def topk_rows(x, k: int):
    """x (..., n) -> (idx int64 (..., k), val float32 (..., k)) in canonical order."""
    x = _c(x, np.float32)
    n = x.shape[-1]
    rows = x.reshape(-1, n)
    idx = np.zeros((rows.shape[0], k), dtype=np.int64)
    val = np.zeros((rows.shape[0], k), dtype=np.float32)
    lib().orc_topk_rows(_ptr(rows), rows.shape[0], n, k, _ptr(idx), _ptr(val))
    return idx.reshape(x.shape[:-1] + (k,)), val.reshape(x.shape[:-1] + (k,))


def compress(x, topk: int):
    """TopKCompressor.compress without quantisation (:385-423): x is the encoded tensor
    (Y, X, h, w) or (rows, n).  Returns (packed idx uint8, val, xshape, totalk)."""
    x = _c(x, np.float32)
    xshape = x.shape
    flat = x.reshape(x.shape[0], x.shape[1], -1) if x.ndim > 2 else x
    totalk = flat.shape[-1]
    k = clamp_topk(totalk, topk)
    idx, val = topk_rows(flat, k)
    return pack12(idx), val, xshape, totalk


# ---------------------------------------------------------------- scatter side (:425-580)
def scatter_rows(idx, val, n: int, mean: bool = True) -> np.ndarray:
    idx = _c(idx, np.int64)
    val = _c(val, np.float32)
    kk = idx.shape[-1]
    rows = idx.reshape(-1, kk)
    out = np.zeros((rows.shape[0], n), dtype=np.float32)
    rc = lib().orc_scatter_rows(_ptr(rows), _ptr(val.reshape(-1, kk)), rows.shape[0], kk, n, int(mean), _ptr(out))
    if rc:
        raise IndexError("index out of range in scatter")
    return out.reshape(idx.shape[:-1] + (n,))


def decompress(idx_packed, val, xshape, totalk: int) -> np.ndarray:
    """TopKCompressor.decompress (:425-481) for packed indices and fp32 values."""
    val = _c(val, np.float32)
    idx = unpack12(idx_packed, val.shape)
    dense = scatter_rows(idx, val, totalk, mean=True)
    return dense.reshape(xshape)


def norm2(v) -> float:
    v = _c(v, np.float32).reshape(-1)
    return float(lib().orc_norm2(_ptr(v), v.size))


def clip_scales(norms):
    norms = _c(norms, np.float32)
    scale = np.zeros_like(norms)
    med = lib().orc_clip_scales(_ptr(norms), norms.size, _ptr(scale))
    return float(med), scale


def batch_decompress(idx_packed_list, val_list, xshape, totalk: int, *, block_norms=None, normalise=False,
                     clip_norm=True, mean=True) -> np.ndarray:
    """TopKCompressor.batch_decompress (:483-580), fp32 values, packed indices."""
    vals = [_c(v, np.float32) for v in val_list]
    P = len(vals)
    k = vals[0].shape[-1]
    idxs = [unpack12(i, v.shape).reshape(-1, k) for i, v in zip(idx_packed_list, vals)]
    scale = None
    if clip_norm and not normalise:
        norms = np.asarray(block_norms, dtype=np.float32) if block_norms is not None else np.array(
            [norm2(v) for v in vals], dtype=np.float32)
        _, scale = clip_scales(norms)
    flat_vals = [v.reshape(-1, k) for v in vals]
    n_rows = flat_vals[0].shape[0]
    out = np.zeros((n_rows, totalk), dtype=np.float32)
    ip = (C.c_void_p * P)(*[i.ctypes.data for i in idxs])
    vp = (C.c_void_p * P)(*[v.ctypes.data for v in flat_vals])
    rc = lib().orc_batch_scatter(ip, vp, _ptr(scale) if scale is not None else None, P, n_rows, k, totalk,
                                 int(normalise), int(mean), _ptr(out))
    if rc:
        raise IndexError("index out of range in scatter")
    return out.reshape(xshape)


def aggregate_mean_normalised(idx_packed_list, val_list, xshape, totalk: int, *, use_dct: bool = True,
                              eps: float = 1e-8) -> np.ndarray:
    """The benchmark's wording of the aggregation workload (no counterpart inside tplr.compress): the peers'
    payloads scatter-summed, inverse transform, divided by the number of peers, divided by the L2 norm
    (+ eps) of the result.  Built from batch_decompress in sum mode and decode2d."""
    P = len(val_list)
    dense = batch_decompress(idx_packed_list, val_list, xshape, totalk, clip_norm=False, mean=False)
    x = decode2d(dense, use_dct=use_dct).astype(np.float64) / P
    return (x / (np.sqrt((x * x).sum()) + eps)).astype(np.float32)


# ---------------------------------------------------------------- quantiser (:582-644)
def quantize(val, n_bins: int = 256, range_in_sigmas: float = 6.0):
    v = _c(val, np.float32)
    q = np.zeros(v.size, dtype=np.uint8)
    lookup = np.zeros(n_bins, dtype=np.float32)
    shift = C.c_float(0)
    scale = lib().orc_quantize(_ptr(v.reshape(-1)), v.size, n_bins, range_in_sigmas, _ptr(q), C.byref(shift),
                               _ptr(lookup))
    return q.reshape(v.shape), (float(shift.value), float(scale), n_bins // 2, lookup)


def dequantize(q, qparams) -> np.ndarray:
    shift, _, _, lookup = qparams
    q = _c(q, np.uint8)
    out = np.zeros(q.shape, dtype=np.float32)
    lk = _c(lookup, np.float32)
    lib().orc_dequantize(_ptr(q.reshape(-1)), q.size, _ptr(lk), shift, _ptr(out))
    return out


# ---------------------------------------------------------------- miner step (src/tplr/neurons.py:147-171)
def error_feedback_step(ef, grad, decay: float, topk: int, *, use_dct: bool = True, quant_bins: int = 0,
                        quant_range: float = 6.0, coef_override=None, null_round: bool = False):
    """One parameter's momentum / compress / error-feedback update, line by line:
    ef.mul_(decay); ef.add_(grad) (:151-152); encode (:155); compress (:157-159); decompress (:164-166);
    decode (:169); ef.sub_(decoded) (:171).  `quant_bins` > 0 runs the values through the statistical
    quantiser as compress/decompress do when the compressor quantises.  `coef_override`, if given,
    replaces the encoded tensor that is compressed (to compare selections on another
    implementation's coefficients).  `null_round` zeroes the error feedback instead of updating it (:148-149).
    Returns (ef_accumulated, packed idx, val, ef_new)."""
    ef = _c(ef, np.float32).copy()
    if null_round:
        ef[...] = 0.0                     # :149
    else:
        ef *= np.float32(decay)           # one rounding (:151)
        ef += _c(grad, np.float32)        # a second one (:152)
    enc = encode2d(ef, use_dct=use_dct) if coef_override is None else _c(coef_override, np.float32)
    idx12, val, xshape, totalk = compress(enc, topk)
    sent = val
    if quant_bins:
        q, qp = quantize(val, quant_bins, quant_range)
        sent = dequantize(q, qp)
    recon = decode2d(decompress(idx12, sent, xshape, totalk), use_dct=use_dct)
    return ef, idx12, val, ef - recon


# ---------------------------------------------------------------- outer step (src/tplr/neurons.py:341-447)
def outer_step(param, idx_packed_list, val_list, xshape, totalk: int, lr: float, *, use_dct: bool = True):
    """One parameter's pass through outer_step with the plain SGD the reference builds for it
    (neurons/trainer.py:128-130: SGD(lr), no momentum, no weight decay): block norms of the peers' values (:346),
    batch_decompress with the median clip (:355-365), decode (:367), the gradient's L2 norm and mean for the
    fingerprint (:380-385), and - unless an element of the gradient is not finite, in which case the parameter is
    left alone (:438-442) - p <- p - lr * grad (optimizer.step(), :446).
    Returns (new_param, grad_norm, grad_mean, applied)."""
    p = _c(param, np.float32)
    vals = [_c(v, np.float32) for v in val_list]
    norms = np.array([norm2(v) for v in vals], dtype=np.float32)                 # :346
    grad = decode2d(batch_decompress(idx_packed_list, vals, xshape, totalk, block_norms=norms), use_dct=use_dct)
    with np.errstate(all="ignore"):
        g_norm = float(np.sqrt((grad.astype(np.float64) ** 2).sum()))            # :381
        g_mean = float(grad.astype(np.float64).mean())                           # :385
    if not np.isfinite(grad).all():                                              # :438
        return p.copy(), g_norm, g_mean, False
    return (p - np.float32(lr) * grad).astype(np.float32), g_norm, g_mean, True  # :446


# ---------------------------------------------------------------- index checks
def index_overlap(idx_list):
    """Pairwise overlap of peers' index rows, as check_uid_index_overlap computes it per
    parameter (src/tplr/neurons.py:1366-1378): idx_list[p] is peer p's (C, k) int64 indices.
    Returns (inter, frac): inter[i, j] (i < j) = sum over chunks of `(a == b).any(-1).sum(-1)`,
    frac[i, j] = mean over chunks of inter_c / k (its `mean_frac`)."""
    P = len(idx_list)
    rows = [_c(i, np.int64).reshape(-1, np.shape(i)[-1]) for i in idx_list]
    Cn, k = rows[0].shape
    inter = np.zeros((P, P), dtype=np.int64)
    frac = np.zeros((P, P), dtype=np.float64)
    for i in range(P):
        for j in range(i + 1, P):
            a = rows[i][:, :, None]          # (C, k, 1)   :1373
            b = rows[j][:, None, :]          # (C, 1, k)   :1374
            per_chunk = (a == b).any(-1).sum(-1)  # :1375
            inter[i, j] = per_chunk.sum()
            frac[i, j] = (per_chunk.astype(np.float32) / k).mean()  # :1376
    return inter, frac


def index_bounds(idx, totalk: int):
    """The bounds check of Comms.check_compressed_indices (src/tplr/comms.py:2573-2581):
    None if every index is in [0, totalk), else the first offending index."""
    t = _c(idx, np.int64).reshape(-1)
    if t.size == 0:
        raise ValueError("empty index list")
    bad = t[(t < 0) | (t >= totalk)]
    return None if bad.size == 0 else int(bad[0])

