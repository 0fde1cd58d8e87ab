"""Host-side mirror of templar's gradient codec API (reference: src/tplr/compress.py,
tplr 2.1.28) on top of libtplr_hip.so.

Same names, arguments, return tuples and error messages as the reference, so that
`neurons/miner.py`, `neurons/validator.py` and `src/tplr/neurons.py` can use this module in
place of `tplr.compress`:

    pack_12bit_indices / unpack_12bit_indices          (reference :51-142)
    ChunkingTransformer.encode / decode / einsum_2d(_t) (reference :145-292)
    TopKCompressor.compress / decompress / batch_decompress / quantiser (reference :295-696)
    _dct, _idct, _get_smaller_split, _get_divisors, _get_prime_divisors (reference :700-872)
    TransformDCT = ChunkingTransformer, CompressDCT = TopKCompressor     (DeMo-era names)

All tensor arithmetic of the codec runs in the HIP library on the tensor's device and on
torch's current stream; nothing here synchronises except where the reference does
(`pack_12bit_indices` reads back the range-check flag, as the reference's `.item()` does).
Only the basis construction at start-up and the small statistical quantiser use torch ops.
The two fused entry points `encode_compress` and `batch_decompress_decode` do what the
callers' back-to-back `encode`+`compress` and `batch_decompress`+`decode` do, in one kernel
each and without materialising the dense coefficient tensor.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import math
import os
from typing import Sequence, TypeAlias

import torch

from . import _lib

try:  # DTensor inputs are unwrapped exactly where the reference does (:398-399)
    from torch.distributed.tensor import DTensor as _DT
except Exception:  # pragma: no cover - torch without distributed
    _DT = ()

ShapeT: TypeAlias = tuple[int, ...]
Shape4D = tuple[int, int, int, int]
TotK: TypeAlias = int
IdxT: TypeAlias = torch.Tensor
ValT: TypeAlias = torch.Tensor
QuantParamsT: TypeAlias = tuple[torch.Tensor, float, int, torch.Tensor, torch.dtype]

_CH = 64  # chunk edge served by the factorised transform kernels


# ----------------------------------------------------------------------------------------
# plumbing
# ----------------------------------------------------------------------------------------
def _ptr(t: torch.Tensor | None):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(dev: torch.device):
    return C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _on(dev: torch.device):
    """Context in which `dev` is the current device (kernel launches go to the current one);
    free when it already is."""
    if torch.cuda.current_device() == dev.index:
        return contextlib.nullcontext()
    return torch.cuda.device(dev)


def _need_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"templar_amd.{what}: tensor is on '{t.device}'; the codec kernels run on a HIP device only "
            "(there is no CPU code path)"
        )


def _val_on(v: torch.Tensor, dev: torch.device) -> torch.Tensor:
    """Values as the kernels read them: fp32, contiguous, on `dev` (no work when they already are)."""
    if v.device == dev and v.dtype == torch.float32 and v.is_contiguous():
        return v
    return _f32c(v.to(dev))


def _idx_on(i: torch.Tensor, dev: torch.device) -> torch.Tensor:
    """A packed index stream as the kernels read it: flat, contiguous, on `dev`."""
    if i.device == dev and i.dim() == 1 and i.is_contiguous():
        return i
    return i.to(dev).reshape(-1).contiguous()


def _f32c(t: torch.Tensor) -> torch.Tensor:
    """fp32, contiguous (the kernels' only element type)."""
    if t.dtype != torch.float32:
        t = t.float()
    return t.contiguous()


# ----------------------------------------------------------------------------------------
# 12-bit index packing (reference :51-142)
# ----------------------------------------------------------------------------------------
def pack_12bit_indices(indices: torch.Tensor) -> torch.Tensor:
    """Pack an even number of indices < 4096 into 3 bytes per pair (reference :51-99)."""
    lib = _lib.load()
    n = indices.numel()
    flat = indices.reshape(-1)
    if flat.dtype != torch.int64:
        flat = flat.to(torch.int64)
    flat = flat.contiguous()
    if flat.is_cuda:
        with _on(flat.device):
            # the reference finds the maximum first (and raises on it) before the parity check
            err = torch.zeros(1, dtype=torch.int32, device=flat.device)
            out = torch.empty((n // 2) * 3, dtype=torch.uint8, device=flat.device)
            if n >= 2:
                st = lib.tplr_pack12(_ptr(flat), n - (n % 2), _ptr(out), _ptr(err), _stream(flat.device))
                _lib.check(st, "tplr_pack12")
            worst = int(err.item())  # the reference synchronises here as well (.item(), :64)
            if n % 2:
                worst = max(worst, int(flat[-1].item()))
    else:
        out = torch.empty((n // 2) * 3, dtype=torch.uint8)
        bad = C.c_int64(0)
        if n >= 2:
            st = lib.tplr_pack12_host(_ptr(flat), n - (n % 2), _ptr(out), C.byref(bad))
            _lib.check(st, "tplr_pack12_host")
        worst = int(bad.value)
        if n % 2:
            worst = max(worst, int(flat[-1]))
    if worst >= 4096:
        raise ValueError(f"Index {worst} exceeds 12-bit limit (4095)")
    if n % 2 != 0:
        raise ValueError(f"Number of indices must be even, got {n}")
    return out


def unpack_12bit_indices(packed: torch.Tensor, values_shape: ShapeT) -> torch.Tensor:
    """Inverse of pack_12bit_indices; int64 tensor of `values_shape` (reference :102-142)."""
    n = int(math.prod(tuple(values_shape)))
    if n == 0:
        return torch.zeros(tuple(values_shape), dtype=torch.int64, device=packed.device)
    if n % 2 != 0:
        raise ValueError(f"Number of indices must be even, got {n}")
    if packed.dtype != torch.uint8:
        packed = packed.to(torch.uint8)
    packed = packed.reshape(-1).contiguous()
    if packed.numel() * 2 != n * 3:
        # the reference fails here with torch's shape-mismatch RuntimeError
        raise RuntimeError(
            f"shape mismatch: {packed.numel()} packed bytes cannot hold {n} 12-bit indices (need {n // 2 * 3})"
        )
    lib = _lib.load()
    out = torch.empty(n, dtype=torch.int64, device=packed.device)
    if packed.is_cuda:
        with _on(packed.device):
            _lib.check(lib.tplr_unpack12(_ptr(packed), n, _ptr(out), _stream(packed.device)), "tplr_unpack12")
    else:
        _lib.check(lib.tplr_unpack12_host(_ptr(packed), n, _ptr(out)), "tplr_unpack12_host")
    return out.reshape(tuple(values_shape))


# ----------------------------------------------------------------------------------------
# divisor rule and basis (reference :700-872)
# ----------------------------------------------------------------------------------------
def _get_prime_divisors(n: int) -> list[int]:
    """Prime factors of n with multiplicity, ascending (reference :791-817)."""
    out: list[int] = []
    p = 2
    while p * p <= n:
        while n % p == 0:
            out.append(p)
            n //= p
        p += 1 if p == 2 else 2
    if n > 1:
        out.append(n)
    return out


def _get_divisors(n: int) -> list[int]:
    """All divisors of n, ascending; [] for n < 1 (reference :820-850)."""
    if n < 1:
        return []
    small = [d for d in range(1, math.isqrt(n) + 1) if n % d == 0]
    large = [n // d for d in reversed(small) if d * d != n]
    return small + large


def _get_smaller_split(n: int, close_to: int) -> int:
    """Largest divisor of n that is <= close_to; the smallest divisor if none is; n itself
    when every divisor is below close_to (reference :853-872)."""
    divs = _get_divisors(n)
    for pos, d in enumerate(divs):
        if d == close_to:
            return d
        if d > close_to:
            return d if pos == 0 else divs[pos - 1]
    return n


def _cos_table(n: int, dtype, device) -> torch.Tensor:
    i = torch.arange(n, dtype=torch.float64, device=device)
    return torch.cos(math.pi * (2.0 * i[:, None] + 1.0) * i[None, :] / (2.0 * n))  # [sample, freq]


def _dct(x: torch.Tensor, norm: str | None = None) -> torch.Tensor:
    """DCT-II over the last dimension with torch-dct scaling (reference :710-741):
    norm=None gives 2*sum_n x[n] cos(pi(2n+1)k/2N); norm="ortho" the orthonormal transform."""
    n = x.shape[-1]
    m = 2.0 * _cos_table(n, x.dtype, x.device)
    if norm == "ortho":
        m[:, 0] *= 1.0 / (2.0 * math.sqrt(n))
        m[:, 1:] *= 1.0 / (2.0 * math.sqrt(n / 2.0))
    return (x.to(torch.float64) @ m).to(x.dtype)


def _idct(X: torch.Tensor, norm: str | None = None) -> torch.Tensor:
    """Inverse of _dct (a scaled DCT-III), reference :744-788."""
    n = X.shape[-1]
    c = _cos_table(n, X.dtype, X.device)  # [sample, freq]
    if norm == "ortho":
        w = torch.full((n,), math.sqrt(2.0 / n), dtype=torch.float64, device=X.device)
        w[0] = math.sqrt(1.0 / n)
    else:
        w = torch.full((n,), 1.0 / n, dtype=torch.float64, device=X.device)
        w[0] = 1.0 / (2.0 * n)
    return ((X.to(torch.float64) * w) @ c.T).to(X.dtype)


# ----------------------------------------------------------------------------------------
# ChunkingTransformer (reference :145-292)
# ----------------------------------------------------------------------------------------
class ChunkingTransformer:
    """Chunks tensors into (y, x, h, w) blocks and applies the per-chunk 2-D DCT."""

    @torch.no_grad()
    def __init__(self, model, target_chunk, norm="ortho"):
        self.target_chunk = target_chunk
        # the factorised 64-point kernels are the orthonormal transform; any other `norm` goes through the
        # dense contraction with this instance's own bases
        self._fast64 = norm == "ortho"
        self.shape_dict: dict[int, int] = {}
        self.f_dict: dict[int, torch.Tensor] = {}
        self.b_dict: dict[int, torch.Tensor] = {}
        for _, p in model.named_parameters():
            if not p.requires_grad:
                continue
            for s in p.shape:
                sc = _get_smaller_split(s, self.target_chunk)
                self.shape_dict[s] = sc
                if sc not in self.f_dict:
                    eye = torch.eye(sc)
                    self.f_dict[sc] = _dct(eye, norm=norm).to(p.dtype).to(p.device)
                    self.b_dict[sc] = _idct(eye, norm=norm).to(p.dtype).to(p.device)

    # -- dense contraction through the library (any basis, chunk edge <= 64) --------------
    @staticmethod
    def _basis32(table: dict, n: int, dev: torch.device) -> torch.Tensor:
        return table[n].to(device=dev, dtype=torch.float32).contiguous()

    @staticmethod
    def _dense(x: torch.Tensor, R: int, Cc: int, h: int, w: int, bh: torch.Tensor, bw: torch.Tensor,
               in_chunked: bool, out_chunked: bool) -> torch.Tensor:
        _need_device(x, "ChunkingTransformer (DCT)")
        if h > 64 or w > 64:
            raise NotImplementedError(f"chunk {h}x{w}: the HIP transform kernels handle chunk edges up to 64")
        lib = _lib.load()
        xin = _f32c(x)
        out = torch.empty((R // h, Cc // w, h, w) if out_chunked else (R, Cc), dtype=torch.float32, device=x.device)
        if out.numel():
            with _on(x.device):
                st = lib.tplr_dct2d_dense(_ptr(xin), R, Cc, h, w, _ptr(_f32c(bh)), _ptr(_f32c(bw)), int(in_chunked),
                                          int(out_chunked), _ptr(out), _stream(x.device))
            _lib.check(st, "tplr_dct2d_dense")
        return out

    @torch.no_grad()
    def einsum_2d(self, x, b, d=None) -> torch.Tensor:
        """"...ij, jb -> ...ib" (d is None) or "...ijkl, kb, ld -> ...ijbd" (reference :186-203)."""
        if d is None:
            rows = x.reshape(-1, x.shape[-1])
            one = torch.ones(1, 1, dtype=torch.float32, device=x.device)
            out = self._dense(rows, rows.shape[0], rows.shape[1], 1, rows.shape[1], one, b, False, True)
            return out.reshape(x.shape[:-1] + (b.shape[1],)).to(x.dtype)
        lead = x.shape[:-4]
        y4 = x.reshape((-1,) + tuple(x.shape[-3:]))  # fold leading dims and y together
        Y, X, h, w = y4.shape
        out = self._dense(y4, Y * h, X * w, h, w, b, d, True, True)
        return out.reshape(lead + tuple(x.shape[-4:])).to(x.dtype)

    @torch.no_grad()
    def einsum_2d_t(self, x, b, d=None) -> torch.Tensor:
        """"...ij, jb -> ...ib" (d is None) or "...ijbd, bk, dl -> ...ijkl" (reference :205-222)."""
        return self.einsum_2d(x, b, d)

    # -- encode / decode ------------------------------------------------------------------
    @torch.no_grad()
    def encode(self, x: torch.Tensor, *, use_dct: bool = False) -> torch.Tensor:
        """(R, C) -> (R/h, C/w, h, w), or (N,) -> (N/w, w); DCT-II per chunk when use_dct
        (reference :224-257).  Without use_dct the result is a view, as in the reference."""
        if x.dim() > 1:
            n1 = self.shape_dict[x.shape[0]]
            n2 = self.shape_dict[x.shape[1]]
            R, Cc = x.shape
            if not use_dct:
                return x.reshape(R // n1, n1, Cc // n2, n2).permute(0, 2, 1, 3)
            _need_device(x, "ChunkingTransformer.encode(use_dct=True)")
            if n1 == _CH and n2 == _CH and self._fast64:
                lib = _lib.load()
                xin = x if (x.dtype == torch.float32 and x.stride(1) == 1 and x.stride(0) >= Cc) else _f32c(x)
                out = torch.empty((R // _CH, Cc // _CH, _CH, _CH), dtype=torch.float32, device=x.device)
                with _on(x.device):
                    st = lib.tplr_dct2d_fwd(_ptr(xin), R, Cc, xin.stride(0), _ptr(out), _stream(x.device))
                _lib.check(st, "tplr_dct2d_fwd")
                return out if x.dtype == torch.float32 else out.to(x.dtype)
            out = self._dense(x, R, Cc, n1, n2, self._basis32(self.f_dict, n1, x.device),
                              self._basis32(self.f_dict, n2, x.device), False, True)
            return out if x.dtype == torch.float32 else out.to(x.dtype)
        n1 = self.shape_dict[x.shape[0]]
        rows = x.reshape(-1, n1)
        if not use_dct:
            return rows
        _need_device(x, "ChunkingTransformer.encode(use_dct=True)")
        if n1 == _CH and self._fast64:
            lib = _lib.load()
            xin = _f32c(rows)
            out = torch.empty_like(xin)
            with _on(x.device):
                st = lib.tplr_dct1d(_ptr(xin), xin.shape[0], 0, _ptr(out), _stream(x.device))
            _lib.check(st, "tplr_dct1d")
            return out if x.dtype == torch.float32 else out.to(x.dtype)
        return self.einsum_2d(rows, self._basis32(self.f_dict, n1, x.device))

    @torch.no_grad()
    def decode(self, x: torch.Tensor, *, use_dct: bool = False) -> torch.Tensor:
        """(y, x, h, w) -> (y*h, x*w), or (x, w) -> (x*w,); inverse DCT per chunk when use_dct
        (reference :259-292)."""
        if isinstance(x, LazyAggregate):
            if use_dct and not self._fast64:  # (the fused kernel is the orthonormal transform)
                return self.decode(x.dense(), use_dct=True)
            return x.decode(use_dct=use_dct)
        if x.dim() > 2:
            Y, X, h, w = x.shape
            if not use_dct:
                return x.permute(0, 2, 1, 3).reshape(Y * h, X * w)
            _need_device(x, "ChunkingTransformer.decode(use_dct=True)")
            if h == _CH and w == _CH and self._fast64:
                lib = _lib.load()
                xin = _f32c(x)
                out = torch.empty((Y * h, X * w), dtype=torch.float32, device=x.device)
                with _on(x.device):
                    st = lib.tplr_dct2d_inv(_ptr(xin), Y * h, X * w, _ptr(out), X * w, _stream(x.device))
                _lib.check(st, "tplr_dct2d_inv")
                return out if x.dtype == torch.float32 else out.to(x.dtype)
            out = self._dense(x, Y * h, X * w, h, w, self._basis32(self.b_dict, h, x.device),
                              self._basis32(self.b_dict, w, x.device), True, False)
            return out if x.dtype == torch.float32 else out.to(x.dtype)
        if not use_dct:
            return x.reshape(-1)
        _need_device(x, "ChunkingTransformer.decode(use_dct=True)")
        n1 = x.shape[1]
        if n1 == _CH and self._fast64:
            lib = _lib.load()
            xin = _f32c(x)
            out = torch.empty_like(xin)
            with _on(x.device):
                st = lib.tplr_dct1d(_ptr(xin), xin.shape[0], 1, _ptr(out), _stream(x.device))
            _lib.check(st, "tplr_dct1d")
            out = out.reshape(-1)
            return out if x.dtype == torch.float32 else out.to(x.dtype)
        return self.einsum_2d_t(x, self._basis32(self.b_dict, n1, x.device)).reshape(-1)


_FLAT_DESC: dict = {}


def _flat_desc(rows: int, dev: torch.device) -> torch.Tensor:
    """Device descriptor of one un-chunked tensor of `rows` payload rows (what the flat-payload
    kernels take for a single parameter); a few hundred distinct sizes per model, kept."""
    import numpy as np

    key = (dev, rows)
    t = _FLAT_DESC.get(key)
    if t is None:
        if len(_FLAT_DESC) >= 4096:
            _FLAT_DESC.clear()
        desc = np.zeros(1, dtype=np.dtype([("dense", "<u8"), ("ld", "<i8"), ("chunk_begin", "<i8"), ("x_chunks", "<i4"),
                                           ("y_chunks", "<i4")]))
        desc[0] = (0, 0, 0, rows, 1)
        t = _FLAT_DESC[key] = torch.from_numpy(desc.view(np.uint8).copy()).to(dev)
    return t


# ----------------------------------------------------------------------------------------
# kernels behind TopKCompressor
# ----------------------------------------------------------------------------------------
def _as_chunk_view(x: torch.Tensor):
    """If x is the zero-copy (Y, X, 64, 64) view of a row-major (R, C) fp32 tensor that
    encode(use_dct=False) returns, give (R, C, ld); else None."""
    if x.dim() != 4 or x.dtype != torch.float32 or x.shape[2] != _CH or x.shape[3] != _CH:
        return None
    Y, X = x.shape[0], x.shape[1]
    s = x.stride()
    ld = s[2]
    if s[3] == 1 and s[1] == _CH and ld >= X * _CH and (s[0] == _CH * ld or Y == 1):
        return Y * _CH, X * _CH, ld
    return None


def _clamp_k(last_dim: int, topk: int) -> int:
    k = max(min(int(topk), int(last_dim)), 2)
    return k - (k % 2)


def _row_layout(xshape: tuple) -> tuple[int, int]:
    """(number of rows, row length) of the flattened-last-dims view compress/decompress use."""
    if len(xshape) > 2:
        return xshape[0] * xshape[1], xshape[2] * xshape[3]
    return (math.prod(xshape[:-1]) if len(xshape) > 1 else 1), xshape[-1]


def _topk_rows(rows: torch.Tensor, k: int):
    """rows (n_rows, n) fp32 contiguous on device -> (packed idx uint8, val (n_rows, k))."""
    n_rows, n = rows.shape
    if n > _lib.TPLR_MAX_ROW:  # (the 12-bit index ends there as well)
        raise NotImplementedError(f"top-{k} of rows of {n}: the HIP select kernel handles rows up to {_lib.TPLR_MAX_ROW}")
    lib = _lib.load()
    idx = torch.empty(n_rows * (k // 2) * 3, dtype=torch.uint8, device=rows.device)
    val = torch.empty((n_rows, k), dtype=torch.float32, device=rows.device)
    if n_rows:
        with _on(rows.device):
            st = lib.tplr_topk_pack(_ptr(rows), n_rows, n, k, _ptr(idx), _ptr(val), _stream(rows.device))
        _lib.check(st, "tplr_topk_pack")
    return idx, val


def _encode_topk(x2d: torch.Tensor, R: int, Cc: int, ld: int, k: int, use_dct: bool):
    lib = _lib.load()
    n_chunks = (R // _CH) * (Cc // _CH)
    if k > _lib.TPLR_MAX_K and n_chunks:
        # more entries than the fused kernel's select holds: the chunked (transformed) tensor is written out
        # and every chunk sorted whole - exact, far slower; no setting of templar's comes here
        coef = torch.empty((n_chunks, _CH * _CH), dtype=torch.float32, device=x2d.device)
        with _on(x2d.device):
            if use_dct:
                st = lib.tplr_dct2d_fwd(_ptr(x2d), R, Cc, ld, _ptr(coef), _stream(x2d.device))
                _lib.check(st, "tplr_dct2d_fwd")
            else:
                coef.view(R // _CH, Cc // _CH, _CH, _CH).copy_(
                    torch.as_strided(x2d, (R // _CH, Cc // _CH, _CH, _CH), (ld * _CH, _CH, ld, 1)))
        idx, val = _topk_rows(coef, k)
        return idx, val.view(R // _CH, Cc // _CH, k)
    idx = torch.empty(n_chunks * (k // 2) * 3, dtype=torch.uint8, device=x2d.device)
    val = torch.empty((R // _CH, Cc // _CH, k), dtype=torch.float32, device=x2d.device)
    if n_chunks:
        with _on(x2d.device):
            st = lib.tplr_encode_topk_pack(_ptr(x2d), R, Cc, ld, k, int(use_dct), _ptr(idx), _ptr(val),
                                           _stream(x2d.device))
        _lib.check(st, "tplr_encode_topk_pack")
    return idx, val


def _peer_scales(vals: Sequence[torch.Tensor], block_norms: torch.Tensor | None, dev: torch.device) -> torch.Tensor:
    """Clip factors min(1, median / (norm_p + 1e-8)) on the device (reference :526-535, :553-556)."""
    lib = _lib.load()
    P = len(vals)
    if P > _lib.TPLR_MAX_PEERS:
        raise NotImplementedError(f"{P} peers: the HIP aggregate kernel takes up to {_lib.TPLR_MAX_PEERS}")
    scale = torch.empty(P, dtype=torch.float32, device=dev)
    with _on(dev):
        if block_norms is not None:
            norms = block_norms.to(device=dev, dtype=torch.float32).reshape(-1).contiguous()
            n_norms = norms.numel()
            # the reference takes the median of every entry (:535) and indexes norms[i] per peer (:554)
            if n_norms < P:
                raise IndexError(f"index {n_norms} is out of bounds for dimension 0 with size {n_norms}")
            if n_norms > _lib.TPLR_MAX_PEERS:
                raise NotImplementedError(f"{n_norms} block norms: the clip kernel takes up to {_lib.TPLR_MAX_PEERS}")
            if n_norms > P:
                scale = torch.empty(n_norms, dtype=torch.float32, device=dev)
            st = lib.tplr_clip_scales(_ptr(norms), n_norms, 0, _ptr(scale), None, _stream(dev))
            scale = scale[:P]
        else:
            ptrs = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
            n = vals[0].numel()
            if any(v.numel() != n for v in vals):
                raise ValueError("batch_decompress: all peers must send the same number of values")
            # about 32 K values per block, so that one large tensor still spreads over the device
            slices = max(1, min(256, n // 32768))
            ss = torch.empty((P, slices), dtype=torch.float32, device=dev)
            _lib.check(lib.tplr_peer_sumsq(ptrs, P, n, slices, _ptr(ss), _stream(dev)), "tplr_peer_sumsq")
            st = lib.tplr_clip_scales(_ptr(ss), P, slices, _ptr(scale), None, _stream(dev))
    _lib.check(st, "tplr_clip_scales")
    return scale


def _aggregate_chunks(idxs: Sequence[torch.Tensor], vals: Sequence[torch.Tensor], scale: torch.Tensor | None,
                      Y: int, X: int, k: int, *, normalise: bool, use_dct: bool, mean: bool = True,
                      out: torch.Tensor | None = None, sumsq: torch.Tensor | None = None,
                      rows: bool = False) -> torch.Tensor:
    """Fused unpack + scatter over peers (+ inverse DCT) on 64x64 chunks.  Without the transform
    the result is the dense coefficient tensor (Y, X, 64, 64), or with `rows` the (R, C) tensor."""
    lib = _lib.load()
    P = len(vals)
    dev = vals[0].device
    if P > _lib.TPLR_MAX_PEERS:
        raise NotImplementedError(f"{P} peers: the HIP aggregate kernel takes up to {_lib.TPLR_MAX_PEERS}")
    n_chunks = Y * X
    for i, v in zip(idxs, vals):
        if v.numel() != n_chunks * k or i.numel() * 2 != n_chunks * k * 3:
            raise RuntimeError(
                f"payload size mismatch: {i.numel()} index bytes / {v.numel()} values for {n_chunks} chunks, k={k}"
            )
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    vp = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
    R, Cc = Y * _CH, X * _CH
    as_rows = use_dct or rows
    if out is None:
        out = torch.empty((R, Cc) if as_rows else (Y, X, _CH, _CH), dtype=torch.float32, device=dev)
    if n_chunks:
        with _on(dev):
            st = lib.tplr_decode_aggregate(ip, vp, _ptr(scale), P, k, R, Cc,
                                           _lib.REDUCE_MEAN if mean else _lib.REDUCE_SUM, int(normalise), int(use_dct),
                                           _ptr(out), out.stride(0) if as_rows else 0, _ptr(sumsq), _stream(dev))
        _lib.check(st, "tplr_decode_aggregate")
    return out


def _scatter_rows(idx: torch.Tensor, val: torch.Tensor, n_rows: int, kk: int, row_len: int, *,
                  validate: bool = True) -> torch.Tensor:
    """Generic rows: idx is packed uint8 or int64, val is (rows_sent, kk) with rows_sent <= n_rows
    (torch's scatter lets the index cover fewer rows than the target; the rest stay zero)."""
    if row_len > _lib.TPLR_MAX_ROW:
        raise NotImplementedError(f"rows of {row_len}: the HIP scatter kernel handles rows up to {_lib.TPLR_MAX_ROW}")
    lib = _lib.load()
    dev = val.device
    rows_sent = val.numel() // kk if kk else 0
    if rows_sent > n_rows:
        raise RuntimeError(f"{rows_sent} rows of values for a target of {n_rows} rows")
    out = torch.empty((n_rows, row_len), dtype=torch.float32, device=dev)
    if rows_sent < n_rows:
        out[rows_sent:].zero_()
    n_rows = rows_sent
    if n_rows == 0:
        return out
    err = torch.zeros(1, dtype=torch.int32, device=dev)
    packed = idx.dtype == torch.uint8
    with _on(dev):
        st = lib.tplr_scatter_rows(_ptr(idx) if packed else None, None if packed else _ptr(idx), _ptr(val), n_rows, kk,
                                   row_len, _lib.REDUCE_MEAN, _ptr(out), _ptr(err), _stream(dev))
    _lib.check(st, "tplr_scatter_rows")
    bad = int(err.item()) if validate else 0  # the reference's scatter raises on an out-of-range index as well
    if bad:
        raise RuntimeError(f"index {bad} is out of bounds for dimension -1 with size {row_len}")
    return out


class LazyAggregate:
    """What batch_decompress returns when `defer=True`: the peers' payloads plus clip factors,
    not yet scattered.  ChunkingTransformer.decode() turns it into the dense gradient with the
    fused kernel; `.dense()` gives the coefficient tensor the reference would have returned."""

    def __init__(self, idxs, vals, scale, xshape, k, normalise, dtype):
        self.idxs, self.vals, self.scale = idxs, vals, scale
        self.shape = tuple(xshape)
        self.k, self.normalise, self.dtype = k, normalise, dtype
        self.device = vals[0].device

    def dense(self) -> torch.Tensor:
        Y, X = self.shape[0], self.shape[1]
        out = _aggregate_chunks(self.idxs, self.vals, self.scale, Y, X, self.k, normalise=self.normalise, use_dct=False)
        return out if self.dtype == torch.float32 else out.to(self.dtype)

    def decode(self, *, use_dct: bool) -> torch.Tensor:
        Y, X = self.shape[0], self.shape[1]
        out = _aggregate_chunks(self.idxs, self.vals, self.scale, Y, X, self.k, normalise=self.normalise,
                                use_dct=use_dct, rows=True)
        return out if self.dtype == torch.float32 else out.to(self.dtype)


# ----------------------------------------------------------------------------------------
# TopKCompressor (reference :295-696)
# ----------------------------------------------------------------------------------------
class TopKCompressor:
    """Top-k sparsifier with 12-bit index packing and the optional 8-bit value quantiser."""

    use_quantization: bool
    n_bins: int
    range_in_sigmas: int

    def __class_getitem__(cls, item):  # TopKCompressor[Literal[True]] in annotations
        return cls

    @torch.no_grad()
    def __init__(self, *, use_quantization: bool = False, quantization_bins: int = 256,
                 quantization_range: int = 6) -> None:
        self.use_quantization = use_quantization
        if self.use_quantization:
            self.n_bins = quantization_bins
            self.range_in_sigmas = quantization_range

    def _clamp_topk(self, x, topk) -> int:
        """min(topk, last dim), at least 2, rounded down to even (reference :352-367)."""
        return _clamp_k(x.shape[-1], topk)

    @torch.no_grad()
    def compress(self, x: torch.Tensor, topk: int):
        """Top-k by magnitude per chunk / row -> (packed idx, values, xshape, totalk[, qparams])
        (reference :385-423).  Values come out in descending-magnitude order."""
        if _DT and isinstance(x, _DT):
            x = x.to_local()
        xshape = x.shape
        _need_device(x, "TopKCompressor.compress")
        totalk = (x.shape[2] * x.shape[3]) if x.dim() > 2 else x.shape[-1]
        topk = _clamp_k(totalk, topk)

        view = _as_chunk_view(x)
        if view is not None:
            R, Cc, ld = view  # the un-transformed chunk view of a dense tensor: select straight from it
            idx, val = _encode_topk(x, R, Cc, ld, topk, use_dct=False)
        else:
            rows = _f32c(x).reshape(-1, totalk)
            idx, val = _topk_rows(rows, topk)
            val = val.reshape(tuple(x.shape[:2]) + (topk,)) if x.dim() > 2 else val.reshape(tuple(x.shape[:-1]) + (topk,))
        if val.dtype != x.dtype:
            val = val.to(x.dtype)
        if self.use_quantization:
            val, qparams = self._quantize_values(val)
            return idx, val, xshape, totalk, qparams
        return idx, val, xshape, totalk

    @torch.no_grad()
    def decompress(self, p: torch.Tensor, idx: torch.Tensor, val: torch.Tensor, xshape: ShapeT, totalk: int,
                   quantize_params: QuantParamsT | None = None) -> torch.Tensor:
        """Scatter values back into a zero tensor of `xshape`, averaging duplicates
        (reference :425-481).  `p` only supplies device and dtype."""
        if self.use_quantization and quantize_params is not None:
            val = self._dequantize_values(val, quantize_params)
        if idx.dtype not in (torch.uint8, torch.int64):
            raise ValueError(f"Expected uint8 (packed) or int64 (unpacked) indices, got {idx.dtype}")
        _need_device(p, "TopKCompressor.decompress")
        dev = p.device
        val = _f32c(val.to(dev))
        idx = idx.to(dev).contiguous()
        xshape = tuple(xshape)
        kk = val.shape[-1]
        n_rows, row_len = _row_layout(xshape)
        if (len(xshape) > 2 and xshape[2] == _CH and xshape[3] == _CH and idx.dtype == torch.uint8 and kk % 2 == 0
                and kk >= 2 and val.numel() == n_rows * kk):
            out = _aggregate_chunks([idx.reshape(-1)], [val], None, xshape[0], xshape[1], kk, normalise=False,
                                    use_dct=False)
        else:
            if idx.dtype == torch.uint8:
                if kk % 2:
                    # the reference's unpack rejects an odd count
                    raise ValueError(f"Number of indices must be even, got {val.numel()}")
                if idx.numel() * 2 != val.numel() * 3:
                    raise RuntimeError(f"{idx.numel()} packed bytes cannot hold {val.numel()} 12-bit indices")
            elif idx.numel() != val.numel():
                raise RuntimeError(f"index shape {tuple(idx.shape)} does not match values {tuple(val.shape)}")
            out = _scatter_rows(idx.reshape(-1), val, n_rows, kk, row_len).reshape(xshape)
        return out if p.dtype == torch.float32 else out.to(p.dtype)

    @torch.no_grad()
    def batch_decompress(self, p: torch.Tensor, idx: torch.Tensor | Sequence[torch.Tensor],
                         val: torch.Tensor | Sequence[torch.Tensor], xshape: ShapeT, totalk: int,
                         quantize_params: Sequence[QuantParamsT] | None = None, *,
                         block_norms: torch.Tensor | None = None, normalise: bool = False, clip_norm: bool = True,
                         defer: bool = False):
        """Combine several peers' payloads: per-peer median-norm clip (or per-chunk
        normalisation), then the coefficient-wise mean over the peers that sent each
        coefficient (reference :483-580).  With `defer=True` (an extension) the scatter is
        postponed so that ChunkingTransformer.decode() can run it fused with the inverse DCT."""
        if quantize_params is not None and not isinstance(quantize_params, list):
            quantize_params = [quantize_params] * len(val)
        val_list = list(val) if isinstance(val, (list, tuple)) else [val]
        idx_list = list(idx) if isinstance(idx, (list, tuple)) else [idx]
        if self.use_quantization and quantize_params:
            val_list = [self._dequantize_values(v, quantize_params[i]) for i, v in enumerate(val_list)]
        for i_data in idx_list:
            if i_data.dtype != torch.uint8:
                raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i_data.dtype}")
        _need_device(p, "TopKCompressor.batch_decompress")
        dev = p.device
        vals = [_val_on(v, dev) for v in val_list]
        idxs = [_idx_on(i, dev) for i in idx_list]
        xshape = tuple(xshape)
        k = vals[0].shape[-1]
        scale = None
        if clip_norm and not normalise:
            scale = _peer_scales(vals, block_norms, dev)
        chunked = len(xshape) > 2 and xshape[2] == _CH and xshape[3] == _CH and k % 2 == 0 and \
            all(v.shape[-1] == k and v.numel() == xshape[0] * xshape[1] * k for v in vals)
        if chunked:
            if defer:
                return LazyAggregate(idxs, vals, scale, xshape, k, normalise, p.dtype)
            out = _aggregate_chunks(idxs, vals, scale, xshape[0], xshape[1], k, normalise=normalise, use_dct=False)
            return out if p.dtype == torch.float32 else out.to(p.dtype)
        # generic layout (1-D tensors, un-chunked rows)
        n_rows, row_len = _row_layout(xshape)
        sent = vals[0].numel() // k if k else 0
        if (not normalise and k >= 2 and k % 2 == 0 and 0 < sent <= n_rows and row_len <= _lib.TPLR_MAX_ROW
                and len(vals) <= _lib.TPLR_MAX_PEERS and all(v.numel() == sent * k and v.shape[-1] == k for v in vals)
                and all(i.numel() * 2 == sent * k * 3 for i in idxs)):
            # all peers in one launch: entries added in peer order, as the concatenation is (reference :559-580)
            lib = _lib.load()
            P = len(vals)
            out = torch.empty((n_rows, row_len), dtype=torch.float32, device=dev)
            if sent < n_rows:
                out[sent:].zero_()  # torch's scatter lets the index cover fewer rows than the target
            err = torch.zeros(1, dtype=torch.int32, device=dev)
            ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
            vp = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
            with _on(dev):
                st = lib.tplr_aggregate_rows(ip, vp, _ptr(scale), P, k, _ptr(_flat_desc(sent, dev)), 1, sent, row_len,
                                             _lib.REDUCE_MEAN, _ptr(out), _ptr(err), _stream(dev))
            _lib.check(st, "tplr_aggregate_rows")
            bad = int(err.item())  # the reference's scatter raises on an out-of-range index as well
            if bad:
                raise RuntimeError(f"index {bad} is out of bounds for dimension -1 with size {row_len}")
            out = out.reshape(xshape)
            return out if p.dtype == torch.float32 else out.to(p.dtype)
        # peers of different sizes, per-row normalisation: unpack, scale, concatenate in peer order
        # (reference :559-575), then one row scatter
        parts_i, parts_v = [], []
        for pi, (i_data, v) in enumerate(zip(idxs, vals)):
            v2 = v.reshape(-1, v.shape[-1])
            if normalise and v.dim() == 1:
                # a single row of values: the reference divides by the norm itself, and only when it
                # exceeds 1e-8 (:548-551)
                nrm = torch.linalg.vector_norm(v)
                v2 = torch.where(nrm > 1e-8, v2 / nrm, v2)
            elif normalise:
                v2 = v2 / (torch.linalg.vector_norm(v2, dim=1, keepdim=True) + 1e-8)
            elif scale is not None:
                v2 = v2 * scale[pi]
            parts_i.append(unpack_12bit_indices(i_data, v2.shape))
            parts_v.append(v2)
        cat_i = torch.cat(parts_i, dim=1).contiguous()
        cat_v = torch.cat(parts_v, dim=1).contiguous()
        out = _scatter_rows(cat_i, cat_v, n_rows, cat_v.shape[1], row_len).reshape(xshape)
        return out if p.dtype == torch.float32 else out.to(p.dtype)

    # -- statistical 8-bit quantiser (reference :582-696); payload-sized torch ops ----------
    @torch.no_grad()
    def _quantize_values(self, val: torch.Tensor) -> tuple[torch.Tensor, QuantParamsT]:
        half = self.n_bins // 2
        n = val.numel()
        if (val.is_cuda and val.dtype == torch.float32 and n >= 4 and n % 4 == 0 and self.n_bins <= 256
                and (val.data_ptr() % 16 == 0 or not val.is_contiguous())):  # (the kernel reads 16 bytes at a time)
            # one launch (sums in double) instead of a dozen reductions and scatters; the scale is the
            # only value that travels to the host, as in the reference (float(scale), :620)
            lib = _lib.load()
            dev = val.device
            v = val.contiguous()
            q = torch.empty(val.shape, dtype=torch.uint8, device=dev)
            stats = torch.empty(2, dtype=torch.float32, device=dev)
            lookup = torch.empty(self.n_bins, dtype=torch.float32, device=dev)
            slices = max(1, min(256, n // 16384))
            work = torch.empty(slices * (2 + 2 * self.n_bins), dtype=torch.float64, device=dev)
            with _on(dev):
                st = lib.tplr_quantize_batch(_ptr(v), 4, _ptr(_flat_desc(n // 4, dev)), 1, self.n_bins,
                                             C.c_float(self.range_in_sigmas), slices, _ptr(work), _ptr(q),
                                             _ptr(stats[0:1]), _ptr(stats[1:2]), _ptr(lookup), _stream(dev))
            _lib.check(st, "tplr_quantize_batch")
            return q, (stats[0], float(stats[1]), half, lookup, val.dtype)
        shift = val.mean()
        centred = val - shift
        scale = self.range_in_sigmas * (centred.norm() / math.sqrt(centred.numel() - 1)) / self.n_bins
        if scale == 0 or torch.isnan(scale) or torch.isinf(scale):
            scale = torch.tensor(1.0, dtype=centred.dtype, device=val.device)
        c32 = centred.to(torch.float32)
        q = (c32 / scale + half).round().clamp(0, self.n_bins - 1).to(torch.uint8)
        bins = q.flatten().long()
        sums = torch.zeros(self.n_bins, dtype=torch.float32, device=q.device).scatter_add_(0, bins, c32.flatten())
        counts = torch.zeros(self.n_bins, dtype=torch.float32, device=q.device).scatter_add_(
            0, bins, torch.ones_like(c32.flatten()))
        lookup = torch.where(counts > 0, sums / counts, torch.zeros_like(sums))
        return q, (shift, float(scale), half, lookup, val.dtype)

    @torch.no_grad()
    def _dequantize_values(self, val: torch.Tensor, qparams: QuantParamsT) -> torch.Tensor:
        if val.dtype != torch.uint8:
            return val
        if val.is_cuda:
            fast = self._dequantize_peers([val], [qparams], val.device)
            if fast is not None:
                return fast[0]
        shift, _, _, lookup, orig_dtype = qparams
        if isinstance(lookup, torch.Tensor):
            lookup = lookup.to(val.device)
        return (lookup[val.long()] + shift).to(orig_dtype)

    def _dequantize_peers(self, vals, qparams, device) -> list[torch.Tensor] | None:
        """All peers' codes of one parameter in one launch, when they are plain: uint8 on one HIP device,
        equal sizes (a multiple of 4), fp32 targets, a 5-tuple for every peer.  None otherwise."""
        P = len(vals)
        dev = torch.device(device)
        if dev.type != "cuda" or P == 0 or P > _lib.TPLR_MAX_PEERS or len(qparams) < P:
            return None
        if dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        n = vals[0].numel()
        if n == 0 or n % 4:
            return None
        vals = [v if v.device == dev else v.to(dev, non_blocking=True) for v in vals]
        for v, qp in zip(vals, qparams):
            if qp is None or len(qp) != 5 or qp[4] != torch.float32 or not isinstance(qp[3], torch.Tensor) \
                    or v.numel() != n or v.device != dev or not v.is_contiguous():
                return None
        try:
            lookup, shift, n_bins = _qparam_tables(qparams[:P], dev)
        except (RuntimeError, TypeError):
            return None
        if n_bins > 256:
            return None
        lib = _lib.load()
        outs = [torch.empty(v.shape, dtype=torch.float32, device=dev) for v in vals]
        cp = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
        op = (C.c_void_p * P)(*[o.data_ptr() for o in outs])
        with _on(dev):
            st = lib.tplr_dequantize_peers(cp, P, n, _ptr(lookup), _ptr(shift), n_bins, op, _stream(dev))
        _lib.check(st, "tplr_dequantize_peers")
        return outs

    def maybe_dequantize_values(self, vals: list[torch.Tensor], qparams: list[QuantParamsT],
                                device: torch.device) -> list[torch.Tensor]:
        """Dequantise a list of per-peer values when all of them are uint8 (reference :646-696)."""
        if not isinstance(vals, (list, tuple)):
            vals = [vals]
        if qparams is None or not all(v.dtype == torch.uint8 for v in vals):
            return vals
        if isinstance(qparams, tuple) and len(qparams) == 5 and not all(
                isinstance(q, (tuple, list)) and len(q) == 5 for q in qparams):
            qparams = [qparams]  # a single 5-tuple
        if not isinstance(qparams, list):
            qparams = [qparams]
        fast = self._dequantize_peers(vals, qparams, device)
        if fast is not None:
            return fast
        out: list[torch.Tensor] = []
        for i, v in enumerate(vals):
            v = v.to(device)
            if v.dtype == torch.uint8:
                if qparams[i] is None:
                    import logging
                    logging.getLogger("templar").warning(f"Missing quant_params for vals[{i}]]; skip.")
                    break
                v = self._dequantize_values(v, qparams[i]).to(device)
            out.append(v)
        if len(out) != len(vals):
            raise IndexError(f"Mismatch in val lengths: dequant({len(out)}) vs original({len(vals)})")
        return out


# ----------------------------------------------------------------------------------------
# fused entry points (what the callers' back-to-back calls amount to)
# ----------------------------------------------------------------------------------------
@torch.no_grad()
def encode_compress(x: torch.Tensor, topk: int, *, use_dct: bool = True):
    """encode(x, use_dct) followed by compress(., topk) for a 2-D fp32 tensor whose dimensions
    are multiples of 64 (src/tplr/neurons.py:155-159), in one kernel: the 2-D DCT of every
    64x64 chunk stays in registers and only indices and values are written.
    Returns (packed idx, values (Y, X, k), xshape (Y, X, 64, 64), totalk 4096)."""
    _need_device(x, "encode_compress")
    if x.dim() != 2 or x.shape[0] % _CH or x.shape[1] % _CH:
        raise ValueError(f"encode_compress needs a 2-D tensor with dimensions divisible by {_CH}, got {tuple(x.shape)}")
    R, Cc = x.shape
    k = max(min(topk, _CH * _CH), 2)
    k -= k % 2
    xin = x if (x.dtype == torch.float32 and x.stride(1) == 1 and x.stride(0) >= Cc) else _f32c(x)
    idx, val = _encode_topk(xin, R, Cc, xin.stride(0), k, use_dct)
    return idx, val, (R // _CH, Cc // _CH, _CH, _CH), _CH * _CH


@torch.no_grad()
def batch_decompress_decode(idxs: Sequence[torch.Tensor], vals: Sequence[torch.Tensor], xshape: ShapeT, *,
                            block_norms: torch.Tensor | None = None, normalise: bool = False,
                            clip_norm: bool = True, use_dct: bool = True, mean: bool = True,
                            out: torch.Tensor | None = None, sumsq: torch.Tensor | None = None) -> torch.Tensor:
    """batch_decompress(...) followed by decode(., use_dct) (src/tplr/neurons.py:355-367) in one
    kernel per tensor: unpack, clip, scatter-mean over the peers and inverse DCT per chunk in
    LDS; the per-peer dense tensors and the dense coefficient tensor never exist in memory.
    `mean=False` gives the plain sum; `sumsq` (n_chunks floats) receives per-chunk sums of
    squares of the result for callers that normalise it."""
    xshape = tuple(xshape)
    if len(xshape) != 4 or xshape[2] != _CH or xshape[3] != _CH:
        raise ValueError(f"batch_decompress_decode needs xshape (Y, X, {_CH}, {_CH}), got {xshape}")
    for i in idxs:
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
    dev = vals[0].device
    _need_device(vals[0], "batch_decompress_decode")
    vals = [_val_on(v, dev) for v in vals]
    idxs = [_idx_on(i, dev) for i in idxs]
    scale = None
    if clip_norm and not normalise:
        scale = _peer_scales(vals, block_norms, dev)
    return _aggregate_chunks(idxs, vals, scale, xshape[0], xshape[1], vals[0].shape[-1], normalise=normalise,
                             use_dct=use_dct, mean=mean, out=out, sumsq=sumsq, rows=True)


# ----------------------------------------------------------------------------------------
# whole-gradient-set entry points: one launch for all tensors, flat payloads
# ----------------------------------------------------------------------------------------
class TensorBatch:
    """A set of 2-D fp32 device tensors (dimensions multiples of 64) addressed as one list of
    64x64 chunks: tensor by tensor, chunks row-major.  Holds the device-side descriptor table
    the batch kernels walk.  The flat payload of a batch is indexed by the global chunk id:
    indices of chunk g at byte g*3k/2, values at float g*k.  Build it once per model; the
    tensors' storage must stay where it is (error-feedback buffers, gradients)."""

    def __init__(self, tensors: Sequence[torch.Tensor]):
        import numpy as np

        if not tensors:
            raise ValueError("TensorBatch needs at least one tensor")
        dev = tensors[0].device
        desc = np.zeros(len(tensors), dtype=np.dtype([("dense", "<u8"), ("ld", "<i8"), ("chunk_begin", "<i8"),
                                                      ("x_chunks", "<i4"), ("y_chunks", "<i4")]))
        begin = 0
        self.offsets: list[int] = []
        for i, t in enumerate(tensors):
            _need_device(t, "TensorBatch")
            if t.device != dev or t.dtype != torch.float32 or t.dim() != 2 or t.shape[0] % _CH or t.shape[1] % _CH \
                    or t.stride(1) != 1 or t.stride(0) < t.shape[1]:
                raise ValueError(f"tensor {i}: need fp32, 2-D, row-major, dimensions divisible by {_CH}, one device")
            y, x = t.shape[0] // _CH, t.shape[1] // _CH
            desc[i] = (t.data_ptr(), t.stride(0), begin, x, y)
            self.offsets.append(begin)
            begin += x * y
        self.tensors = list(tensors)  # keeps the storage alive
        self.total_chunks = begin
        self.device = dev
        self.desc = desc  # host copy of the table
        self.table = torch.from_numpy(desc.view(np.uint8).copy()).to(dev)

    def __len__(self) -> int:
        return len(self.tensors)

    def xshape(self, i: int) -> Shape4D:
        t = self.tensors[i]
        return (t.shape[0] // _CH, t.shape[1] // _CH, _CH, _CH)

    def payload_rows(self, i: int) -> int:
        """Rows of payload (chunks) of tensor i."""
        t = self.tensors[i]
        return (t.shape[0] // _CH) * (t.shape[1] // _CH)

    def payload_slice(self, i: int, idx12: torch.Tensor, val: torch.Tensor, k: int):
        """Tensor i's part of a flat payload, in the reference's per-parameter form."""
        y, x, _, _ = self.xshape(i)
        b, n = self.offsets[i], y * x
        return idx12[b * (k // 2) * 3:(b + n) * (k // 2) * 3], val[b:b + n].reshape(y, x, k)


@torch.no_grad()
def encode_compress_batch(batch: TensorBatch, topk: int, *, use_dct: bool = True, idx12: torch.Tensor | None = None,
                          val: torch.Tensor | None = None):
    """encode + compress of every tensor of the batch in one launch (the per-parameter loop of
    src/tplr/neurons.py:114-159).  Returns the flat payload (idx12 uint8, val (total_chunks, k))."""
    lib = _lib.load()
    k = _clamp_k(_CH * _CH, topk)
    n = batch.total_chunks
    if idx12 is None:
        idx12 = torch.empty(n * (k // 2) * 3, dtype=torch.uint8, device=batch.device)
    if val is None:
        val = torch.empty((n, k), dtype=torch.float32, device=batch.device)
    if k > _lib.TPLR_MAX_K:  # tensor by tensor through the whole-row sort
        for i, t in enumerate(batch.tensors):
            ti, tv = _encode_topk(t, t.shape[0], t.shape[1], t.stride(0), k, use_dct)
            si, sv = batch.payload_slice(i, idx12, val, k)
            si.copy_(ti.reshape(si.shape))
            sv.copy_(tv.reshape(sv.shape))
        return idx12, val
    with _on(batch.device):
        st = lib.tplr_encode_topk_pack_batch(_ptr(batch.table), len(batch), n, k, int(use_dct), _ptr(idx12), _ptr(val),
                                             _stream(batch.device))
    _lib.check(st, "tplr_encode_topk_pack_batch")
    return idx12, val


class PeerNorms:
    """The peers' per-parameter norms of a window, kept as one float per payload row.

    The reference takes `torch.linalg.vector_norm` of every peer's values of every parameter when it
    aggregates (src/tplr/neurons.py:346) and batch_decompress clips by their median
    (src/tplr/compress.py:526-556): a pass over all values on the aggregate's critical path.  Here the pass is
    made once per peer when its payload arrives (`arrived`: a row's sum of squares, one launch, which runs
    while the next peer is still in transfer), and the clip factors of the whole window come from those
    figures in two small launches (`clip_scales`), for several batches at once (a model's 2-D parameters and
    its 1-D ones).  The additions have a fixed order, so factors computed on arrival and factors computed from
    the values at aggregate time (`peer_clip_scales_batch`) are the same bits."""

    def __init__(self, batches: "Sequence[TensorBatch | RowBatch]", max_peers: int):
        import numpy as np

        if not batches:
            raise ValueError("PeerNorms needs at least one batch")
        if max_peers < 1 or max_peers > _lib.TPLR_MAX_PEERS:
            raise ValueError(f"max_peers must be in [1, {_lib.TPLR_MAX_PEERS}]")
        dev = batches[0].device
        self.batches, self.max_peers, self.device = list(batches), max_peers, dev
        self.row_begin: list[int] = []
        self.tensor_begin: list[int] = []
        tables, rows, tensors = [], 0, 0
        for b in batches:
            if b.device != dev:
                raise ValueError("PeerNorms: the batches live on different devices")
            d = b.desc.copy()
            d["chunk_begin"] += rows  # this batch's rows follow the previous batches' in the row figures
            tables.append(d)
            self.row_begin.append(rows)
            self.tensor_begin.append(tensors)
            rows += b.total_chunks
            tensors += len(b)
        self.total_rows, self.n_tensors = rows, tensors
        self.table = batches[0].table if len(batches) == 1 else \
            torch.from_numpy(np.concatenate(tables).view(np.uint8).copy()).to(dev)
        self.row_sumsq = torch.empty((max_peers, max(rows, 1)), dtype=torch.float32, device=dev)
        self.slices = max(1, min(64, 4096 // (tensors * max_peers)))
        self._partial = torch.empty((tensors, max_peers, self.slices), dtype=torch.float64, device=dev)
        self._scale = torch.empty((tensors, max_peers), dtype=torch.float32, device=dev)
        self._median = torch.empty(tensors, dtype=torch.float32, device=dev)

    @torch.no_grad()
    def arrived(self, p: int, vals: "Sequence[torch.Tensor | None]") -> None:
        """Peer p's fp32 values have arrived: vals[b] is its flat payload for batch b ((rows, k) or flat; None:
        that part is not here yet).  One launch per part, on the current stream."""
        if not 0 <= p < self.max_peers:
            raise IndexError(f"peer {p} of a window of {self.max_peers}")
        if len(vals) != len(self.batches):
            raise IndexError(f"{len(vals)} payload parts for {len(self.batches)} batches")
        lib = _lib.load()
        with _on(self.device):
            for b, v in zip(range(len(self.batches)), vals):
                if v is None:
                    continue
                n = self.batches[b].total_chunks
                _need_device(v, "PeerNorms.arrived")
                if v.dtype != torch.float32 or not v.is_contiguous() or n == 0 or v.numel() % n:
                    raise RuntimeError(f"batch {b}: {v.numel()} values of {v.dtype} for {n} rows")
                vp = (C.c_void_p * 1)(v.data_ptr())
                op = (C.c_void_p * 1)(self.row_sumsq[p].data_ptr() + 4 * self.row_begin[b])
                _lib.check(lib.tplr_row_sumsq(vp, 1, v.numel() // n, n, op, _stream(self.device)), "tplr_row_sumsq")

    @torch.no_grad()
    def arrived_all(self, b: int, vals: Sequence[torch.Tensor]) -> None:
        """All peers' values of batch b at once (peer p = vals[p]), one launch."""
        P, n = len(vals), self.batches[b].total_chunks
        if P < 1 or P > self.max_peers:
            raise ValueError(f"{P} peers for a window of {self.max_peers}")
        k = vals[0].numel() // max(n, 1)
        for v in vals:
            _need_device(v, "PeerNorms.arrived_all")
            if v.dtype != torch.float32 or not v.is_contiguous() or n == 0 or v.numel() != n * k:
                raise RuntimeError(f"batch {b}: {v.numel()} values of {v.dtype} for {n} rows of {k}")
        lib = _lib.load()
        vp = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
        op = (C.c_void_p * P)(*[self.row_sumsq[p].data_ptr() + 4 * self.row_begin[b] for p in range(P)])
        with _on(self.device):
            _lib.check(lib.tplr_row_sumsq(vp, P, k, n, op, _stream(self.device)), "tplr_row_sumsq")

    @torch.no_grad()
    def clip_scales(self, n_peers: int, *, return_median: bool = False):
        """Clip factors min(1, median_t / (norm_tp + 1e-8)) of the first n_peers peers for every parameter of
        every batch, two launches: a list with one (T_b, n_peers) tensor per batch (views of one buffer, valid
        until the next call); return_median: also the list of (T_b,) medians of the peers' norms."""
        if n_peers < 1 or n_peers > self.max_peers:
            raise ValueError(f"{n_peers} peers for a window of {self.max_peers}")
        lib = _lib.load()
        T = self.n_tensors
        rp = (C.c_void_p * n_peers)(*[self.row_sumsq[p].data_ptr() for p in range(n_peers)])
        scale = self._scale.reshape(-1)[:T * n_peers].view(T, n_peers)
        with _on(self.device):
            _lib.check(lib.tplr_clip_scales_rows(rp, n_peers, _ptr(self.table), T, self.slices, _ptr(self._partial),
                                                 _ptr(scale), _ptr(self._median), _stream(self.device)),
                       "tplr_clip_scales_rows")
        ends = self.tensor_begin[1:] + [T]
        scales = [scale[a:e] for a, e in zip(self.tensor_begin, ends)]
        if return_median:
            return scales, [self._median[a:e] for a, e in zip(self.tensor_begin, ends)]
        return scales


@torch.no_grad()
def peer_clip_scales_batch(batch: "TensorBatch | RowBatch", vals: Sequence[torch.Tensor], k: int, *,
                           return_median: bool = False):
    """(n_tensors, n_peers) clip factors min(1, median_t / (norm_tp + 1e-8)) from flat payloads:
    what outer_step's block_norms and batch_decompress's clip compute per parameter
    (src/tplr/neurons.py:346, src/tplr/compress.py:526-556), for all parameters in three launches (the rows'
    sums of squares of all peers, their sums per parameter, the factors); a window whose payloads were noted
    on arrival (PeerNorms) skips the first, the only one that reads the values.
    return_median: also the (n_tensors,) medians of the peers' norms, the per-parameter clip norms the validator
    keeps for its evaluation updates (clip_norm_dict, neurons/validator.py:3568)."""
    P = len(vals)
    if P > _lib.TPLR_MAX_PEERS:
        raise NotImplementedError(f"{P} peers: the HIP aggregate kernel takes up to {_lib.TPLR_MAX_PEERS}")
    for v in vals:
        if v.numel() != batch.total_chunks * k:
            raise RuntimeError(f"flat payload mismatch: {v.numel()} values for {batch.total_chunks} rows, k={k}")
    norms = PeerNorms([batch], P)
    norms.arrived_all(0, vals)
    if return_median:
        scales, medians = norms.clip_scales(P, return_median=True)
        return scales[0], medians[0]
    return norms.clip_scales(P)[0]


@torch.no_grad()
def batch_decompress_decode_batch(out: TensorBatch, idxs: Sequence[torch.Tensor], vals: Sequence[torch.Tensor], k: int,
                                  *, clip_norm: bool = True, scale: torch.Tensor | None = None, normalise: bool = False,
                                  use_dct: bool = True, mean: bool = True, sumsq: torch.Tensor | None = None,
                                  stats: bool = False) -> "torch.Tensor | None":
    """batch_decompress + decode of every parameter in one launch (src/tplr/neurons.py:309-367):
    peer p's flat payload is (idxs[p], vals[p]); results are written into the tensors of `out`.
    stats=True also returns a (T, 4) tensor {L2 norm, mean, all-finite flag (1.0 / 0.0), sum of squares}
    of every decoded parameter - what outer_step computes next with three more passes over each dense
    gradient (fingerprint norm and mean :380-385, the isfinite test :411/:438) - from two floats per chunk that
    the aggregate kernel leaves on its way."""
    lib = _lib.load()
    P = len(vals)
    if P > _lib.TPLR_MAX_PEERS:
        raise NotImplementedError(f"{P} peers: the HIP aggregate kernel takes up to {_lib.TPLR_MAX_PEERS}")
    n = out.total_chunks
    for i, v in zip(idxs, vals):
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
        if v.dtype != torch.float32 or v.numel() != n * k or i.numel() * 2 != n * k * 3 or not v.is_contiguous():
            raise RuntimeError(f"flat payload mismatch: {i.numel()} index bytes / {v.numel()} values for {n} chunks, k={k}")
    if scale is None and clip_norm and not normalise:
        scale = peer_clip_scales_batch(out, vals, k)
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    vp = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
    if stats:
        if sumsq is not None:
            raise ValueError("stats=True keeps its own per-chunk figures: pass either `sumsq` or `stats`")
        per_chunk = torch.empty((max(n, 1), 2), dtype=torch.float32, device=out.device)
        per_tensor = torch.empty((len(out), 4), dtype=torch.float32, device=out.device)
        with _on(out.device):
            st = lib.tplr_decode_aggregate_stats_batch(ip, vp, _ptr(scale), P, k, _ptr(out.table), len(out), n,
                                                       _lib.REDUCE_MEAN if mean else _lib.REDUCE_SUM, int(normalise),
                                                       int(use_dct), _ptr(per_chunk), _ptr(per_tensor), _stream(out.device))
        _lib.check(st, "tplr_decode_aggregate_stats_batch")
        return per_tensor
    with _on(out.device):
        st = lib.tplr_decode_aggregate_batch(ip, vp, _ptr(scale), P, k, _ptr(out.table), len(out), n,
                                             _lib.REDUCE_MEAN if mean else _lib.REDUCE_SUM, int(normalise), int(use_dct),
                                             _ptr(sumsq), _stream(out.device))
    _lib.check(st, "tplr_decode_aggregate_batch")
    return None


@torch.no_grad()
def aggregate_mean_normalised_batch(out: TensorBatch, idxs: Sequence[torch.Tensor], vals: Sequence[torch.Tensor], k: int,
                                    *, use_dct: bool = True, eps: float = 1e-8, two_pass: bool = False) -> torch.Tensor:
    """The aggregation as the benchmark's workload words it: every peer's payload scatter-summed, inverse
    transform, mean over the peers (the sum divided by their number, whoever sent a coefficient), then
    every tensor divided by its L2 norm (+ eps).  tplr.compress itself has no such mode (batch_decompress
    takes the mean over the senders of each coefficient, src/tplr/compress.py:472-474).
    The transform is orthonormal, so a tensor's norm is that of its summed coefficients: one launch over the
    payloads alone gives the per-chunk sums of squares, a small one the per-tensor factors, and the aggregate
    in sum mode with those factors writes the normalised mean directly - the dense tensors are written once
    and never read.  two_pass=True is the literal order instead (aggregate with the factor 1/P, norms from
    the per-chunk sums of squares of the result, one scaling pass over the dense tensors).
    Returns the (T,) factors 1 / (norm + eps)."""
    lib = _lib.load()
    P, T, n, dev = len(vals), len(out), out.total_chunks, out.device
    ss = torch.empty(n, dtype=torch.float32, device=dev)
    factor = torch.empty(T, dtype=torch.float32, device=dev)
    if two_pass:
        scale = torch.full((T, P), 1.0 / P, dtype=torch.float32, device=dev)
        batch_decompress_decode_batch(out, idxs, vals, k, scale=scale, use_dct=use_dct, mean=False, sumsq=ss)
        with _on(dev):
            _lib.check(lib.tplr_tensor_rnorm(_ptr(ss), _ptr(out.table), T, C.c_float(eps), _ptr(factor), _stream(dev)),
                       "tplr_tensor_rnorm")
            _lib.check(lib.tplr_scale_batch(_ptr(out.table), T, n, _ptr(factor), _stream(dev)), "tplr_scale_batch")
        return factor
    if P > _lib.TPLR_MAX_PEERS:
        raise NotImplementedError(f"{P} peers: the HIP aggregate kernel takes up to {_lib.TPLR_MAX_PEERS}")
    for i, v in zip(idxs, vals):
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
        if v.dtype != torch.float32 or v.numel() != n * k or i.numel() * 2 != n * k * 3 or not v.is_contiguous():
            raise RuntimeError(f"flat payload mismatch: {i.numel()} index bytes / {v.numel()} values for {n} chunks, k={k}")
    scale = torch.empty((T, P), dtype=torch.float32, device=dev)
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    vp = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
    with _on(dev):
        _lib.check(lib.tplr_aggregate_sumsq_batch(ip, vp, None, P, k, _ptr(out.table), T, n, _ptr(ss), _stream(dev)),
                   "tplr_aggregate_sumsq_batch")
        _lib.check(lib.tplr_tensor_rnorm_scales(_ptr(ss), _ptr(out.table), T, P, C.c_float(1.0 / P), C.c_float(eps),
                                                _ptr(factor), _ptr(scale), _stream(dev)), "tplr_tensor_rnorm_scales")
    batch_decompress_decode_batch(out, idxs, vals, k, scale=scale, use_dct=use_dct, mean=False)
    return factor


@torch.no_grad()
def apply_decoded_batch(params: TensorBatch, idx12: torch.Tensor, val: torch.Tensor, k: int, *, alpha: float = 1.0,
                        clip: torch.Tensor | None = None, clip_norm: torch.Tensor | None = None,
                        use_dct: bool = True, on_nonfinite: str = "raise") -> "torch.Tensor | None":
    """param <- param - alpha * decode(decompress(payload * clip)) for every parameter of the set in one launch:
    the validator's per-peer evaluation update (neurons/validator.py:3595-3737, update_model_with_gradient: the
    evaluated peer's values times its clip factor, decompress, decode, p.data.sub_(decoded, alpha=lr *
    eval_lr_factor)).  `idx12`, `val`: that peer's flat payload (de-quantised values); `clip_norm`: (T,) clip norms
    (the validator's clip_norm_dict, one per parameter): the factors min(1, clip_norm_t / (norm_t + 1e-8)) of
    validator.py:3608-3612 are formed here from the payload's own per-parameter norms; or `clip`: (T,) ready
    factors; or neither.  alpha and the factors ride on the values (the transform is linear), so the dense gradient
    is never formed and every parameter is read and written once.  k <= 64.

    The reference tests every decoded gradient for NaN and infinities before it subtracts it and raises
    ValueError for the peer (validator.py:3646-3660, :3677-3680).  The launch makes the same test on the decoded
    values (alpha and the clip factor included, so an overflow of that product counts) chunk by chunk: a chunk
    that holds a non-finite value is not subtracted - the parameter keeps its bits there.  on_nonfinite="raise"
    (default) then raises the reference's ValueError, at the cost of one synchronisation, as the reference's own
    test; every chunk that decoded to finite values HAS been subtracted by then (the reference, too, has
    updated the parameters that precede the offending one), and the same call with `alpha` negated takes the
    update back up to rounding, skipping the same chunks.  "flags" returns the (T,) int32 tensor of flags without
    synchronising (1: some chunk of that parameter was skipped); "ignore" makes no test and subtracts everything."""
    if on_nonfinite not in ("raise", "flags", "ignore"):
        raise ValueError(f"on_nonfinite must be 'raise', 'flags' or 'ignore', got {on_nonfinite!r}")
    lib = _lib.load()
    T, n, dev = len(params), params.total_chunks, params.device
    if idx12.dtype != torch.uint8:
        raise ValueError(f"Expected uint8 for 12-bit packed indices, got {idx12.dtype}")
    if val.dtype != torch.float32 or val.numel() != n * k or idx12.numel() * 2 != n * k * 3 or not val.is_contiguous():
        raise RuntimeError(f"flat payload mismatch: {idx12.numel()} index bytes / {val.numel()} values for {n} chunks, k={k}")
    if k > _CH:
        raise NotImplementedError(f"top-{k}: the fused update handles k up to {_CH}")
    if clip_norm is not None:
        if clip is not None:
            raise ValueError("give clip_norm or clip, not both")
        if clip_norm.numel() != T:
            raise IndexError(f"{clip_norm.numel()} clip norms for {T} parameters")
        slices = max(1, min(64, 4096 // T))
        ss = torch.empty((T, 1, slices), dtype=torch.float32, device=dev)
        vp = (C.c_void_p * 1)(val.data_ptr())
        with _on(dev):
            _lib.check(lib.tplr_segment_sumsq(vp, 1, k, _ptr(params.table), T, slices, _ptr(ss), _stream(dev)),
                       "tplr_segment_sumsq")
        norm = ss.reshape(T, slices).sum(dim=1).sqrt()
        clip = (clip_norm.to(device=dev, dtype=torch.float32).reshape(T) / (norm + 1e-8)).clamp(max=1)
    factor = None
    if clip is not None or alpha != 1.0:
        factor = torch.full((T,), float(alpha), dtype=torch.float32, device=dev)
        if clip is not None:
            if clip.numel() != T:
                raise IndexError(f"{clip.numel()} clip factors for {T} parameters")
            factor = factor * clip.to(device=dev, dtype=torch.float32).reshape(T)
    flags = None if on_nonfinite == "ignore" else torch.zeros(T, dtype=torch.int32, device=dev)
    with _on(dev):
        st = lib.tplr_apply_decoded_batch(_ptr(idx12), _ptr(val), _ptr(factor), k, _ptr(params.table), T, n, int(use_dct),
                                          _ptr(flags), _stream(dev))
    _lib.check(st, "tplr_apply_decoded_batch")
    if on_nonfinite == "raise":
        bad = torch.nonzero(flags).reshape(-1).tolist()  # synchronises, as the reference's isnan().any() does
        if bad:
            raise ValueError(f"Invalid gradient: the decoded gradient of parameter {bad[0]} contains NaN/Inf "
                             f"({len(bad)} of {T} parameters affected; their non-finite chunks were not applied)")
        return None
    return flags


@torch.no_grad()
def outer_step_batch(params: TensorBatch, idxs: Sequence[torch.Tensor], vals: Sequence[torch.Tensor], k: int, lr: float, *,
                     scale: torch.Tensor | None = None, use_dct: bool = True, stats: bool = True):
    """outer_step for every 2-D parameter of a model in one launch (src/tplr/neurons.py:309-447 with the plain
    SGD of neurons/trainer.py:128-130): per parameter the reference forms the peers' block norms, the dense
    gradient decode(batch_decompress(..., clip_norm=True)), its L2 norm and mean for the fingerprint (:380-385),
    tests torch.isfinite(grad).all() (:411, :438) and lets optimizer.step() compute p <- p - lr * grad.  Here the
    aggregate's result is subtracted from the parameters in the launch that forms it, lr and the clip factors
    riding on the values (the transform is linear): the dense gradients are never written.

    `idxs[p]`, `vals[p]`: peer p's flat payload; `scale`: ready (T, P) clip factors (PeerNorms.clip_scales), else
    taken from the values.  Returns (stats, skipped): stats a (T, 4) tensor {grad L2 norm, grad mean, all-finite
    flag, grad sum of squares} per parameter (None without `stats`), skipped the list of parameters left
    untouched because their gradient holds a NaN or an infinity, as the reference leaves them.

    A parameter whose peers' norms are all finite and positive under a finite median has a finite gradient (every
    clipped value is bounded by the median, 15 of them add up per coefficient, the transform's gain is 64), so it
    goes through the fused launch.  Any other parameter - a NaN or infinite norm, a zero factor - is kept out of
    it (its factors become NaN: no chunk of it is written) and served the reference's way afterwards: dense
    gradient, test, subtraction.  Reading the launch's per-parameter flags costs the one synchronisation of
    the call.  Settings the fused launch does not serve (no transform, k > 64, more than 15 peers) take that
    route for every parameter."""
    lib = _lib.load()
    P, T, n, dev = len(vals), len(params), params.total_chunks, params.device
    if lr == 0 or lr != lr:
        raise ValueError(f"lr must be a non-zero number, got {lr}")
    for i, v in zip(idxs, vals):
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
        if v.dtype != torch.float32 or v.numel() != n * k or i.numel() * 2 != n * k * 3 or not v.is_contiguous():
            raise RuntimeError(f"flat payload mismatch: {i.numel()} index bytes / {v.numel()} values for {n} chunks, k={k}")
    if scale is None:
        scale = peer_clip_scales_batch(params, vals, k)
    elif tuple(scale.shape) != (T, P) or scale.dtype != torch.float32 or not scale.is_contiguous():
        raise ValueError(f"scale: expected a contiguous fp32 ({T}, {P}) tensor, got {tuple(scale.shape)}")
    out = torch.zeros((T, 4), dtype=torch.float32, device=dev) if stats else None
    fused = use_dct and 4 <= k <= _CH and P <= 15
    flagged = list(range(T))
    if fused:
        sound = (torch.isfinite(scale) & (scale > 0)).all(dim=1, keepdim=True)
        factor = torch.where(sound, scale * float(lr), torch.full_like(scale, float("nan"))).contiguous()
        flags = torch.zeros(T, dtype=torch.int32, device=dev)
        per_chunk = torch.empty((max(n, 1), 2), dtype=torch.float32, device=dev) if stats else None
        ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
        vp = (C.c_void_p * P)(*[v.data_ptr() for v in vals])
        with _on(dev):
            st = lib.tplr_outer_step_batch(ip, vp, _ptr(factor), P, k, _ptr(params.table), T, n, _ptr(per_chunk), _ptr(out),
                                           _ptr(flags), _stream(dev))
        _lib.check(st, "tplr_outer_step_batch")
        if stats:  # the launch's figures are those of lr * grad
            out[:, 0] /= abs(float(lr))
            out[:, 1] /= float(lr)
            out[:, 3] /= float(lr) * float(lr)
        flagged = torch.nonzero(flags).reshape(-1).tolist()  # the call's one synchronisation
    skipped = []
    for t in flagged:  # the reference's own sequence, one parameter at a time
        y, x = params.xshape(t)[:2]
        sl = [params.payload_slice(t, idxs[p], vals[p], k) for p in range(P)]
        grad = _aggregate_chunks([a.contiguous() for a, _ in sl], [b.contiguous() for _, b in sl], scale[t].contiguous(),
                                 y, x, k, normalise=False, use_dct=use_dct, rows=True)
        finite = bool(torch.isfinite(grad).all())
        if stats:
            ss = (grad.double() ** 2).sum()
            out[t] = torch.stack([ss.sqrt(), grad.double().mean(), torch.tensor(float(finite), device=dev, dtype=torch.float64),
                                  ss]).float()
        if finite:
            params.tensors[t].sub_(grad, alpha=float(lr))
        else:
            skipped.append(t)
    return out, skipped


@torch.no_grad()
def error_feedback_step_batch(ef: TensorBatch, grad: TensorBatch, decay: float, topk: int, *, use_dct: bool = True,
                              compressor: "TopKCompressor | None" = None, null_round: bool = False):
    """The miner's per-parameter loop of src/tplr/neurons.py:147-171 for a whole set of 2-D
    parameters in two launches:

        ef <- ef * decay + grad (or 0 on a null round), in place          (:148-152)
        payload = compress(encode(ef))                                     (:155-159)
        ef <- ef - decode(decompress(payload))                             (:162-171)

    `ef` and `grad` describe the error-feedback tensors and the gradients (same shapes, same
    order).  Returns (idx12, val, quant): the flat payload by global chunk id, and, when
    `compressor` quantises, quant = list of (uint8 values, quant_params) per tensor (what the
    reference's compress returns per parameter), the subtraction then using the de-quantised
    values exactly as the reference's decompress does; otherwise quant is None."""
    lib = _lib.load()
    if len(ef) != len(grad) or ef.offsets != grad.offsets or ef.total_chunks != grad.total_chunks:
        raise ValueError("error-feedback and gradient sets differ in shape")
    k = _clamp_k(_CH * _CH, topk)
    if k > 64:
        raise NotImplementedError(f"top-{k}: the fused error-feedback step handles k up to 64")
    dev, n = ef.device, ef.total_chunks
    idx12 = torch.empty(n * (k // 2) * 3, dtype=torch.uint8, device=dev)
    val = torch.empty((n, k), dtype=torch.float32, device=dev)
    quantises = compressor is not None and compressor.use_quantization
    if use_dct and not quantises and not null_round:
        # nothing sits between the two halves of the step: one launch, every chunk read once and written once
        with _on(dev):
            st = lib.tplr_ef_step_batch(_ptr(ef.table), _ptr(grad.table), len(ef), n, C.c_float(decay), k, _ptr(idx12),
                                        _ptr(val), _stream(dev))
        _lib.check(st, "tplr_ef_step_batch")
        return idx12, val, None
    with _on(dev):
        if null_round:
            for t in ef.tensors:
                t.zero_()
            st = lib.tplr_encode_topk_pack_batch(_ptr(ef.table), len(ef), n, k, int(use_dct), _ptr(idx12), _ptr(val),
                                                 _stream(dev))
        else:
            st = lib.tplr_ef_encode_topk_pack_batch(_ptr(ef.table), _ptr(grad.table), len(ef), n, C.c_float(decay), k,
                                                    int(use_dct), _ptr(idx12), _ptr(val), _stream(dev))
    _lib.check(st, "tplr_ef_encode_topk_pack_batch")
    quant, sent, codes = None, val, None
    if compressor is not None and compressor.use_quantization:
        codes, shift, scale, lookup = quantize_batch(ef, val, k, compressor.n_bins, compressor.range_in_sigmas)
        sent = dequantize_batch(ef, codes.reshape(-1), None, k, out=torch.empty_like(val), tables=(lookup, shift))
        # the reference's quant_params carry the scale as a Python float (:620): the copy to the host
        # is queued here and read after the subtraction has been launched
        with _on(dev):
            scale_host = torch.empty(len(ef), dtype=torch.float32, pin_memory=True)
            scale_host.copy_(scale, non_blocking=True)
            copied = torch.cuda.Event()
            copied.record()
    with _on(dev):
        if use_dct:
            st = lib.tplr_ef_subtract_batch(_ptr(idx12), _ptr(sent), k, _ptr(ef.table), len(ef), n, 1, _stream(dev))
        else:
            # the payload was selected from these very tensors: a selected position holds the payload's own value,
            # so the tensors need not be read (k scattered stores per chunk instead of k read-modify-writes)
            st = lib.tplr_ef_subtract_own_batch(_ptr(idx12), _ptr(sent), _ptr(val), k, _ptr(ef.table), len(ef), n,
                                                _stream(dev))
    _lib.check(st, "tplr_ef_subtract_batch")
    if codes is not None:
        # the per-parameter form of the reference's compress output
        parts = []
        for i in range(len(ef)):
            y, x, _, _ = ef.xshape(i)
            b = ef.offsets[i]
            parts.append((codes[b:b + y * x].view(y, x, k), shift[i], lookup[i]))
        copied.synchronize()
        half = compressor.n_bins // 2
        quant = [(q, (sh, sc, half, lut, torch.float32)) for (q, sh, lut), sc in zip(parts, scale_host.tolist())]
    return idx12, val, quant


# ---- the 1-D parameters of a model (norm vectors): rows of 64, a handful of launches for all of them ----
class RowBatch:
    """A set of 1-D fp32 device tensors whose lengths are multiples of 64, addressed as one list of
    rows of 64 elements, tensor by tensor (ChunkingTransformer's 1-D layout, reference :244-251 with
    a chunk of 64).  The flat payload of the set is indexed by the global row id, like a
    TensorBatch's by the chunk id: indices of row g at byte g*3k/2, values at float g*k."""

    def __init__(self, tensors: Sequence[torch.Tensor]):
        if not tensors:
            raise ValueError("RowBatch needs at least one tensor")
        dev = tensors[0].device
        self.offsets: list[int] = []
        begin = 0
        for i, t in enumerate(tensors):
            _need_device(t, "RowBatch")
            if t.device != dev or t.dtype != torch.float32 or t.dim() != 1 or t.numel() % _CH or not t.is_contiguous():
                raise ValueError(f"tensor {i}: need fp32, 1-D, contiguous, length divisible by {_CH}, one device")
            self.offsets.append(begin)
            begin += t.numel() // _CH
        self.tensors = list(tensors)
        self.rows = [t.numel() // _CH for t in tensors]
        self.total_rows = begin
        self.device = dev
        # tensors that lie back to back in one allocation (views of a flat parameter buffer) are
        # read and written in place, without a gathering copy
        self.flat = None
        first = tensors[0]
        if all(t.untyped_storage().data_ptr() == first.untyped_storage().data_ptr() for t in tensors) and \
                all(b.data_ptr() == a.data_ptr() + a.numel() * 4 for a, b in zip(tensors, tensors[1:])):
            self.flat = torch.as_strided(first, (begin * _CH,), (1,))
        # row -> tensor id, for per-tensor factors applied to flat payloads
        self.segment = torch.repeat_interleave(torch.arange(len(tensors), device=dev),
                                               torch.tensor(self.rows, device=dev))
        # the descriptor table the flat-payload kernels walk: a tensor's rows in place of its chunks
        import numpy as np

        desc = np.zeros(len(tensors), dtype=np.dtype([("dense", "<u8"), ("ld", "<i8"), ("chunk_begin", "<i8"),
                                                      ("x_chunks", "<i4"), ("y_chunks", "<i4")]))
        for i, (b, n) in enumerate(zip(self.offsets, self.rows)):
            desc[i] = (tensors[i].data_ptr(), _CH, b, n, 1)
        self.desc = desc  # host copy of the table
        self.table = torch.from_numpy(desc.view(np.uint8).copy()).to(dev)
        self.total_groups = sum((n + _CH - 1) // _CH for n in self.rows)  # waves of up to 64 rows of one tensor

    def __len__(self) -> int:
        return len(self.tensors)

    @property
    def total_chunks(self) -> int:  # the flat-payload routines count rows of payload, whatever their length
        return self.total_rows

    def xshape(self, i: int) -> tuple[int, int]:
        return (self.rows[i], _CH)

    def payload_rows(self, i: int) -> int:
        return self.rows[i]

    def payload_slice(self, i: int, idx12: torch.Tensor, val: torch.Tensor, k: int):
        """Tensor i's part of a flat payload, in the reference's per-parameter form (xshape (rows, 64))."""
        b, n = self.offsets[i], self.rows[i]
        return idx12[b * (k // 2) * 3:(b + n) * (k // 2) * 3], val[b:b + n]


@torch.no_grad()
def encode_compress_rows_batch(batch: RowBatch, topk: int, *, use_dct: bool = True, idx12: torch.Tensor | None = None,
                               val: torch.Tensor | None = None):
    """encode + compress of every 1-D tensor of the set (src/tplr/neurons.py:155-159 per parameter) in
    one launch: every tensor is read where it lies, its rows of 64 go through the 64-point transform and the
    top-k in registers.  Returns the flat payload (idx12 uint8, val (total_rows, k)); totalk is 64 for
    every row."""
    lib = _lib.load()
    k = _clamp_k(_CH, topk)
    dev = batch.device
    n = batch.total_rows
    if idx12 is None:
        idx12 = torch.empty(n * (k // 2) * 3, dtype=torch.uint8, device=dev)
    if val is None:
        val = torch.empty((n, k), dtype=torch.float32, device=dev)
    with _on(dev):
        st = lib.tplr_encode_rows_batch(_ptr(batch.table), len(batch), batch.total_groups, k, int(use_dct), _ptr(idx12),
                                        _ptr(val), _stream(dev))
    _lib.check(st, "tplr_encode_rows_batch")
    return idx12, val


@torch.no_grad()
def batch_decompress_decode_rows_batch(out: RowBatch, idxs: Sequence[torch.Tensor], vals: Sequence[torch.Tensor], k: int,
                                       *, clip_norm: bool = True, use_dct: bool = True, validate: bool = True,
                                       two_step: bool = False, scale: torch.Tensor | None = None) -> None:
    """batch_decompress + decode (src/tplr/neurons.py:341-367) of every 1-D parameter at once: peer p's
    flat payload is (idxs[p], vals[p]).  Per parameter and peer the values are clipped to the median
    norm over the peers (reference :526-556), every row takes the mean over the peers that sent each
    element (:574-580), the rows go back through the 64-point transform and into the tensors of `out`.
    The payloads are a few hundred KB: a fixed, small number of launches whatever the number of
    parameters.  `validate` (default) raises on an index of 64 or more, as torch's scatter does, which
    costs a synchronisation; without it such entries are dropped.  `two_step` keeps the aggregate and the
    transform as two launches with the rows in a buffer between them (the same bits).  `scale`: ready (T, P) clip
    factors (PeerNorms.clip_scales) instead of the norms taken here."""
    lib = _lib.load()
    P, R, T, dev = len(vals), out.total_rows, len(out), out.device
    for i, v in zip(idxs, vals):
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
        if v.dtype != torch.float32 or v.numel() != R * k or i.numel() * 2 != R * k * 3:
            raise RuntimeError(f"flat payload mismatch: {i.numel()} index bytes / {v.numel()} values for {R} rows, k={k}")
    vals = [_val_on(x, dev) for x in vals]
    idxs = [_idx_on(i, dev) for i in idxs]
    if scale is None and clip_norm:
        scale = peer_clip_scales_batch(out, vals, k)                                  # (T, P), three launches
    elif scale is not None and (tuple(scale.shape) != (T, P) or scale.dtype != torch.float32 or not scale.is_contiguous()):
        raise ValueError(f"scale: expected a contiguous fp32 ({T}, {P}) tensor, got {tuple(scale.shape)}")
    err = torch.zeros(1, dtype=torch.int32, device=dev) if validate else None
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    vp = (C.c_void_p * P)(*[x.data_ptr() for x in vals])
    if k <= _CH and not two_step:
        # one launch: scatter-mean of every row, its inverse transform, written into its tensor
        with _on(dev):
            st = lib.tplr_decode_rows_batch(ip, vp, _ptr(scale), P, k, _ptr(out.table), T, R, _lib.REDUCE_MEAN,
                                            int(use_dct), _ptr(err), _stream(dev))
        _lib.check(st, "tplr_decode_rows_batch")
        if validate:
            bad = int(err.item())  # torch's scatter raises on an out-of-range index as well
            if bad:
                raise RuntimeError(f"index {bad} is out of bounds for dimension -1 with size {_CH}")
        return
    rows = torch.empty((R, _CH), dtype=torch.float32, device=dev)
    with _on(dev):
        st = lib.tplr_aggregate_rows(ip, vp, _ptr(scale), P, k, _ptr(out.table), T, R, _CH, _lib.REDUCE_MEAN, _ptr(rows),
                                     _ptr(err), _stream(dev))
    _lib.check(st, "tplr_aggregate_rows")
    if validate:
        bad = int(err.item())  # torch's scatter raises on an out-of-range index as well
        if bad:
            raise RuntimeError(f"index {bad} is out of bounds for dimension -1 with size {_CH}")
    if use_dct:
        dec = out.flat.view(R, _CH) if out.flat is not None else torch.empty_like(rows)
        with _on(dev):
            st = lib.tplr_dct1d(_ptr(rows), R, 1, _ptr(dec), _stream(dev))
        _lib.check(st, "tplr_dct1d")
        if out.flat is not None:
            return
        rows = dec
    if out.flat is not None:
        out.flat.copy_(rows.reshape(-1))
    else:
        torch._foreach_copy_(out.tensors, list(rows.reshape(-1).split([t.numel() for t in out.tensors])))


@torch.no_grad()
def outer_step_rows_batch(params: RowBatch, idxs: Sequence[torch.Tensor], vals: Sequence[torch.Tensor], k: int, lr: float, *,
                          scale: torch.Tensor | None = None, use_dct: bool = True, stats: bool = True):
    """outer_step_batch for the 1-D parameters (src/tplr/neurons.py:341-447 with the plain SGD of
    neurons/trainer.py:128-130): the peers' payloads are aggregated and decoded in one launch into a scratch
    copy of the set (a few hundred KB for a model's norm vectors), every parameter whose gradient is finite
    takes p <- p - lr * grad, the others keep their bits.  Returns (stats, skipped) as outer_step_batch does."""
    if lr == 0 or lr != lr:
        raise ValueError(f"lr must be a non-zero number, got {lr}")
    dev = params.device
    grads = [torch.empty_like(t) for t in params.tensors]
    batch_decompress_decode_rows_batch(RowBatch(grads), idxs, vals, k, clip_norm=scale is None, use_dct=use_dct,
                                       validate=False, scale=scale)
    flat = torch.cat([g.reshape(-1) for g in grads]).double()
    sizes = torch.tensor([g.numel() for g in grads], device=dev)
    seg = torch.repeat_interleave(torch.arange(len(grads), device=dev), sizes)
    ss = torch.zeros(len(grads), dtype=torch.float64, device=dev).index_add_(0, seg, flat * flat)
    sm = torch.zeros(len(grads), dtype=torch.float64, device=dev).index_add_(0, seg, flat)
    finite = torch.isfinite(ss) & torch.isfinite(sm)  # a NaN or an infinity in a gradient shows in its sums
    keep = finite.tolist()  # the call's one synchronisation
    good = [i for i, ok in enumerate(keep) if ok]
    if good:
        torch._foreach_sub_([params.tensors[i] for i in good], [grads[i] for i in good], alpha=float(lr))
    out = None
    if stats:
        out = torch.stack([ss.sqrt(), sm / sizes.double(), finite.double(), ss], dim=1).float()
    return out, [i for i, ok in enumerate(keep) if not ok]


@torch.no_grad()
def error_feedback_step_rows_batch(ef: RowBatch, grad: RowBatch, decay: float, topk: int, *, use_dct: bool = True,
                                   compressor: "TopKCompressor | None" = None, null_round: bool = False):
    """error_feedback_step_batch for the 1-D parameters: the loop body of src/tplr/neurons.py:147-171
    for all of them in about ten launches.  Returns (idx12, val, quant) as its 2-D counterpart does."""
    lib = _lib.load()
    if len(ef) != len(grad) or ef.rows != grad.rows:
        raise ValueError("error-feedback and gradient sets differ in shape")
    k = _clamp_k(_CH, topk)
    dev, R, T = ef.device, ef.total_rows, len(ef)
    # tensors that are not views of one buffer are gathered into one, worked on there and copied back
    ef_flat = ef.flat if ef.flat is not None else torch.cat(ef.tensors)
    if null_round:
        ef_flat.zero_()                                        # :148-149
    else:
        g_flat = grad.flat if grad.flat is not None else torch.cat(grad.tensors)
        with _on(dev):                                         # :151-152, two roundings
            _lib.check(lib.tplr_flat_update(_ptr(ef_flat), _ptr(g_flat), ef_flat.numel(), C.c_float(decay), 0,
                                            _stream(dev)), "tplr_flat_update")
    work = ef if ef.flat is not None else RowBatch(list(ef_flat.split([t.numel() for t in ef.tensors])))
    idx12, val = encode_compress_rows_batch(work, k, use_dct=use_dct)    # :155-159
    quant, sent = None, val
    if compressor is not None and compressor.use_quantization:
        codes, shift, scale, lookup = quantize_batch(ef, val, k, compressor.n_bins, compressor.range_in_sigmas)
        sent = dequantize_batch(ef, codes.reshape(-1), None, k, tables=(lookup, shift))
        half = compressor.n_bins // 2
        quant = [(codes[b:b + n], (shift[i], sc, half, lookup[i], torch.float32))
                 for i, (b, n, sc) in enumerate(zip(ef.offsets, ef.rows, scale.tolist()))]
    # :162-171: the sent part back through decompress + decode, subtracted from the error feedback
    rows = torch.empty((R, _CH), dtype=torch.float32, device=dev)
    ip, vp = (C.c_void_p * 1)(idx12.data_ptr()), (C.c_void_p * 1)(sent.data_ptr())
    with _on(dev):
        st = lib.tplr_aggregate_rows(ip, vp, None, 1, k, None, 0, R, _CH, _lib.REDUCE_MEAN, _ptr(rows), None, _stream(dev))
        _lib.check(st, "tplr_aggregate_rows")
        if use_dct:
            dec = torch.empty_like(rows)
            _lib.check(lib.tplr_dct1d(_ptr(rows), R, 1, _ptr(dec), _stream(dev)), "tplr_dct1d")
            rows = dec
        _lib.check(lib.tplr_flat_update(_ptr(ef_flat), _ptr(rows), ef_flat.numel(), C.c_float(0.0), 1, _stream(dev)),
                   "tplr_flat_update")
    if ef.flat is None:
        torch._foreach_copy_(ef.tensors, list(ef_flat.split([t.numel() for t in ef.tensors])))
    return idx12, val, quant


def check_compressed_indices(param_name: str, idxs, totalk: int, allowed_topk: int | None = None,
                             vals: torch.Tensor | None = None, *, topk_compression: int | None = None) -> None:
    """Validation of one parameter's packed indices as Comms.check_compressed_indices does it
    (src/tplr/comms.py:2538-2610), with its error messages: uint8 tensor, values present,
    non-empty, last dimension == min(allowed top-k, totalk), every index in [0, totalk).
    `topk_compression` stands in for the reference's `self.hparams.topk_compression` when
    `allowed_topk` is not given.  Works on host and device tensors; raises ValueError."""
    if allowed_topk is None:
        if topk_compression is None:
            raise TypeError("check_compressed_indices needs allowed_topk or topk_compression")
        allowed_topk = min(int(topk_compression), totalk)
    else:
        allowed_topk = min(allowed_topk, totalk)
    if not isinstance(idxs, torch.Tensor):
        raise ValueError(f"[{param_name}] Expected tensor but got {type(idxs)}")
    if idxs.dtype != torch.uint8:
        raise ValueError(f"[{param_name}] Expected uint8 for 12-bit packed indices, got {idxs.dtype}")
    if vals is None:
        raise ValueError(f"[{param_name}] Values tensor required to validate 12-bit packed indices")
    if idxs.numel() == 0:
        raise ValueError(f"[{param_name}] Empty packed indices tensor")
    try:
        unpacked = unpack_12bit_indices(idxs, vals.shape)
        if unpacked.shape[-1] != allowed_topk:
            raise ValueError(f"[{param_name}] Invalid topk dimension: "
                             f"shape[-1]={unpacked.shape[-1]} but expected {allowed_topk}")
        if unpacked.numel() == 0:
            raise ValueError(f"[{param_name}] empty index list")
        if unpacked.min().item() < 0 or unpacked.max().item() >= totalk:
            bad = unpacked[(unpacked < 0) | (unpacked >= totalk)][0].item()
            raise ValueError(f"[{param_name}] Index {bad} out of bounds (totalk = {totalk})")
    except Exception as e:  # the reference wraps every failure the same way (:2607-2608)
        raise ValueError(f"[{param_name}] Failed to unpack 12-bit indices: {e}")


def _qparam_tables(qparams: Sequence[QuantParamsT], dev: torch.device) -> tuple[torch.Tensor, torch.Tensor, int]:
    """(rows, n_bins) lookups and (rows,) shifts of a list of quant_params 5-tuples on `dev`: stacked
    where they live, moved once.  The reference de-quantises to `(lookup[code] + shift).to(orig_dtype)`
    (src/tplr/compress.py:641-643): a tuple whose fifth entry is not float32 gets its row as that sum rounded
    through that dtype, with a zero shift, so that the kernels' fp32 `lookup[code] + shift` gives the rounded
    value exactly.  All tuples must come from quantisers of one size."""
    n_bins = int(qparams[0][3].numel())
    if any(int(qp[3].numel()) != n_bins for qp in qparams):
        sizes = sorted({int(qp[3].numel()) for qp in qparams})
        raise ValueError(f"quant_params of quantisers of different sizes in one call: lookup tables of {sizes} entries")
    try:  # the usual case: every lookup a flat fp32 tensor, every shift a 0-dim fp32 tensor, one device
        lookup = torch.stack([qp[3] for qp in qparams])
        shift = torch.stack([qp[0] for qp in qparams])
        if lookup.dtype != torch.float32 or shift.dtype != torch.float32 or lookup.shape != (len(qparams), n_bins) \
                or shift.shape != (len(qparams),):
            raise TypeError
    except (TypeError, RuntimeError):
        lookup = torch.stack([qp[3].reshape(n_bins).float() for qp in qparams])
        shift = torch.stack([torch.as_tensor(qp[0], dtype=torch.float32, device=lookup.device).reshape(())
                             for qp in qparams])
    narrow = [r for r, qp in enumerate(qparams) if len(qp) > 4 and isinstance(qp[4], torch.dtype) and qp[4] != torch.float32]
    if narrow:
        lookup, shift = lookup.clone(), shift.clone()
        for r in narrow:
            dt = qparams[r][4]
            if not dt.is_floating_point:
                raise NotImplementedError(f"quant_params with orig_dtype {dt}")
            lookup[r] = (lookup[r] + shift[r]).to(dt).float()
            shift[r] = 0.0
    return lookup.to(dev).contiguous(), shift.to(dev).contiguous(), n_bins


@torch.no_grad()
def quantize_batch(batch: TensorBatch, val: torch.Tensor, k: int, n_bins: int = 256, range_in_sigmas: float = 6.0):
    """TopKCompressor._quantize_values (reference :582-621) for every parameter of a flat payload
    in one launch: codes (total_chunks, k) uint8, and per parameter shift (T,), scale (T,) and
    lookup (T, n_bins), all on the device.  Sums are carried in double and rounded once."""
    lib = _lib.load()
    dev, n, T = batch.device, batch.total_chunks, len(batch)
    if val.dtype != torch.float32 or val.numel() != n * k or not val.is_contiguous():
        raise RuntimeError(f"{val.numel()} values of {val.dtype} for {n} chunks of k={k}")
    codes = torch.empty((n, k), dtype=torch.uint8, device=dev)
    shift = torch.empty(T, dtype=torch.float32, device=dev)
    scale = torch.empty(T, dtype=torch.float32, device=dev)
    lookup = torch.empty((T, n_bins), dtype=torch.float32, device=dev)
    if k % 4:
        # the whole-set kernel reads the values four at a time; a top-k that is not a multiple of four (the clamp
        # only makes it even) goes parameter by parameter through the compressor's own quantiser, on the device
        comp = TopKCompressor(use_quantization=True, quantization_bins=n_bins, quantization_range=range_in_sigmas)
        for i in range(T):
            b, rows = batch.offsets[i], batch.payload_rows(i)
            q, (sh, sc, _, lk, _) = comp._quantize_values(val[b:b + rows])
            codes[b:b + rows].copy_(q)
            shift[i], scale[i] = sh, sc
            lookup[i].copy_(lk)
        return codes, shift, scale, lookup
    slices = max(1, min(64, 2048 // T))  # enough workgroups to fill the device
    work = torch.empty(T * slices * (2 + 2 * n_bins), dtype=torch.float64, device=dev)
    with _on(dev):
        st = lib.tplr_quantize_batch(_ptr(val), k, _ptr(batch.table), T, n_bins, C.c_float(range_in_sigmas), slices,
                                     _ptr(work), _ptr(codes), _ptr(shift), _ptr(scale), _ptr(lookup), _stream(dev))
    _lib.check(st, "tplr_quantize_batch")
    return codes, shift, scale, lookup


@torch.no_grad()
def dequantize_batch(batch: TensorBatch, codes: torch.Tensor, qparams: Sequence[QuantParamsT] | None, k: int,
                     out: torch.Tensor | None = None, *, tables: tuple[torch.Tensor, torch.Tensor] | None = None
                     ) -> torch.Tensor:
    """One peer's flat payload of 8-bit codes -> fp32 values (total_chunks, k), every parameter
    with its own (shift, lookup): TopKCompressor.maybe_dequantize_values' per-parameter loop
    (reference :646-696, src/tplr/neurons.py:325) in one launch.  qparams[i] is parameter i's
    5-tuple as the reference's compress returns it."""
    lib = _lib.load()
    dev, n = batch.device, batch.total_chunks
    if tables is None and len(qparams) != len(batch):
        raise IndexError(f"Mismatch in val lengths: dequant({len(qparams)}) vs original({len(batch)})")
    if codes.dtype != torch.uint8 or codes.numel() != n * k:
        raise RuntimeError(f"{codes.numel()} codes of {codes.dtype} for {n} chunks of k={k}")
    if tables is not None:  # (lookup (T, n_bins), shift (T,)) already on the device, as quantize_batch returns them
        lookup, shift = tables
        n_bins = int(lookup.shape[1])
    else:
        lookup, shift, n_bins = _qparam_tables(qparams, dev)
    if out is None:
        out = torch.empty((n, k), dtype=torch.float32, device=dev)
    if k % 4:  # (see quantize_batch) lookup[t][code] + shift[t] per parameter by torch's device ops
        codes2 = codes.reshape(n, k)
        for i in range(len(batch)):
            b, rows = batch.offsets[i], batch.payload_rows(i)
            out[b:b + rows] = lookup[i][codes2[b:b + rows].long()] + shift[i]
        return out
    with _on(dev):
        st = lib.tplr_dequantize_batch(_ptr(codes.contiguous()), _ptr(lookup), _ptr(shift), n_bins, k, _ptr(batch.table),
                                       len(batch), n, _ptr(out), _stream(dev))
    _lib.check(st, "tplr_dequantize_batch")
    return out


def dequantised_tables(quant_params: Sequence[Sequence[QuantParamsT]], dev: torch.device) -> tuple[torch.Tensor, int]:
    """quant_params[i][p] (parameter i, peer p, the reference's 5-tuples) -> ((T, P, max(n_bins, 4)) fp32 table
    of lookup + shift, n_bins): the value behind every code of every parameter and peer
    (src/tplr/compress.py:641-643), formed by the same fp32 addition as the element-wise form."""
    T, P = len(quant_params), len(quant_params[0])
    lookup, shift, n_bins = _qparam_tables([quant_params[i][p] for i in range(T) for p in range(P)], dev)
    deq = (lookup + shift[:, None]).view(T, P, n_bins)
    if n_bins < 4:
        deq = torch.cat([deq, torch.zeros((T, P, 4 - n_bins), dtype=torch.float32, device=dev)], dim=2)
    return deq.contiguous(), n_bins


@torch.no_grad()
def batch_decompress_decode_codes_batch(out: TensorBatch, idxs: Sequence[torch.Tensor], codes: Sequence[torch.Tensor],
                                        quant_params: Sequence[Sequence[QuantParamsT]], k: int, *,
                                        clip_norm: bool = True, use_dct: bool = False, mean: bool = True,
                                        validate: bool = True,
                                        tables: "tuple[torch.Tensor, int] | None" = None,
                                        stats: bool = False) -> "torch.Tensor | None":
    """maybe_dequantize_values + block norms + batch_decompress + decode of every parameter
    (src/tplr/neurons.py:325-367) from the peers' QUANTISED flat payloads: codes[p] holds peer p's one-byte
    codes (total_chunks * k), quant_params[i][p] parameter i's 5-tuple from peer p.  With templar's settings - a
    quantiser of at most four bins, chunks not transformed, k <= 64, at most 24 peers - the fp32 values are
    never written: the norms come from four counts per (parameter, peer), and the aggregate kernel picks every
    entry's value among its peer's four.  Other settings de-quantise first (one launch per peer) and take the
    fp32 path: the same results either way.  `validate` raises on a code the quantiser cannot have produced,
    as the reference's table lookup does, at the cost of a synchronisation.  `tables` = what
    dequantised_tables(quant_params, device) returns, for callers that build it once per window (a few thousand
    small tensors are stacked to make it).  stats=True returns the (T, 4) statistics of the decoded parameters
    as batch_decompress_decode_batch does."""
    lib = _lib.load()
    P, T, n, dev = len(codes), len(out), out.total_chunks, out.device
    if tables is None and (len(quant_params) != T or any(len(q) != P for q in quant_params)):
        raise IndexError("quant_params must hold one entry per parameter and peer")
    for i, c in zip(idxs, codes):
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
        if c.dtype != torch.uint8 or c.numel() != n * k or i.numel() * 2 != n * k * 3 or not c.is_contiguous():
            raise RuntimeError(f"flat payload mismatch: {i.numel()} index bytes / {c.numel()} codes for {n} chunks, k={k}")
    n_bins = int(tables[1]) if tables is not None else int(quant_params[0][0][3].numel())
    if n_bins > 4 or use_dct or k > _CH or P > 24:
        if quant_params is None:
            raise ValueError("these settings de-quantise first: pass quant_params, not only `tables`")
        if validate:  # the reference's table lookup raises on a code past the table (the batch kernel would clamp it)
            worst = int(torch.stack([c.max() for c in codes]).max().item()) if n else 0
            if worst >= n_bins:
                raise IndexError(f"index {worst} is out of bounds for dimension 0 with size {n_bins}")
        vals = []
        for p in range(P):
            vals.append(dequantize_batch(out, codes[p].reshape(-1), [quant_params[i][p] for i in range(T)], k))
        return batch_decompress_decode_batch(out, idxs, vals, k, clip_norm=clip_norm, use_dct=use_dct, mean=mean, stats=stats)
    deq, n_bins = tables if tables is not None else dequantised_tables(quant_params, dev)
    if deq.shape != (T, P, 4) or deq.dtype != torch.float32 or not deq.is_contiguous():
        raise ValueError(f"tables: expected a contiguous fp32 ({T}, {P}, 4) tensor, got {tuple(deq.shape)}")
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    cp = (C.c_void_p * P)(*[c.data_ptr() for c in codes])
    scale = None
    bad = torch.zeros(1, dtype=torch.int32, device=dev) if validate else None
    with _on(dev):
        if clip_norm or validate:
            slices = max(1, min(64, 8192 // (T * P)))
            ss = torch.empty((T, P, slices), dtype=torch.float32, device=dev)
            _lib.check(lib.tplr_code_sumsq(cp, P, k, _ptr(out.table), T, slices, n_bins, _ptr(deq), _ptr(ss), _ptr(bad),
                                           _stream(dev)), "tplr_code_sumsq")
            if clip_norm:
                scale = torch.empty((T, P), dtype=torch.float32, device=dev)
                _lib.check(lib.tplr_clip_scales_batch(_ptr(ss), T, P, slices, _ptr(scale), None, _stream(dev)),
                           "tplr_clip_scales_batch")
        if validate:
            worst = int(bad.item())
            if worst:
                raise IndexError(f"index {worst} is out of bounds for dimension 0 with size {n_bins}")
        if stats:
            per_chunk = torch.empty((max(n, 1), 2), dtype=torch.float32, device=dev)
            per_tensor = torch.empty((T, 4), dtype=torch.float32, device=dev)
            st = lib.tplr_decode_aggregate_codes_stats_batch(ip, cp, _ptr(deq), _ptr(scale), P, k, _ptr(out.table), T, n,
                                                             _lib.REDUCE_MEAN if mean else _lib.REDUCE_SUM,
                                                             _ptr(per_chunk), _ptr(per_tensor), _stream(dev))
            _lib.check(st, "tplr_decode_aggregate_codes_stats_batch")
            return per_tensor
        st = lib.tplr_decode_aggregate_codes_batch(ip, cp, _ptr(deq), _ptr(scale), P, k, _ptr(out.table), T, n,
                                                   _lib.REDUCE_MEAN if mean else _lib.REDUCE_SUM, None, _stream(dev))
    _lib.check(st, "tplr_decode_aggregate_codes_batch")
    return None


@torch.no_grad()
def outer_step_codes_batch(params: TensorBatch, idxs: Sequence[torch.Tensor], codes: Sequence[torch.Tensor],
                           quant_params: "Sequence[Sequence[QuantParamsT]] | None", k: int, lr: float, *,
                           tables: "tuple[torch.Tensor, int] | None" = None, stats: bool = True, validate: bool = True):
    """outer_step_batch at templar's own settings (hparams/hparams.json: 4-bin quantiser, chunks not transformed,
    top-k 64, 20 peers): maybe_dequantize_values, block norms, batch_decompress, decode, the gradient's norm, mean and
    isfinite test and SGD's p <- p - lr * grad (src/tplr/neurons.py:325-447, neurons/trainer.py:128-130) for every
    2-D parameter in one launch straight from the codes - no fp32 copy of the payload, no dense gradient.
    codes[p], quant_params[i][p] / `tables` as in batch_decompress_decode_codes_batch; the payloads must be a staged
    window (PayloadStage.load(..., expand=False)).  Returns (stats, skipped) as outer_step_batch does.  A parameter the
    fused launch cannot vouch for, and settings it does not serve (more than four bins, k other than 32 or 64, more
    than 24 peers, payloads not equally spaced), take the reference's route on de-quantised values inside the call.
    `validate` raises IndexError on a code the quantiser cannot have produced, before anything is written."""
    lib = _lib.load()
    P, T, n, dev = len(codes), len(params), params.total_chunks, params.device
    if lr == 0 or lr != lr:
        raise ValueError(f"lr must be a non-zero number, got {lr}")
    if tables is None and (quant_params is None or len(quant_params) != T or any(len(q) != P for q in quant_params)):
        raise IndexError("quant_params must hold one entry per parameter and peer")
    for i, c in zip(idxs, codes):
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
        if c.dtype != torch.uint8 or c.numel() != n * k or i.numel() * 2 != n * k * 3 or not c.is_contiguous():
            raise RuntimeError(f"flat payload mismatch: {i.numel()} index bytes / {c.numel()} codes for {n} chunks, k={k}")
    deq, n_bins = tables if tables is not None else dequantised_tables(quant_params, dev)

    def dequantised(t=None):
        """fp32 values behind the codes: of parameter t per peer ((rows, k) each), or of everything per peer."""
        if t is None:
            seg = torch.repeat_interleave(torch.arange(T, device=dev),
                                          torch.tensor([params.payload_rows(i) for i in range(T)], device=dev))
            return [deq[seg, p].gather(1, codes[p].view(n, k).long()) for p in range(P)]
        b, rows = params.offsets[t], params.payload_rows(t)
        return [deq[t, p][codes[p].view(n, k)[b:b + rows].long()] for p in range(P)]

    if n_bins > 4 or k not in (32, 64) or P > 24 or deq.shape != (T, P, 4):
        return outer_step_batch(params, idxs, dequantised(), k, lr, use_dct=False, stats=stats)
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    cp = (C.c_void_p * P)(*[c.data_ptr() for c in codes])
    slices = max(1, min(64, 8192 // (T * P)))
    ss = torch.empty((T, P, slices), dtype=torch.float32, device=dev)
    scale = torch.empty((T, P), dtype=torch.float32, device=dev)
    bad = torch.zeros(1, dtype=torch.int32, device=dev)
    with _on(dev):
        _lib.check(lib.tplr_code_sumsq(cp, P, k, _ptr(params.table), T, slices, n_bins, _ptr(deq), _ptr(ss), _ptr(bad),
                                       _stream(dev)), "tplr_code_sumsq")
        _lib.check(lib.tplr_clip_scales_batch(_ptr(ss), T, P, slices, _ptr(scale), None, _stream(dev)),
                   "tplr_clip_scales_batch")
    if validate:
        worst = int(bad.item())
        if worst:
            raise IndexError(f"index {worst} is out of bounds for dimension 0 with size {n_bins}")
    sound = (torch.isfinite(scale) & (scale > 0)).all(dim=1, keepdim=True)
    factor = torch.where(sound, scale * float(lr), torch.full_like(scale, float("nan"))).contiguous()
    flags = torch.zeros(T, dtype=torch.int32, device=dev)
    out = torch.zeros((T, 4), dtype=torch.float32, device=dev) if stats else None
    per_chunk = torch.empty((max(n, 1), 2), dtype=torch.float32, device=dev) if stats else None
    with _on(dev):
        st = lib.tplr_outer_step_codes_batch(ip, cp, _ptr(deq), _ptr(factor), P, k, _ptr(params.table), T, n,
                                             _ptr(per_chunk), _ptr(out), _ptr(flags), _stream(dev))
    if st == _lib.TPLR_E_SHAPE:  # the payloads are not a staged window
        return outer_step_batch(params, idxs, dequantised(), k, lr, use_dct=False, stats=stats)
    _lib.check(st, "tplr_outer_step_codes_batch")
    if stats:  # the launch's figures are those of lr * grad
        out[:, 0] /= abs(float(lr))
        out[:, 1] /= float(lr)
        out[:, 3] /= float(lr) * float(lr)
    skipped = []
    for t in torch.nonzero(flags).reshape(-1).tolist():  # the reference's own sequence, one parameter at a time
        y, x = params.xshape(t)[:2]
        b, rows = params.offsets[t], params.payload_rows(t)
        ti = [i[b * (k // 2) * 3:(b + rows) * (k // 2) * 3].contiguous() for i in idxs]
        grad = _aggregate_chunks(ti, [v.contiguous() for v in dequantised(t)], scale[t].contiguous(), y, x, k,
                                 normalise=False, use_dct=False, rows=True)
        finite = bool(torch.isfinite(grad).all())
        if stats:
            s2 = (grad.double() ** 2).sum()
            out[t] = torch.stack([s2.sqrt(), grad.double().mean(), torch.tensor(float(finite), device=dev, dtype=torch.float64),
                                  s2]).float()
        if finite:
            params.tensors[t].sub_(grad, alpha=float(lr))
        else:
            skipped.append(t)
    return out, skipped


class PayloadStage:
    """One window's payloads of all peers as flat buffers in the layout the batch kernels read.

    The reference keeps a gathered window as per-parameter Python lists, `state_dict.<name>idxs`,
    `<name>vals` and `<name>quant_params`, one entry per peer (src/tplr/comms.py:1938-1963), and moves
    them tensor by tensor (torch.load with map_location :602-606; pinned offload and reload,
    neurons/validator.py:94-219).  Here peer p's parameters are concatenated in TensorBatch order
    into one region of a pinned host buffer, the whole window crosses to the device in one copy,
    and 8-bit codes are expanded on the device by one launch per peer.  Buffers are allocated once
    (`max_peers` regions) and reused every window; the lists `load` returns are views of them,
    valid until the next `load`."""

    _ALIGN = 256

    def __init__(self, batch: TensorBatch, k: int, max_peers: int, *, quantized: bool = True,
                 host_threads: int | None = None, norms: "PeerNorms | None" = None):
        if max_peers < 1 or max_peers > _lib.TPLR_MAX_PEERS:
            raise ValueError(f"max_peers must be in [1, {_lib.TPLR_MAX_PEERS}]")
        if k < 2 or k % 2:
            raise ValueError(f"k must be even and at least 2, got {k}")
        n = batch.total_chunks
        self.batch, self.k, self.max_peers, self.quantized = batch, k, max_peers, quantized
        self.idx_bytes = n * (k // 2) * 3
        self.val_bytes = n * k * (1 if quantized else 4)
        up = lambda b: -(-b // self._ALIGN) * self._ALIGN  # noqa: E731
        self.val_off = up(self.idx_bytes)
        self.stride = self.val_off + up(self.val_bytes)
        self.host = torch.empty(max_peers * self.stride, dtype=torch.uint8, pin_memory=True)
        self.dev = torch.empty(max_peers * self.stride, dtype=torch.uint8, device=batch.device)
        self.values: torch.Tensor | None = None  # fp32 copy of a quantised window, made by the first load that expands
        self._copied: torch.cuda.Event | None = None  # the last host-to-device copy out of `host`
        self._val_sizes = [batch.payload_rows(i) * k for i in range(len(batch))]
        self._idx_sizes = [v // 2 * 3 for v in self._val_sizes]
        self._threads = max(1, min(64, host_threads if host_threads else min(8, os.cpu_count() or 1)))
        # norms: a PeerNorms whose first batch is `batch`; every load then leaves each peer's row figures there as
        # soon as the peer's fp32 values are on the device, so the window's clip factors need no pass over them
        if norms is not None and (norms.batches[0] is not batch or norms.max_peers < max_peers):
            raise ValueError("norms: its first batch must be this stage's batch, its window at least as wide")
        self.norms = norms
        self.tables = None

    @torch.no_grad()
    def offload(self, n_peers: int) -> None:
        """The staged window back into the pinned host buffer in one copy (what
        offload_gather_results, neurons/validator.py:94-160, does tensor by tensor to free the device
        during evaluation).  The device buffer stays allocated; its contents may be overwritten
        until `reload`."""
        n = n_peers * self.stride
        with _on(self.dev.device):
            self.host[:n].copy_(self.dev[:n], non_blocking=True)
            self._copied = torch.cuda.Event()
            self._copied.record()

    @torch.no_grad()
    def reload(self, n_peers: int):
        """The offloaded window onto the device again (neurons/validator.py:162-219), one copy; returns
        the lists `load` returned.  De-quantised values are rebuilt by the caller's next `load` only when
        the stage holds codes: here the codes come back and are expanded again."""
        n = n_peers * self.stride
        with _on(self.dev.device):
            self.dev[:n].copy_(self.host[:n], non_blocking=True)
        out_i, out_v = [], []
        for p in range(n_peers):
            ri, rv = self._regions(self.dev, p)
            out_i.append(ri)
            out_v.append(rv.view(-1, self.k))
        if not self.quantized:
            return out_i, out_v
        lookup, shift = self._tables
        T = len(self.batch)
        values = self._expanded()
        for p in range(n_peers):
            dequantize_batch(self.batch, out_v[p].reshape(-1), None, self.k, out=values[p],
                             tables=(lookup[p * T:(p + 1) * T], shift[p * T:(p + 1) * T]))
        return out_i, [values[p] for p in range(n_peers)]

    def _expanded(self) -> torch.Tensor:
        if self.values is None:
            self.values = torch.empty((self.max_peers, self.batch.total_chunks, self.k), dtype=torch.float32,
                                      device=self.dev.device)
        return self.values

    def regions(self, p: int) -> tuple[torch.Tensor, torch.Tensor]:
        """Peer p's place in the device buffer: (packed indices, values (n, k) or codes).  The peers'
        places are equally spaced, which is what lets the aggregate kernels address them with scalar
        arithmetic; payloads produced on the device (tests, benchmarks, a local peer) can be written here
        directly."""
        ri, rv = self._regions(self.dev, p)
        return ri, rv.view(-1, self.k)

    def _regions(self, buf: torch.Tensor, p: int) -> tuple[torch.Tensor, torch.Tensor]:
        b = p * self.stride
        idx = buf[b:b + self.idx_bytes]
        val = buf[b + self.val_off:b + self.val_off + self.val_bytes]
        return idx, (val if self.quantized else val.view(torch.float32))

    @torch.no_grad()
    def load(self, idxs: Sequence[Sequence[torch.Tensor]], vals: Sequence[Sequence[torch.Tensor]],
             quant_params: Sequence[Sequence[QuantParamsT]] | None = None, *, expand: bool = True):
        """`idxs[i][p]`, `vals[i][p]`, `quant_params[i][p]`: parameter i (TensorBatch order), peer p, as in
        the reference's lists.  Host tensors go through the pinned buffer and one copy; device tensors
        are concatenated on the device.  Returns (idx12, val): lists over peers of the flat packed
        indices and the fp32 values (total_chunks, k), ready for batch_decompress_decode_batch,
        peer_clip_scales_batch and index_stats_batch.  expand=False (a stage that holds codes) leaves the
        codes as they are: it returns them in place of the values and keeps `self.tables`, what
        batch_decompress_decode_codes_batch takes as `tables` to aggregate straight from them."""
        T = len(self.batch)
        if len(idxs) != T or len(vals) != T:
            raise IndexError(f"{len(idxs)} index lists / {len(vals)} value lists for {T} parameters")
        P = len(idxs[0])
        if P < 1 or P > self.max_peers:
            raise ValueError(f"{P} peers for a stage of {self.max_peers}")
        want_dtype = torch.uint8 if self.quantized else torch.float32
        for p in range(P):  # sizes and types of all tensors of a peer, compared as lists
            try:
                pi, pv = [row[p] for row in idxs], [row[p] for row in vals]
            except IndexError:
                raise IndexError(f"every parameter needs {P} index and value entries") from None
            if [a.numel() for a in pi] != self._idx_sizes or [v.numel() for v in pv] != self._val_sizes:
                bad = next(i for i in range(T) if pi[i].numel() != self._idx_sizes[i] or pv[i].numel() != self._val_sizes[i])
                raise RuntimeError(f"parameter {bad}, peer {p}: {pi[bad].numel()} index bytes / {pv[bad].numel()} values for "
                                   f"{self._val_sizes[bad] // self.k} chunks of k={self.k}")
            for a in pi:
                if a.dtype != torch.uint8:
                    raise ValueError(f"Expected uint8 for 12-bit packed indices, got {a.dtype}")
            for v in pv:
                if v.dtype != want_dtype:
                    raise ValueError(f"peer {p}: values are {v.dtype}, the stage holds {want_dtype}")
        if any(len(row) != P for row in idxs) or any(len(row) != P for row in vals):
            raise IndexError(f"every parameter needs {P} index and value entries")
        on_host = idxs[0][0].device.type == "cpu"
        if any(t.device.type != idxs[0][0].device.type for row in list(idxs) + list(vals) for t in row):
            raise ValueError("PayloadStage.load: the lists mix host and device tensors")
        if on_host and self._copied is not None:
            self._copied.synchronize()  # the previous window's copy still reads the pinned buffer
        if on_host:
            # per peer: the library's host threads concatenate the parameters' tensors into the
            # peer's region of the pinned buffer, whose transfer then runs while the next peer is packed
            lib = _lib.load()
            with _on(self.dev.device):
                for p in range(P):
                    for part, off, nbytes in ((idxs, 0, self.idx_bytes), (vals, self.val_off, self.val_bytes)):
                        src = [part[i][p] if part[i][p].is_contiguous() else part[i][p].contiguous() for i in range(T)]
                        ptrs = (C.c_void_p * T)(*[t.data_ptr() for t in src])
                        sizes = (C.c_int64 * T)(*[t.numel() * t.element_size() for t in src])
                        _lib.check(lib.tplr_gather_host(ptrs, sizes, T, self.host.data_ptr() + p * self.stride + off,
                                                        self._threads), "tplr_gather_host")
                    b = p * self.stride
                    self.dev[b:b + self.stride].copy_(self.host[b:b + self.stride], non_blocking=True)
                self._copied = torch.cuda.Event()
                self._copied.record()
        else:
            for p in range(P):
                ri, rv = self._regions(self.dev, p)
                torch.cat([idxs[i][p].reshape(-1) for i in range(T)], out=ri)
                torch.cat([vals[i][p].reshape(-1) for i in range(T)], out=rv)
        out_i, out_v = [], []
        self.tables = None
        for p in range(P):
            ri, rv = self._regions(self.dev, p)
            out_i.append(ri)
            out_v.append(rv.view(-1, self.k))
        if not self.quantized:
            self._note_arrivals(out_v)
            return out_i, out_v
        if quant_params is None or len(quant_params) != T or any(len(q) != P for q in quant_params):
            raise IndexError("quant_params must hold one entry per parameter and peer")
        if not expand:
            self.tables = dequantised_tables(quant_params, self.dev.device)
            return out_i, out_v
        lookup, shift, n_bins = _qparam_tables([quant_params[i][p] for p in range(P) for i in range(T)], self.dev.device)
        values = self._expanded()
        for p in range(P):
            dequantize_batch(self.batch, out_v[p].reshape(-1), None, self.k, out=values[p],
                             tables=(lookup[p * T:(p + 1) * T], shift[p * T:(p + 1) * T]))
        self._tables = (lookup, shift)  # alive until the launches above have run
        self._note_arrivals([values[p] for p in range(P)])
        return out_i, [values[p] for p in range(P)]

    def _note_arrivals(self, vals: Sequence[torch.Tensor]) -> None:
        if self.norms is not None:
            rest = [None] * (len(self.norms.batches) - 1)
            for p, v in enumerate(vals):
                self.norms.arrived(p, [v] + rest)


@torch.no_grad()
def index_stats_batch(batch: "TensorBatch | RowBatch | Sequence[int]", idxs: Sequence[torch.Tensor], k: int):
    """Checks on P peers' packed index streams in one launch.

    `batch` is a TensorBatch (rows = its 64x64 chunks), a RowBatch, or a list of row counts per
    parameter for payloads whose rows are not chunks.  Returns (pair, dup, top):
      pair (T, P, P) int64: pair[t, i, j] for i < j = entries of peer i that also occur in the same
          row of peer j, summed over parameter t's rows - what check_uid_index_overlap
          (src/tplr/neurons.py:1373-1378) sums before dividing by k and averaging over rows;
      dup (T, P) int64: repeated entries inside a row (a top-k selection has none);
      top (T, P) int32: the largest index, for the bounds check of check_compressed_indices
          (src/tplr/comms.py:2573-2581)."""
    import numpy as np

    lib = _lib.load()
    P = len(idxs)
    if P > 32:
        raise NotImplementedError(f"{P} peers: the index statistics kernel takes up to 32")
    dev = idxs[0].device
    _need_device(idxs[0], "index_stats_batch")
    if isinstance(batch, (TensorBatch, RowBatch)):
        table, T, total = batch.table, len(batch), batch.total_chunks
    else:
        counts = [int(c) for c in batch]
        desc = np.zeros(len(counts), dtype=np.dtype([("dense", "<u8"), ("ld", "<i8"), ("chunk_begin", "<i8"),
                                                     ("x_chunks", "<i4"), ("y_chunks", "<i4")]))
        begin = 0
        for i, c in enumerate(counts):
            desc[i] = (0, 0, begin, c, 1)
            begin += c
        table, T, total = torch.from_numpy(desc.view(np.uint8).copy()).to(dev), len(counts), begin
    for i in idxs:
        if i.dtype != torch.uint8:
            raise ValueError(f"Expected uint8 for 12-bit packed indices, got {i.dtype}")
        if i.numel() * 2 != total * k * 3:
            raise RuntimeError(f"{i.numel()} index bytes for {total} rows of k={k}")
    pair = torch.zeros((T, P, P), dtype=torch.int64, device=dev)
    dup = torch.zeros((T, P), dtype=torch.int64, device=dev)
    top = torch.full((T, P), -1, dtype=torch.int32, device=dev)
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    with _on(dev):
        st = lib.tplr_index_stats_batch(ip, P, k, _ptr(table), T, total, _ptr(pair), _ptr(dup), _ptr(top), _stream(dev))
    _lib.check(st, "tplr_index_stats_batch")
    return pair, dup, top


def overlap_fractions(pair: torch.Tensor, rows: Sequence[int], k: int) -> torch.Tensor:
    """Size-weighted average overlap per peer pair from index_stats_batch's counts: what
    check_uid_index_overlap accumulates in pair_acc (src/tplr/neurons.py:1376-1385, :1393):
    sum_t mean_frac_t * (C_t k) / sum_t (C_t k) = sum_t pair[t] / (k sum_t C_t)."""
    total = float(sum(int(r) for r in rows)) * k
    return pair.sum(dim=0).double() / total


# the DeMo-era names of the two classes
TransformDCT = ChunkingTransformer
CompressDCT = TopKCompressor

__all__ = [
    "pack_12bit_indices", "unpack_12bit_indices", "ChunkingTransformer", "TopKCompressor", "TransformDCT",
    "CompressDCT", "encode_compress", "batch_decompress_decode", "LazyAggregate", "TensorBatch",
    "encode_compress_batch", "batch_decompress_decode_batch", "aggregate_mean_normalised_batch", "apply_decoded_batch", "outer_step_batch", "outer_step_rows_batch", "outer_step_codes_batch", "batch_decompress_decode_codes_batch", "dequantised_tables", "peer_clip_scales_batch", "error_feedback_step_batch", "index_stats_batch", "overlap_fractions", "dequantize_batch", "quantize_batch", "PayloadStage", "PeerNorms", "RowBatch", "encode_compress_rows_batch", "batch_decompress_decode_rows_batch", "error_feedback_step_rows_batch", "check_compressed_indices", "ShapeT", "Shape4D", "TotK",
    "IdxT", "ValT", "QuantParamsT", "_dct", "_idct", "_get_smaller_split", "_get_divisors", "_get_prime_divisors",
]
