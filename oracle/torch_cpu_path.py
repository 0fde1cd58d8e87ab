"""The reference's op sequence on torch tensors (CPU for the checks and the host baseline; it
follows its inputs' device, so the benchmark can also time it on the GPU).  Test infrastructure only.

This restates src/tplr/compress.py (tplr 2.1.28) as plain functions that issue the same
torch primitives in the same order - strided view + 3-operand einsum, abs/topk(sorted=False)/
gather, strided 12-bit pack, unpack/cat/scatter_reduce_(mean, include_self=False), einsum
back - so that (a) the C oracle can be cross-checked against the installed torch library and
(b) the benchmark has the "reference's PyTorch CPU path" to time on the host cores.
"""
from __future__ import annotations

import math

import torch


# ---- basis: _dct / _idct through the FFT route (:700-788) ----------------------------------
def dct_fft(x: torch.Tensor, ortho: bool = True) -> torch.Tensor:
    n = x.shape[-1]
    rows = x.contiguous().view(-1, n)
    v = torch.cat([rows[:, ::2], rows[:, 1::2].flip([1])], dim=1)          # :725
    spec = torch.view_as_real(torch.fft.fft(v, dim=1))                      # :702
    ang = -torch.arange(n, dtype=x.dtype)[None, :] * math.pi / (2 * n)      # :729
    out = spec[:, :, 0] * torch.cos(ang) - spec[:, :, 1] * torch.sin(ang)   # :733
    if ortho:
        out[:, 0] /= math.sqrt(n) * 2                                       # :736
        out[:, 1:] /= math.sqrt(n / 2) * 2                                  # :737
    return 2 * out.view(*x.shape)                                           # :739


def idct_fft(X: torch.Tensor, ortho: bool = True) -> torch.Tensor:
    n = X.shape[-1]
    xv = X.contiguous().view(-1, n) / 2                                     # :761
    if ortho:
        xv[:, 0] *= math.sqrt(n) * 2                                        # :764
        xv[:, 1:] *= math.sqrt(n / 2) * 2                                   # :765
    ang = torch.arange(n, dtype=X.dtype)[None, :] * math.pi / (2 * n)       # :767-771
    wr, wi = torch.cos(ang), torch.sin(ang)
    tr = xv
    ti = torch.cat([xv[:, :1] * 0, -xv.flip([1])[:, :-1]], dim=1)           # :776
    vr = tr * wr - ti * wi                                                  # :778
    vi = tr * wi + ti * wr                                                  # :779
    v = torch.fft.irfft(torch.view_as_complex(torch.stack([vr, vi], dim=2)), n=n, dim=1)  # :781-783
    x = v.new_zeros(v.shape)
    x[:, ::2] += v[:, : n - (n // 2)]                                       # :785
    x[:, 1::2] += v.flip([1])[:, : n // 2]                                  # :786
    return x.view(*X.shape)


def basis(n: int):
    """f_dict[n], b_dict[n] as ChunkingTransformer.__init__ builds them (:181-184)."""
    eye = torch.eye(n)
    return dct_fft(eye), idct_fft(eye)


# ---- encode / decode (:224-292) -------------------------------------------------------------
def encode(x: torch.Tensor, h: int, w: int, f_h: torch.Tensor, f_w: torch.Tensor, use_dct: bool = True):
    if x.dim() > 1:
        y = x.view(x.shape[0] // h, h, x.shape[1] // w, w).permute(0, 2, 1, 3)   # "(y h) (x w) -> y x h w"
        return torch.einsum("...ijkl, kb, ld -> ...ijbd", y, f_h, f_w) if use_dct else y
    y = x.view(-1, w)
    return torch.einsum("...ij, jb -> ...ib", y, f_w) if use_dct else y


def decode(c: torch.Tensor, b_h: torch.Tensor, b_w: torch.Tensor, use_dct: bool = True):
    if c.dim() > 2:
        if use_dct:
            c = torch.einsum("...ijbd, bk, dl -> ...ijkl", c, b_h, b_w)
        Y, X, h, w = c.shape
        return c.permute(0, 2, 1, 3).reshape(Y * h, X * w)                       # "y x h w -> (y h) (x w)"
    if use_dct:
        c = torch.einsum("...ij, jb -> ...ib", c, b_w)
    return c.reshape(-1)


# ---- pack / unpack (:51-142) ----------------------------------------------------------------
def pack12(indices: torch.Tensor) -> torch.Tensor:
    top = indices.max().item() if indices.numel() > 0 else 0
    if top >= 4096:
        raise ValueError(f"Index {top} exceeds 12-bit limit (4095)")
    flat = indices.flatten()
    if flat.numel() % 2:
        raise ValueError(f"Number of indices must be even, got {flat.numel()}")
    flat = flat.to(torch.int32)
    out = torch.zeros(flat.numel() // 2 * 3, dtype=torch.uint8, device=indices.device)
    if flat.numel():
        a, b = flat.reshape(-1, 2).unbind(1)
        out[0::3] = (a & 0xFF).to(torch.uint8)
        out[1::3] = (((a >> 8) & 0x0F) | ((b & 0x0F) << 4)).to(torch.uint8)
        out[2::3] = ((b >> 4) & 0xFF).to(torch.uint8)
    return out


def unpack12(packed: torch.Tensor, shape) -> torch.Tensor:
    n = int(torch.prod(torch.tensor(shape)).item())
    if n == 0:
        return torch.zeros(shape, dtype=torch.int64, device=packed.device)
    if n % 2:
        raise ValueError(f"Number of indices must be even, got {n}")
    out = torch.zeros(n, dtype=torch.int64, device=packed.device)
    b0, b1, b2 = (packed[i::3].to(torch.int64) for i in range(3))
    out[0::2] = b0 | ((b1 & 0x0F) << 8)
    out[1::2] = ((b1 >> 4) & 0x0F) | (b2 << 4)
    return out.reshape(shape)


# ---- compress / decompress / batch_decompress (:385-580), no quantisation -------------------
def clamp_topk(last: int, topk: int) -> int:
    k = max(min(topk, last), 2)
    return k - k % 2


def compress(x: torch.Tensor, topk: int):
    xshape = x.shape
    if x.dim() > 2:
        x = x.reshape(x.shape[0], x.shape[1], -1)
    totalk = x.shape[-1]
    k = clamp_topk(totalk, topk)
    idx = torch.topk(x.abs(), k=k, dim=-1, largest=True, sorted=False).indices
    val = torch.gather(x, dim=-1, index=idx)
    return pack12(idx), val, xshape, totalk


def decompress(idx: torch.Tensor, val: torch.Tensor, xshape, totalk: int, dtype=torch.float32):
    x = torch.zeros(xshape, dtype=dtype, device=val.device)
    if len(xshape) > 2:
        x = x.reshape(xshape[0], xshape[1], -1)
    if idx.dtype == torch.uint8:
        idx = unpack12(idx, val.shape)
    x.scatter_reduce_(dim=-1, index=idx, src=val.to(dtype), reduce="mean", include_self=False)
    return x.reshape(xshape)


def batch_decompress(idxs, vals, xshape, totalk: int, *, block_norms=None, normalise=False, clip_norm=True):
    norms = clip = None
    if clip_norm:
        norms = block_norms if block_norms is not None else torch.stack([torch.norm(v, p=2) for v in vals])
        clip = torch.median(norms)
    done = []
    for i, v in enumerate(vals):
        if normalise:
            v = v / (torch.norm(v, p=2, dim=-1, keepdim=True) + 1e-8)
        elif clip_norm:
            v = v * torch.clamp(clip / (norms[i] + 1e-8), max=1)
        done.append(v)
    unpacked = [unpack12(i, v.shape) for i, v in zip(idxs, vals)]
    return decompress(torch.cat(unpacked, dim=-1), torch.cat(done, dim=-1), xshape, totalk)


# ---- the statistical quantiser (:582-644) ----------------------------------------------------
def quantize(val: torch.Tensor, n_bins: int = 256, range_in_sigmas: float = 6.0):
    """TopKCompressor._quantize_values op for op: codes (uint8) and (shift, scale, offset, lookup, dtype)."""
    offset = n_bins // 2                                                    # :593
    shift = val.mean()                                                      # :594
    centered = val - shift                                                  # :595
    std = centered.norm() / math.sqrt(centered.numel() - 1)                 # :597
    scale = range_in_sigmas * std / n_bins                                  # :598
    if scale == 0 or torch.isnan(scale) or torch.isinf(scale):              # :599-600
        scale = torch.tensor(1.0, dtype=centered.dtype, device=val.device)
    centered_fp32 = centered.to(torch.float32)                              # :602
    qval = (centered_fp32 / scale + offset).round().clamp(0, n_bins - 1).to(torch.uint8)   # :603-608
    sums = torch.zeros(n_bins, dtype=torch.float32, device=qval.device)
    counts = torch.zeros(n_bins, dtype=torch.float32, device=qval.device)
    sums.scatter_add_(0, qval.flatten().long(), centered_fp32.flatten())    # :614
    counts.scatter_add_(0, qval.flatten().long(), torch.ones_like(centered_fp32.flatten()))  # :615-617
    lookup = torch.where(counts > 0, sums / counts, torch.zeros_like(sums))  # :619
    return qval, (shift, float(scale), offset, lookup, val.dtype)           # :620-621


def dequantize(qval: torch.Tensor, qparams) -> torch.Tensor:
    """TopKCompressor._dequantize_values (:637-643)."""
    shift, _, _, lookup, orig_dtype = qparams
    return (lookup.to(qval.device)[qval.long()] + shift).to(orig_dtype)

