"""Synthetic gradient sets of the five benchmark configurations (shared by bench.py and the tests).

Value law: Student-t(df=3) built as z0 / sqrt((z1^2 + z2^2 + z3^2) / 3) from four
independent normal draws, times 1e-3; configs 2-5 multiply every row by exp(0.5 n_r),
n_r ~ N(0, 1).  Tensor j of a set uses seed S + j; peer p of the aggregation workload is
0.5 * shared + own with seeds 1000 (p + 1) + j.
"""
from __future__ import annotations

import torch


def llama_shapes(layers: int, hidden: int, inter: int, vocab: int) -> list[tuple[int, ...]]:
    shapes: list[tuple[int, ...]] = []
    for _ in range(layers):
        shapes += [(hidden, hidden)] * 4            # q, k, v, o
        shapes += [(inter, hidden)] * 2             # gate, up
        shapes += [(hidden, inter)]                 # down
        shapes += [(hidden,)] * 2                   # two norm gains
    shapes += [(vocab, hidden)] * 2                 # embed, lm_head
    shapes += [(hidden,)]                           # final norm
    return shapes


CONFIGS = {
    "cfg1_2048x2048": {"shapes": [(2048, 2048)], "k": 32, "row_scale": False, "seed": 0},
    "cfg2_llama150m": {"shapes": llama_shapes(12, 768, 3072, 32000), "k": 32, "row_scale": True, "seed": 100},
    "cfg3_llama1b": {"shapes": llama_shapes(16, 2048, 8192, 32000), "k": 32, "row_scale": True, "seed": 200},
    "cfg5_72b_block": {
        "shapes": [(8192, 8192)] * 2 + [(8192, 1024)] * 2 + [(8192, 29568)] * 2 + [(29568, 8192)],
        "k": 64, "row_scale": True, "seed": 300,
    },
}


def student_t3(shape, seed: int, *, row_scale: bool, device="cpu", scale: float = 1e-3) -> torch.Tensor:
    """Seeded heavy-tailed tensor; generated on `device` with that device's generator."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    z = torch.randn((4,) + tuple(shape), generator=g, device=device, dtype=torch.float32)
    t = z[0] / torch.sqrt((z[1] * z[1] + z[2] * z[2] + z[3] * z[3]) / 3.0)
    t = t * scale
    if row_scale and len(shape) == 2:
        r = torch.randn((shape[0], 1), generator=g, device=device, dtype=torch.float32)
        t = t * torch.exp(0.5 * r)
    return t


def gradient_set(name: str, device="cpu") -> list[torch.Tensor]:
    cfg = CONFIGS[name]
    return [student_t3(s, cfg["seed"] + j, row_scale=cfg["row_scale"], device=device)
            for j, s in enumerate(cfg["shapes"])]


def chunks_2d(shapes) -> int:
    return sum((s[0] // 64) * (s[1] // 64) for s in shapes if len(s) == 2)


def encode_bytes(shapes, k: int) -> int:
    """Algorithmic bytes of encode + top-k + pack: 16384 read + 5.5 k written per 2-D chunk;
    1-D tensors (64-element chunks): 256 read + 5.5 min(k, 64) written."""
    total = chunks_2d(shapes) * (16384 + 11 * k // 2)
    for s in shapes:
        if len(s) == 1:
            kk = min(k, 64)
            total += (s[0] // 64) * (256 + 11 * kk // 2)
    return total


def aggregate_bytes(shapes, k: int, peers: int) -> int:
    """Algorithmic bytes of P-peer decode-aggregate: P * 5.5 k read + 16384 written per chunk."""
    total = chunks_2d(shapes) * (peers * 11 * k // 2 + 16384)
    for s in shapes:
        if len(s) == 1:
            kk = min(k, 64)
            total += (s[0] // 64) * (peers * 11 * kk // 2 + 256)
    return total
