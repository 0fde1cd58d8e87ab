"""Randomised properties of the oracle and of the library's host-memory routines (no GPU)."""
import ctypes as C
import os
import sys

import numpy as np
from hypothesis import given, settings
from hypothesis import strategies as st

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import codec as orc  # noqa: E402  (the checker)
from templar_amd import _lib  # noqa: E402


@settings(max_examples=60, deadline=None)
@given(st.lists(st.integers(0, 4095), min_size=0, max_size=200).filter(lambda v: len(v) % 2 == 0))
def test_host_pack_unpack_round_trip_and_oracle_bytes(values):
    lib = _lib.load()
    idx = np.asarray(values, dtype=np.int64)
    packed = np.zeros(idx.size * 3 // 2, dtype=np.uint8)
    bad = C.c_int64(-1)
    assert lib.tplr_pack12_host(idx.ctypes.data if idx.size else None, idx.size, packed.ctypes.data if idx.size else None,
                                C.byref(bad)) == 0
    if idx.size:
        assert bad.value == 0 and np.array_equal(packed, orc.pack12(idx))
        back = np.zeros_like(idx)
        assert lib.tplr_unpack12_host(packed.ctypes.data, idx.size, back.ctypes.data) == 0
        assert np.array_equal(back, idx) and np.array_equal(orc.unpack12(packed, idx.shape), idx)


@settings(max_examples=40, deadline=None)
@given(st.integers(0, 2**31 - 1), st.integers(1, 6), st.sampled_from([2, 4, 8, 16, 32]))
def test_scatter_mean_is_the_mean_over_the_peers_that_sent_a_coefficient(seed, peers, k):
    rng = np.random.default_rng(seed)
    rows = 3
    idx = [np.stack([rng.permutation(64)[:k] for _ in range(rows)]).astype(np.int64) for _ in range(peers)]
    val = [rng.standard_normal((rows, k)).astype(np.float32) for _ in range(peers)]
    dense = orc.batch_decompress([orc.pack12(i) for i in idx], val, (rows, 64), 64, clip_norm=False)
    acc = np.zeros((rows, 64), np.float64)
    cnt = np.zeros((rows, 64), np.int64)
    for i, v in zip(idx, val):
        for r in range(rows):
            acc[r, i[r]] += v[r]
            cnt[r, i[r]] += 1
    want = np.where(cnt > 0, acc / np.maximum(cnt, 1), 0.0)
    assert np.allclose(dense, want, rtol=1e-5, atol=1e-7) and np.array_equal(dense != 0, (cnt > 0) & (want != 0))


@settings(max_examples=25, deadline=None)
@given(st.integers(0, 2**31 - 1), st.sampled_from([4, 16, 256]))
def test_quantiser_invariants(seed, bins):
    rng = np.random.default_rng(seed)
    v = (rng.standard_normal((5, 32)) * rng.uniform(1e-4, 10) + rng.uniform(-1, 1)).astype(np.float32)
    q, (shift, scale, half, lut) = orc.quantize(v, bins, 6.0)
    assert q.min() >= 0 and q.max() < bins and half == bins // 2 and scale > 0
    centred = v - np.float32(shift)
    for b in np.unique(q):
        assert np.isclose(lut[b], centred[q == b].astype(np.float64).mean(), rtol=1e-5, atol=1e-9)
    back = orc.dequantize(q, (shift, scale, half, lut))
    # every value lands within one bin width of itself unless it was clamped at the ends
    inner = (q > 0) & (q < bins - 1)
    assert np.all(np.abs(back - v)[inner] <= scale * 1.0001)
    const = np.full((2, 8), 0.375, np.float32)
    qc, qpc = orc.quantize(const, bins, 6.0)
    assert qpc[1] == 1.0 and np.array_equal(orc.dequantize(qc, qpc), const)


@settings(max_examples=30, deadline=None)
@given(st.integers(0, 2**31 - 1), st.integers(2, 5), st.sampled_from([2, 8, 32]))
def test_index_overlap_counts_are_set_intersections(seed, peers, k):
    rng = np.random.default_rng(seed)
    rows = 4
    idx = [np.stack([rng.permutation(4096 if k > 8 else 24)[:k] for _ in range(rows)]) for _ in range(peers)]
    inter, frac = orc.index_overlap(idx)
    for i in range(peers):
        for j in range(i + 1, peers):
            want = sum(len(set(idx[i][r]) & set(idx[j][r])) for r in range(rows))
            assert inter[i, j] == want and np.isclose(frac[i, j], want / (rows * k))
