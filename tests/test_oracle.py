"""Pins the CPU oracle (oracle/tplr_oracle.c) before anything is compared against it.

Sources of truth, none of which is the oracle's own formula retyped:
  * the reference's inline known-answer vectors (tests/unit/test_compress.py:292-419,
    tests/test_comms.py:1828-2004), transcribed as data in tests/golden/reference_kats.json;
  * library routines: scipy.fft.dctn, torch.topk, Tensor.scatter_reduce_, torch.median;
  * brute force on small inputs and algebraic invariants.
"""
import json
import os

import numpy as np
import pytest
import scipy.fft
import torch

from oracle import codec as orc
from oracle import torch_cpu_path as tcp

GOLD = os.path.join(os.path.dirname(__file__), "golden")
KATS = json.load(open(os.path.join(GOLD, "reference_kats.json")))


# ---------------------------------------------------------------- pack / unpack
@pytest.mark.parametrize("case", KATS["pack_roundtrip"], ids=lambda c: c["name"])
def test_pack_reference_vectors(case):
    idx = np.array(case["indices"], dtype=np.int64)
    packed = orc.pack12(idx)
    assert packed.dtype == np.uint8 and packed.size == case["packed_len"]
    if "packed" in case:
        assert packed.tolist() == case["packed"]
    back = orc.unpack12(packed, idx.shape)
    assert back.dtype == np.int64 and np.array_equal(back, idx)


def test_pack_seed42_vector():
    # tests/unit/test_compress.py:381-392
    torch.manual_seed(42)
    idx = torch.randint(0, 4096, (100,), dtype=torch.int64).numpy()
    packed = orc.pack12(idx)
    assert packed.size == 150
    assert np.array_equal(orc.unpack12(packed, (100,)), idx)


def test_pack_bit_model_exhaustive_pairs():
    # every byte of the format checked against integer arithmetic on a 4096 x 64 sweep of pairs
    a = np.repeat(np.arange(4096, dtype=np.int64), 64)
    b = np.tile(np.arange(0, 4096, 64, dtype=np.int64) + 37 % 64, 4096)
    idx = np.stack([a, b], axis=1).reshape(-1)
    packed = orc.pack12(idx).reshape(-1, 3).astype(np.int64)
    word = a | (b << 12)
    assert np.array_equal(packed[:, 0], word & 0xFF)
    assert np.array_equal(packed[:, 1], (word >> 8) & 0xFF)
    assert np.array_equal(packed[:, 2], (word >> 16) & 0xFF)


def test_pack_errors():
    with pytest.raises(ValueError, match="Number of indices must be even"):
        orc.pack12([1, 2, 3])
    with pytest.raises(ValueError, match="exceeds 12-bit limit"):
        orc.pack12([0, 4096])
    with pytest.raises(ValueError, match="Number of indices must be even"):
        orc.unpack12(np.zeros(6, np.uint8), (3,))
    assert orc.pack12([]).size == 0
    assert orc.unpack12(np.zeros(0, np.uint8), (0,)).size == 0


def test_pack_matches_torch_op_sequence():
    rng = np.random.default_rng(1)
    idx = rng.integers(0, 4096, size=(7, 5, 32), dtype=np.int64)
    ref = tcp.pack12(torch.from_numpy(idx)).numpy()
    assert np.array_equal(orc.pack12(idx), ref)
    assert np.array_equal(orc.unpack12(ref, idx.shape), tcp.unpack12(torch.from_numpy(ref), idx.shape).numpy())


# ---------------------------------------------------------------- divisor rule
@pytest.mark.parametrize("n,c,want", [tuple(x) for x in KATS["smaller_split"]])
def test_smaller_split_reference_vectors(n, c, want):
    assert orc.smaller_split(n, c) == want


def test_smaller_split_brute_force():
    for n in list(range(1, 400)) + [768, 2048, 3072, 8192, 29568, 32000]:
        divs = [d for d in range(1, n + 1) if n % d == 0]
        assert orc.divisors(n) == divs
        for c in (1, 2, 7, 16, 64, 100, 5000):
            le = [d for d in divs if d <= c]
            want = max(le) if le else divs[0]
            if all(d < c for d in divs):
                want = n
            assert orc.smaller_split(n, c) == want, (n, c)


# ---------------------------------------------------------------- DCT
@pytest.mark.parametrize("n", [4, 8, 10, 16, 64])
def test_basis_is_the_orthonormal_dct(n):
    f = orc.dct_basis(n)
    assert np.allclose(f.T @ f, np.eye(n), atol=1e-13)
    want = scipy.fft.dct(np.eye(n), type=2, norm="ortho", axis=1)  # row i = DCT of e_i -> F[i, k]
    assert np.abs(f - want).max() < 1e-14
    # the reference builds the same matrix through an FFT in fp32
    f32, b32 = tcp.basis(n)
    assert np.abs(f32.numpy() - f).max() < 5e-7
    assert np.abs(b32.numpy() - f.T).max() < 5e-7


def test_encode_decode_against_scipy():
    rng = np.random.default_rng(2)
    x = (rng.standard_t(3, size=(128, 192)) * 1e-3).astype(np.float32)
    coef = orc.encode2d(x)
    assert coef.shape == (2, 3, 64, 64)
    blocks = x.reshape(2, 64, 3, 64).transpose(0, 2, 1, 3).astype(np.float64)
    want = scipy.fft.dctn(blocks, type=2, norm="ortho", axes=(2, 3))
    assert np.abs(coef - want).max() <= 1e-7 * np.abs(want).max()
    back = orc.decode2d(coef)
    assert np.abs(back - x).max() <= 2e-7 * np.abs(x).max()
    # Parseval per chunk
    assert np.allclose((coef.astype(np.float64) ** 2).sum((2, 3)), (blocks ** 2).sum((2, 3)), rtol=1e-6)
    # no-DCT path is a pure re-layout
    plain = orc.encode2d(x, use_dct=False)
    assert np.array_equal(plain, blocks.astype(np.float32))
    assert np.array_equal(orc.decode2d(plain, use_dct=False), x)


def test_encode_matches_reference_einsum_within_tolerance():
    rng = np.random.default_rng(3)
    x = (rng.standard_t(3, size=(128, 128)) * 1e-3).astype(np.float32)
    f, b = tcp.basis(64)
    ref = tcp.encode(torch.from_numpy(x), 64, 64, f, f).numpy()
    mine = orc.encode2d(x)
    assert np.abs(ref - mine).max() <= 1e-5 * np.abs(mine).max()
    back_ref = tcp.decode(torch.from_numpy(ref), b, b).numpy()
    assert np.abs(back_ref - orc.decode2d(mine)).max() <= 1e-5 * np.abs(x).max()


def test_dct_special_inputs():
    x = np.zeros((64, 64), np.float32)
    x[:] = 3.0
    c = orc.encode2d(x)[0, 0]
    assert abs(c[0, 0] - 3.0 * 64) < 1e-4 and np.abs(c).sum() - abs(c[0, 0]) < 1e-3  # DC only
    i = np.arange(64)
    x = np.cos(np.pi * (2 * i + 1) * 5 / 128)[:, None] * np.ones(64)[None, :]
    c = orc.encode2d(x.astype(np.float32))[0, 0]
    assert np.unravel_index(np.abs(c).argmax(), c.shape) == (5, 0)  # rows carry frequency 5
    # small / odd chunk sizes and the 1-D form
    rng = np.random.default_rng(4)
    y = rng.standard_normal((4, 8)).astype(np.float32)
    got = orc.dct1d(y)
    assert np.allclose(got, scipy.fft.dct(y.astype(np.float64), type=2, norm="ortho", axis=1), atol=1e-6)
    assert np.allclose(orc.dct1d(got, inverse=True), y, atol=1e-6)  # tests/unit/test_compress.py:281-290
    z = rng.standard_normal((20, 30)).astype(np.float32)
    cz = orc.encode2d(z, h=10, w=15)
    want = scipy.fft.dctn(z.reshape(2, 10, 2, 15).transpose(0, 2, 1, 3).astype(np.float64), norm="ortho", axes=(2, 3))
    assert np.allclose(cz, want, atol=1e-6)


def test_chunk_layout_by_spikes():
    x = np.zeros((128, 192), np.float32)
    spots = [(0, 0), (63, 63), (64, 0), (70, 130), (127, 191)]
    for n, (r, c) in enumerate(spots):
        x[r, c] = n + 1.0
    chunks = orc.encode2d(x, use_dct=False)
    for n, (r, c) in enumerate(spots):
        assert chunks[r // 64, c // 64].reshape(-1)[(r % 64) * 64 + (c % 64)] == n + 1.0


# ---------------------------------------------------------------- top-k
def test_clamp_topk_closed_form():
    for last in (1, 2, 3, 10, 64, 100, 4096):
        for k in (0, 1, 2, 3, 31, 32, 33, 64, 5000):
            want = max(min(k, last), 2)
            want -= want % 2
            assert orc.clamp_topk(last, k) == want


@pytest.mark.parametrize("n,k", [(4096, 32), (4096, 64), (4096, 2), (64, 32), (100, 10), (37, 6)])
def test_topk_brute_force_and_torch(n, k):
    rng = np.random.default_rng(n + k)
    x = (rng.standard_t(3, size=(9, n)) * 1e-3).astype(np.float32)
    idx, val = orc.topk_rows(x, k)
    for r in range(x.shape[0]):
        order = sorted(range(n), key=lambda i: (-abs(float(x[r, i])), i))[:k]
        assert idx[r].tolist() == order
        assert np.array_equal(val[r], x[r, order])
    t = torch.topk(torch.from_numpy(x).abs(), k, dim=-1, largest=True, sorted=False).indices.numpy()
    assert np.array_equal(np.sort(t, axis=1), np.sort(idx, axis=1))
    if k * 64 <= n:  # torch's partial-sort branch: already descending
        assert np.array_equal(t, idx)


def test_topk_ties_nan_zero():
    x = np.zeros((1, 4096), np.float32)
    idx, val = orc.topk_rows(x, 32)
    assert idx[0].tolist() == list(range(32)) and not val.any()
    x[0, [5, 900, 17]] = [2.0, -2.0, 2.0]
    x[0, 100] = np.nan
    x[0, 4000] = -np.inf
    x[0, 7] = -0.0
    idx, val = orc.topk_rows(x, 6)
    assert idx[0].tolist() == [100, 4000, 5, 17, 900, 0]
    assert np.isnan(val[0, 0]) and val[0, 1] == -np.inf and val[0, 4] == -2.0


def test_compress_round_trip_reference_case():
    # tests/unit/test_compress.py:127-158 (10x10 tensor, four spikes, top-4)
    x = np.zeros((10, 10), np.float32)
    for i in range(4):
        x[i, i] = i + 1.0
    idx, val, xshape, totalk = orc.compress(x, 4)
    assert idx.dtype == np.uint8 and val.shape == (10, 4) and totalk == 10 and xshape == (10, 10)
    out = orc.decompress(idx, val, xshape, totalk)
    top = np.sort(np.abs(out).reshape(-1))[::-1][:4]
    assert np.allclose(top, [4, 3, 2, 1], atol=1e-5)


# ---------------------------------------------------------------- scatter-mean / clip
def test_scatter_mean_semantics_hand_cases():
    # overlapping -> average of the contributions only; untouched -> 0 (include_self=False)
    idx = np.array([[1, 3, 1, 5, 1, 3]])
    val = np.array([[1, 2, 3, 4, 5, 6]], np.float32)
    assert orc.scatter_rows(idx, val, 8).tolist() == [[0, 3, 0, 4, 0, 4, 0, 0]]
    assert orc.scatter_rows(idx, val, 8, mean=False).tolist() == [[0, 9, 0, 8, 0, 4, 0, 0]]
    # fp32 sum runs in source order
    idx = np.array([[0, 0, 0]])
    assert orc.scatter_rows(idx, np.array([[1e8, 1.0, -1e8]], np.float32), 2)[0, 0] == 0.0
    assert orc.scatter_rows(idx, np.array([[1e8, -1e8, 1.0]], np.float32), 2)[0, 0] == np.float32(1.0) / np.float32(3.0)
    with pytest.raises(IndexError):
        orc.scatter_rows(np.array([[8, 0]]), np.zeros((1, 2), np.float32), 8)


def test_scatter_matches_torch_scatter_reduce():
    rng = np.random.default_rng(5)
    idx = rng.integers(0, 256, size=(6, 7, 96))
    val = rng.standard_normal((6, 7, 96)).astype(np.float32)
    want = torch.zeros(6, 7, 256).scatter_reduce_(-1, torch.from_numpy(idx), torch.from_numpy(val), reduce="mean",
                                                   include_self=False).numpy()
    assert np.array_equal(orc.scatter_rows(idx, val, 256), want)


def test_clip_scales_lower_median():
    for norms in ([3.0, 1.0, 2.0, 10.0], [5.0], [2.0, 8.0], [1.0, 1.0, 4.0, 0.0, 9.0]):
        med, scale = orc.clip_scales(norms)
        t = torch.tensor(norms)
        assert med == torch.median(t).item() == sorted(norms)[(len(norms) - 1) // 2]
        assert np.array_equal(scale, torch.clamp(torch.median(t) / (t + 1e-8), max=1).numpy())


@pytest.mark.parametrize("normalise,clip", [(False, True), (False, False), (True, True)])
def test_batch_decompress_matches_torch_op_sequence(normalise, clip):
    rng = np.random.default_rng(6)
    P, Y, X, k = 5, 2, 3, 32
    shared = rng.standard_normal((Y, X, 4096)).astype(np.float32)
    idxs, vals = [], []
    for p in range(P):
        g = (0.5 * shared + rng.standard_normal((Y, X, 4096)) * (1 + p)).astype(np.float32)
        i, v = orc.topk_rows(g, k)
        idxs.append(orc.pack12(i))
        vals.append(v)
    got = orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, normalise=normalise, clip_norm=clip)
    ref = tcp.batch_decompress([torch.from_numpy(i) for i in idxs], [torch.from_numpy(v) for v in vals],
                               (Y, X, 64, 64), 4096, normalise=normalise, clip_norm=clip).numpy()
    # norms are accumulated in double here and in float by torch: tolerance, not bits
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max()
    touched = ref != 0
    assert np.array_equal(got != 0, touched)
    # with block norms supplied the clip factors are identical and so is every bit
    norms = torch.stack([torch.norm(torch.from_numpy(v), p=2) for v in vals])
    if not normalise:
        got = orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, block_norms=norms.numpy(), clip_norm=clip)
        ref = tcp.batch_decompress([torch.from_numpy(i) for i in idxs], [torch.from_numpy(v) for v in vals],
                                   (Y, X, 64, 64), 4096, block_norms=norms, clip_norm=clip).numpy()
        assert np.array_equal(got, ref)


# ---------------------------------------------------------------- quantiser
def test_quantiser_closed_form():
    rng = np.random.default_rng(7)
    v = rng.standard_normal((4, 3, 32)).astype(np.float32)
    q, (shift, scale, offset, lookup) = orc.quantize(v, 256, 6)
    assert q.dtype == np.uint8 and offset == 128
    assert abs(shift - v.mean()) < 1e-6
    assert abs(scale - 6 * v.std(ddof=1) / 256) < 1e-6
    c = v - np.float32(shift)
    want_q = np.clip(np.rint(c / np.float32(scale) + 128), 0, 255).astype(np.uint8)
    assert np.array_equal(q, want_q)
    for b in np.unique(q):
        assert abs(lookup[b] - c[q == b].mean()) < 1e-6
    assert lookup[[b for b in range(256) if b not in set(np.unique(q))]].sum() == 0
    deq = orc.dequantize(q, (shift, scale, offset, lookup))
    assert np.abs(deq - v).max() <= scale  # within one bin
    # constant tensor: scale falls back to 1, dequantisation returns the constant
    cst = np.full((8,), 0.25, np.float32)
    q, qp = orc.quantize(cst, 4, 6)
    assert qp[1] == 1.0 and np.allclose(orc.dequantize(q, qp), cst)


def test_golden_fixture_is_reproduced():
    z = np.load(os.path.join(GOLD, "codec_small.npz"))
    coef = orc.encode2d(z["x"])
    assert np.array_equal(coef, z["coef"])
    idx, val, _, _ = orc.compress(coef, 32)
    assert np.array_equal(idx, z["idx12"]) and np.array_equal(val, z["val"])
    assert np.array_equal(orc.decode2d(orc.decompress(idx, val, coef.shape, 4096)), z["recon"])


# ---------------------------------------------------------------- index checks
def test_index_overlap_reference_known_answers():
    # the inline cases of the reference's tests/unit/test_idx_overlap.py:88-140:
    # identical rows -> 1.0, disjoint -> 0.0, two of four shared -> 0.5
    same = np.array([[0, 1, 2, 3]])
    inter, frac = orc.index_overlap([same, same])
    assert inter[0, 1] == 4 and frac[0, 1] == 1.0
    inter, frac = orc.index_overlap([np.array([[0, 1, 2, 3]]), np.array([[4, 5, 6, 7]])])
    assert inter[0, 1] == 0 and frac[0, 1] == 0.0
    inter, frac = orc.index_overlap([np.array([[0, 1, 2, 3]]), np.array([[2, 3, 4, 5]])])
    assert inter[0, 1] == 2 and frac[0, 1] == 0.5
    # against set intersection on random duplicate-free rows, three peers, several chunks
    rng = np.random.default_rng(5)
    rows = [np.stack([rng.permutation(256)[:16] for _ in range(7)]) for _ in range(3)]
    inter, frac = orc.index_overlap(rows)
    for i in range(3):
        for j in range(i + 1, 3):
            want = sum(len(set(rows[i][c]) & set(rows[j][c])) for c in range(7))
            assert inter[i, j] == want and abs(frac[i, j] - want / (7 * 16)) < 1e-6
    assert orc.index_bounds(np.array([0, 63]), 64) is None and orc.index_bounds(np.array([1, 64, 70]), 64) == 64

