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


def _audit_codes(v, q_a, shift_a, scale_a, q_b, shift_b, scale_b, n_bins):
    """Two runs of the quantiser whose shift and scale differ in their last bits may code an entry
    differently only if it sits on a bin boundary to within what those differences move it."""
    diff = np.flatnonzero(q_a.reshape(-1) != q_b.reshape(-1))
    if diff.size == 0:
        return 0
    x = v.reshape(-1)[diff].astype(np.float64)
    t = (x - float(shift_a)) / float(scale_a) + n_bins // 2                       # position in bins
    slack = (abs(float(shift_a) - float(shift_b)) / float(scale_a)
             + np.abs(t) * abs(float(scale_a) - float(scale_b)) / float(scale_a)
             + 8 * np.finfo(np.float32).eps * (np.abs(t) + np.abs(x) / float(scale_a)))
    assert (np.abs(q_a.reshape(-1)[diff].astype(int) - q_b.reshape(-1)[diff].astype(int)) == 1).all()
    assert (np.abs(t - (np.floor(t) + 0.5)) <= slack).all(), (t, slack)
    return diff.size


@pytest.mark.parametrize("n_bins", [4, 256])
@pytest.mark.parametrize("kind", ["normal", "offset", "heavy"])
def test_quantiser_against_torch_op_sequence(n_bins, kind):
    # the reference's own torch ops (fp32 mean, norm / sqrt(n - 1), round, scatter_add_) against the oracle,
    # which carries its sums in double: shift and scale agree to rounding, codes agree except on audited
    # bin boundaries, the per-bin means to rounding
    rng = np.random.default_rng(11 + n_bins)
    v = {"normal": rng.standard_normal((37, 32)) * 0.02,
         "offset": rng.standard_normal((64, 32)) * 1e-3 + 1.0,
         "heavy": rng.standard_t(3, size=(50, 64)) * 1e-4}[kind].astype(np.float32)
    q_t, (shift_t, scale_t, off_t, lut_t, dt) = tcp.quantize(torch.from_numpy(v), n_bins, 6.0)
    q_o, (shift_o, scale_o, off_o, lut_o) = orc.quantize(v, n_bins, 6.0)
    assert off_t == off_o == n_bins // 2 and dt == torch.float32
    assert abs(float(shift_t) - shift_o) <= 4e-7 * max(abs(shift_o), np.abs(v).max() / np.sqrt(v.size))
    assert abs(scale_t - scale_o) <= 1e-6 * scale_o
    n_diff = _audit_codes(v, q_t.numpy(), float(shift_t), scale_t, q_o, shift_o, scale_o, n_bins)
    assert n_diff <= max(2, v.size // 100)
    used = np.unique(q_o)
    same = [b for b in used if (q_t.numpy() == b).sum() == (q_o == b).sum()]
    assert np.allclose(lut_t.numpy()[same], lut_o[same], rtol=1e-4, atol=1e-6 * np.abs(v).max())
    # de-quantisation: same table and codes in, same values out
    want = tcp.dequantize(torch.from_numpy(q_o), (torch.tensor(shift_o), scale_o, off_o, torch.from_numpy(lut_o), dt))
    assert np.array_equal(orc.dequantize(q_o, (shift_o, scale_o, off_o, lut_o)), want.numpy())


@pytest.mark.parametrize("n_bins", [4, 256])
def test_quantiser_ties_and_constants_equal_torch(n_bins):
    # exact halves: range 0 makes the scale fall back to exactly 1 (:599-600) and dyadic, symmetric values make
    # the mean exactly 0 in any summation order, so position = value + n_bins / 2 with ties at every x.5:
    # torch.round rounds them to even (:605), and so must the oracle - every code equal
    half = np.arange(-n_bins // 2 - 3, n_bins // 2 + 4, dtype=np.float32) + np.float32(0.5)
    v = np.concatenate([half, -half, np.array([0.0, 0.25, -0.25, 0.75, -0.75], np.float32)]).astype(np.float32)
    q_t, (shift_t, scale_t, _, lut_t, _) = tcp.quantize(torch.from_numpy(v), n_bins, 0.0)
    q_o, (shift_o, scale_o, _, lut_o) = orc.quantize(v, n_bins, 0.0)
    assert float(shift_t) == shift_o == 0.0 and scale_t == scale_o == 1.0
    assert np.array_equal(q_t.numpy(), q_o)
    assert np.array_equal(q_o, np.clip(np.rint(v + n_bins // 2), 0, n_bins - 1).astype(np.uint8))
    # n_bins / 2 is even: both neighbouring halves round to it
    assert q_o[np.flatnonzero(v == 0.5)[0]] == n_bins // 2 and q_o[np.flatnonzero(v == -0.5)[0]] == n_bins // 2
    assert np.allclose(lut_t.numpy(), lut_o, rtol=1e-6, atol=0)
    # a constant tensor: scale 1, every code n_bins / 2, de-quantised back to the constant
    cst = np.full((6, 32), 0.375, np.float32)
    q_t, (shift_t, scale_t, _, lut_t, _) = tcp.quantize(torch.from_numpy(cst), n_bins, 6.0)
    q_o, (shift_o, scale_o, _, lut_o) = orc.quantize(cst, n_bins, 6.0)
    assert float(shift_t) == shift_o == 0.375 and scale_t == scale_o == 1.0
    assert np.array_equal(q_t.numpy(), q_o) and (q_o == n_bins // 2).all()
    assert np.array_equal(orc.dequantize(q_o, (shift_o, scale_o, n_bins // 2, lut_o)), cst)


def test_clip_scales_with_non_finite_norms_match_torch():
    # torch.median gives NaN as soon as one norm is NaN (:535); an infinite norm is simply the largest
    for norms in ([1.0, float("nan")], [float("nan"), 1.0], [3.0, float("nan"), 1.0, 2.0], [float("inf"), 1.0, 2.0, 5.0],
                  [float("inf"), float("inf"), 1.0], [float("nan"), float("inf"), 2.0, 1.0, 4.0]):
        med, scale = orc.clip_scales(norms)
        t = torch.tensor(norms)
        want_med = torch.median(t)
        want = torch.clamp(want_med / (t + 1e-8), max=1).numpy()
        assert np.array_equal(np.float32(med), want_med.numpy(), equal_nan=True), norms
        assert np.array_equal(scale, want, equal_nan=True), norms


def test_aggregate_mean_normalised_is_the_normalised_mean_of_the_peers_reconstructions():
    # the benchmark's wording of the aggregation: linear in the peers, so it equals the mean of the one-peer
    # reconstructions (each built here with torch's scatter_add_ and scipy's inverse DCT), divided by its norm
    rng = np.random.default_rng(21)
    P, Y, X, k = 5, 2, 3, 32
    idxs, vals = [], []
    for p in range(P):
        i, v = orc.topk_rows(rng.standard_normal((Y, X, 4096)).astype(np.float32), k)
        idxs.append(i)
        vals.append(v)
    got = orc.aggregate_mean_normalised([orc.pack12(i) for i in idxs], vals, (Y, X, 64, 64), 4096)
    acc = np.zeros((Y * 64, X * 64))
    for i, v in zip(idxs, vals):
        dense = torch.zeros(Y * X, 4096, dtype=torch.float64)
        dense.scatter_add_(1, torch.from_numpy(i.reshape(Y * X, k).astype(np.int64)),
                           torch.from_numpy(v.reshape(Y * X, k).astype(np.float64)))
        chunks = scipy.fft.idctn(dense.numpy().reshape(Y, X, 64, 64), type=2, norm="ortho", axes=(2, 3))
        acc += chunks.transpose(0, 2, 1, 3).reshape(Y * 64, X * 64)
    want = acc / P
    want = want / np.sqrt((want ** 2).sum())
    assert got.dtype == np.float32 and got.shape == (Y * 64, X * 64)
    assert abs(float(np.sqrt((got.astype(np.float64) ** 2).sum())) - 1.0) <= 1e-6
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()


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



# ---------------------------------------------------------------- miner step (src/tplr/neurons.py:147-171)
@pytest.mark.parametrize("use_dct", [True, False])
@pytest.mark.parametrize("bins", [0, 4, 256])
@pytest.mark.parametrize("null_round", [False, True])
def test_error_feedback_step_against_the_torch_op_sequence(use_dct, bins, null_round):
    # orc.error_feedback_step against the reference's own order of operations replayed with torch on the CPU
    # (oracle/torch_cpu_path.py holds its compress.py halves; the neurons.py lines are written out here):
    # :148-152 zero or decay-and-add, :155 encode, :157-159 compress (+ quantise), :164-166 decompress
    # (+ de-quantise), :169 decode, :171 subtract
    torch.manual_seed(7)
    R, Cc, k, decay = 128, 192, 32, 0.95
    ef0 = torch.randn(R, Cc) * 1e-3
    grad = torch.distributions.StudentT(3.0).sample((R, Cc)) * 1e-3
    b64 = tcp.basis(64)
    ef = ef0.clone()
    if null_round:
        ef.zero_()
    else:
        ef.mul_(decay)
        ef.add_(grad)
    enc = tcp.encode(ef, 64, 64, b64[0], b64[0], use_dct=use_dct)
    idx12, val, xshape, totalk = tcp.compress(enc, k)
    sent = val
    if bins:
        q, qp = tcp.quantize(val, bins, 6.0)
        sent = tcp.dequantize(q, qp)
    new = ef - tcp.decode(tcp.decompress(idx12, sent, xshape, totalk), b64[1], b64[1], use_dct=use_dct)

    got_acc, got_idx, got_val, got_new = orc.error_feedback_step(ef0.numpy(), grad.numpy(), decay, k, use_dct=use_dct,
                                                                 quant_bins=bins, null_round=null_round)
    assert np.array_equal(got_acc, ef.numpy())        # two roundings, as mul_ then add_; zeros on a null round
    if null_round:
        # nothing to select from: every chunk sends zeros and the error feedback stays zero
        assert not got_val.any() and not got_new.any() and not new.any()
        return
    scale = float(ef.abs().max())
    if use_dct:
        # with the oracle's own transform the selections are made on coefficients that differ from torch's in
        # their last bits: the sent sets agree wherever the k-th and (k+1)-th magnitudes are further apart
        want_idx = tcp.unpack12(idx12, val.shape).numpy().reshape(-1, k)
        mine = orc.unpack12(got_idx, (want_idx.shape[0], k))
        assert np.mean([set(a) == set(b) for a, b in zip(want_idx.tolist(), mine.tolist())]) > 0.9
        # on torch's coefficients (identical inputs to the selection) everything downstream is pinned: the same
        # bytes and values, and the same remainder to fp32 tolerance
        _, got_idx, got_val, got_new = orc.error_feedback_step(ef0.numpy(), grad.numpy(), decay, k, use_dct=True,
                                                               quant_bins=bins, coef_override=enc.numpy())
        tol = 1e-5
    else:
        tol = 1e-6  # no transform: only the subtraction rounds
    assert np.array_equal(got_idx, idx12.numpy()) and np.array_equal(got_val.reshape(-1), val.numpy().reshape(-1))
    assert np.abs(got_new - new.numpy()).max() <= tol * scale


def test_error_feedback_step_closed_form_against_scipy():
    # ef_new = ef_acc - IDCT(top-k(DCT(ef_acc))) with scipy's orthonormal transforms and a brute-force selection:
    # the remainder has nothing left at the sent coefficients and everything at the others
    rng = np.random.default_rng(3)
    ef0 = (rng.standard_normal((64, 128)) * 1e-3).astype(np.float32)
    grad = (rng.standard_t(3, (64, 128)) * 1e-3).astype(np.float32)
    decay, k = 0.9, 16
    acc, idx12, val, new = orc.error_feedback_step(ef0, grad, decay, k, use_dct=True)
    want_acc = (ef0 * np.float32(decay) + grad).astype(np.float32)
    assert np.array_equal(acc, want_acc)
    chunks = want_acc.astype(np.float64).reshape(1, 64, 2, 64).transpose(0, 2, 1, 3)
    coef = scipy.fft.dctn(chunks, axes=(-2, -1), norm="ortho").reshape(-1, 4096)
    keep = np.zeros_like(coef)
    order = np.argsort(-np.abs(coef), axis=1, kind="stable")[:, :k]
    np.put_along_axis(keep, order, np.take_along_axis(coef, order, 1), 1)
    recon = scipy.fft.idctn(keep.reshape(1, 2, 64, 64), axes=(-2, -1), norm="ortho")
    want_new = chunks - recon
    want_new = want_new.transpose(0, 2, 1, 3).reshape(64, 128)
    assert np.abs(new - want_new).max() <= 1e-5 * np.abs(want_acc).max()
    # what was sent: the k largest coefficients of each chunk, by index set and by value
    mine = orc.unpack12(idx12, (2, k))
    assert all(set(a) == set(b) for a, b in zip(mine.tolist(), order.tolist()))
    assert np.allclose(np.sort(val.reshape(2, k), 1), np.sort(np.take_along_axis(coef, order, 1), 1), atol=1e-5 * np.abs(coef).max())
    # the remainder's own transform is zero at the sent coefficients
    left = scipy.fft.dctn(new.astype(np.float64).reshape(1, 64, 2, 64).transpose(0, 2, 1, 3), axes=(-2, -1), norm="ortho").reshape(-1, 4096)
    assert np.abs(np.take_along_axis(left, order, 1)).max() <= 2e-5 * np.abs(coef).max()


# ---------------------------------------------------------------- outer step (src/tplr/neurons.py:341-447)
@pytest.mark.parametrize("use_dct", [True, False])
@pytest.mark.parametrize("poison", [None, "nan", "inf"])
def test_outer_step_against_torch_sgd_on_the_torch_op_sequence(use_dct, poison):
    # orc.outer_step against the reference's own lines replayed with torch on the CPU: block norms (:346),
    # batch_decompress with them (:355-365), decode (:367), norm and mean (:381-385), the isfinite gate (:438-442)
    # and torch.optim.SGD(lr).step() (:446; neurons/trainer.py:128-130)
    torch.manual_seed(11)
    R, Cc, k, P, lr = 128, 192, 32, 5, 0.4
    b64 = tcp.basis(64)
    pay = []
    for p in range(P):
        g = torch.distributions.StudentT(3.0).sample((R, Cc)) * 1e-3 * (1 + p)
        pay.append(tcp.compress(tcp.encode(g, 64, 64, b64[0], b64[0], use_dct=use_dct), k))
    idxs, vals = [a[0] for a in pay], [a[1].clone() for a in pay]
    xshape, totalk = pay[0][2], pay[0][3]
    if poison == "nan":
        vals[2][0, 1, 3] = float("nan")
    elif poison == "inf":
        vals[4][1, 0, 0] = float("inf")
    param = torch.nn.Parameter(torch.randn(R, Cc))
    before = param.detach().clone()
    opt = torch.optim.SGD([param], lr=lr)
    norms = torch.stack([torch.norm(v, p=2) for v in vals])
    grad = tcp.decode(tcp.batch_decompress(idxs, vals, xshape, totalk, block_norms=norms), b64[1], b64[1], use_dct=use_dct)
    want_norm, want_mean = torch.norm(grad, p=2).item(), grad.mean().item()
    applied = bool(torch.isfinite(grad).all())
    if applied:
        param.grad = grad
        opt.step()
    got, g_norm, g_mean, got_applied = orc.outer_step(before.numpy(), [i.numpy() for i in idxs], [v.numpy() for v in vals],
                                                      tuple(xshape), totalk, lr, use_dct=use_dct)
    assert got_applied == applied == (poison is None)
    if not applied:
        assert np.array_equal(got, before.numpy())      # the parameter keeps its bits
        assert not np.isfinite(g_norm) or np.isnan(g_norm)
        return
    assert np.abs(got - param.detach().numpy()).max() <= 1e-6 * float(before.abs().max())
    assert np.isclose(g_norm, want_norm, rtol=1e-5) and np.isclose(g_mean, want_mean, rtol=1e-3, atol=1e-9)
    # the step really is p - lr * grad: undoing it with the gradient returns the parameter
    assert np.abs(got + np.float32(lr) * grad.numpy() - before.numpy()).max() <= 1e-6 * float(before.abs().max())
