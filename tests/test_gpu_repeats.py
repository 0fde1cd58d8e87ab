"""Payloads with repeated indices inside one peer's row, through every aggregate entry point.

A top-k selection never repeats an index, but payloads come from other machines and nothing
upstream rejects repeats (src/tplr/comms.py:2538-2610 checks dtype, count and bounds only).  The
reference adds every entry and divides by the number of entries (scatter_reduce "mean" on the
concatenation, src/tplr/compress.py:472-474, 574-580).  The oracle does exactly that; the device
must agree: sums and means bit for bit where no transform follows, within 1e-5 after the
inverse DCT, neighbours of a repeated coefficient untouched.
"""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import codec as orc  # noqa: E402  (the checker)
import templar_amd.compress as tc  # noqa: E402
from templar_amd import _lib  # noqa: E402

TOL = 1e-5


def relerr(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def peers_with_repeats(P, Y, X, k, seed, every=1):
    """P peers' (indices (Y*X, k) int64, values (Y*X, k) fp32): top-k selections of correlated
    noise, then repeats planted in every `every`-th row."""
    rng = np.random.default_rng(seed)
    n = Y * X
    shared = rng.standard_normal((n, 4096)).astype(np.float32)
    idxs, vals = [], []
    for p in range(P):
        g = (0.5 * shared + rng.standard_normal((n, 4096)) * (1 + 0.3 * p)).astype(np.float32) * 1e-3
        i, v = orc.topk_rows(g, k)
        idxs.append(i.astype(np.int64).copy())
        vals.append(v.copy())
    for r in range(0, n, every):
        kind = (r // every) % 4
        if k < 8:
            kind = 1 if kind < 2 else 3
        if kind == 0:
            # every peer sends coefficient 777 (once), one peer sends it twice: P + 1 entries on one coefficient;
            # its neighbours 776 and 778 are sent once each by two other peers
            for p in range(P):
                row = idxs[p][r]
                if 777 not in row:
                    row[0] = 777
            row = idxs[3 % P][r]
            row[int(np.flatnonzero(row != 777)[0])] = 777
            for nb, p in ((776, 0), (778, P - 1)):
                row = idxs[p][r]
                if nb not in row:
                    row[int(np.flatnonzero((row != 777) & (row != 776) & (row != 778))[-1])] = nb
        elif kind == 1:
            idxs[0][r][:] = 1234  # k copies of one index from one peer
        elif kind == 2:
            # two different repeated pairs in one peer, a triple in another, the same coefficient in both
            a = idxs[2 % P][r]
            a[1] = a[0]
            a[5] = a[4]
            b = idxs[(P - 1) // 2][r]
            b[2] = b[3] = b[7] = a[0]
        else:
            # a repeat of the last entry at the first position (the two ends of a wave instruction)
            a = idxs[r % P][r]
            a[0] = a[k - 1]
    return idxs, vals


def on_device(idxs, vals, dev):
    di = [torch.from_numpy(orc.pack12(i)).to(dev) for i in idxs]
    dv = [torch.from_numpy(v).to(dev) for v in vals]
    return di, dv


# (peers, k): the 8-, 16- and 24-unit register paths, 4- and 5-bit counters, the generic path (many peers, long rows)
CASES = [(1, 32), (2, 2), (8, 32), (15, 32), (15, 64), (20, 64), (24, 32), (31, 16), (5, 128), (40, 64)]


@pytest.mark.parametrize("P,k", CASES)
def test_batch_decompress_with_repeats_bit_exact(dev, P, k):
    Y, X = 2, 4
    idxs, vals = peers_with_repeats(P, Y, X, k, 1000 + 7 * P + k)
    norms = np.array([orc.norm2(v) for v in vals], np.float32)
    packed = [orc.pack12(i) for i in idxs]
    want = orc.batch_decompress(packed, vals, (Y, X, 64, 64), 4096, block_norms=norms)
    # the repeated coefficient of row 0 really holds P + 1 entries, and its neighbours one each
    cat = np.concatenate([i[0] for i in idxs])
    assert k < 8 or (cat == 777).sum() == P + 1
    di, dv = on_device(idxs, vals, dev)
    got = tc.TopKCompressor().batch_decompress(torch.empty(Y * 64, X * 64, device=dev), di, dv, (Y, X, 64, 64), 4096,
                                               block_norms=torch.from_numpy(norms).to(dev))
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # plain sums, no clip factors
    want_sum = orc.batch_decompress(packed, vals, (Y, X, 64, 64), 4096, clip_norm=False, mean=False)
    got_sum = tc._aggregate_chunks(di, dv, None, Y, X, k, normalise=False, use_dct=False, mean=False)
    assert np.array_equal(got_sum.cpu().numpy().view(np.uint32), want_sum.view(np.uint32))
    # the (R, C) layout of decode(use_dct=False)
    got_rows = tc._aggregate_chunks(di, dv, None, Y, X, k, normalise=False, use_dct=False, mean=False, rows=True)
    assert np.array_equal(got_rows.cpu().numpy(), orc.decode2d(want_sum, use_dct=False))


@pytest.mark.parametrize("P,k", CASES)
def test_batch_decompress_decode_with_repeats(dev, P, k):
    Y, X = 3, 2
    idxs, vals = peers_with_repeats(P, Y, X, k, 2000 + 7 * P + k)
    norms = np.array([orc.norm2(v) for v in vals], np.float32)
    dense = orc.batch_decompress([orc.pack12(i) for i in idxs], vals, (Y, X, 64, 64), 4096, block_norms=norms)
    want = orc.decode2d(dense)
    di, dv = on_device(idxs, vals, dev)
    ss = torch.zeros(Y * X, device=dev)
    got = tc.batch_decompress_decode(di, dv, (Y, X, 64, 64), block_norms=torch.from_numpy(norms).to(dev), sumsq=ss)
    assert relerr(got.cpu().numpy(), want) <= TOL
    per_chunk = (want.reshape(Y, 64, X, 64).astype(np.float64) ** 2).sum((1, 3)).reshape(-1)
    assert np.allclose(ss.cpu().numpy(), per_chunk, rtol=1e-4)


def test_normalised_aggregate_with_repeats(dev):
    P, k, Y, X = 4, 32, 2, 2
    idxs, vals = peers_with_repeats(P, Y, X, k, 31)
    want = orc.batch_decompress([orc.pack12(i) for i in idxs], vals, (Y, X, 64, 64), 4096, normalise=True)
    di, dv = on_device(idxs, vals, dev)
    got = tc.TopKCompressor().batch_decompress(torch.empty(1, device=dev), di, dv, (Y, X, 64, 64), 4096, normalise=True)
    assert relerr(got.cpu().numpy(), want) <= 1e-6
    assert np.array_equal(got.cpu().numpy() != 0, want != 0)


def staged(di, dv):
    """The same payloads equally spaced in one buffer (a staged window): the kernels then address the peers
    with scalar arithmetic, a code path of its own."""
    P = len(di)
    ib = torch.empty((P, di[0].numel() + 64), dtype=torch.uint8, device=di[0].device)
    vb = torch.empty((P, dv[0].numel() + 16), dtype=torch.float32, device=dv[0].device)
    out_i, out_v = [], []
    for p in range(P):
        ib[p, :di[p].numel()] = di[p]
        vb[p, :dv[p].numel()] = dv[p].reshape(-1)
        out_i.append(ib[p, :di[p].numel()])
        out_v.append(vb[p, :dv[p].numel()].view(dv[p].shape))
    return out_i, out_v


@pytest.mark.parametrize("P,k", [(1, 32), (8, 32), (15, 32), (15, 64), (20, 64), (24, 32)])
@pytest.mark.parametrize("use_dct", [True, False])
def test_staged_window_gives_the_same_bits_as_separate_payloads(dev, P, k, use_dct):
    Y, X = 5, 7
    idxs, vals = peers_with_repeats(P, Y, X, k, 4000 + P + k, every=6)
    di, dv = on_device(idxs, vals, dev)
    si, sv = staged(di, dv)
    assert all(b.data_ptr() - a.data_ptr() == si[1].data_ptr() - si[0].data_ptr() for a, b in zip(si, si[1:])) or P == 1
    scale = torch.from_numpy((np.random.default_rng(9).random(P) * 0.5 + 0.5).astype(np.float32)).to(dev)
    want = tc._aggregate_chunks(di, dv, scale, Y, X, k, normalise=False, use_dct=use_dct, rows=True)
    got = tc._aggregate_chunks(si, sv, scale, Y, X, k, normalise=False, use_dct=use_dct, rows=True)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


@pytest.mark.parametrize("P,k,use_dct,window", [(15, 32, True, False), (15, 32, True, True), (15, 32, False, False),
                                                (15, 32, False, True), (20, 64, True, True), (31, 32, True, False)])
def test_whole_set_aggregate_with_repeats_in_some_rows(dev, P, k, use_dct, window):
    # enough chunks that every wave walks several, a repeat planted in every 5th row: marked rows in the
    # middle of a wave's range, at its first and at its last chunk; the other rows go the fast way
    shapes = [(64 * 70, 64 * 48), (64 * 33, 64 * 64), (64, 64), (64 * 50, 64 * 40)]
    counts = [(s[0] // 64) * (s[1] // 64) for s in shapes]
    n = sum(counts)
    idxs, vals = peers_with_repeats(P, 1, n, k, 77 + P + k, every=5)
    di, dv = on_device(idxs, vals, dev)
    if window:
        di, dv = staged(di, dv)
    outs = [torch.full(s, 7.0, device=dev) for s in shapes]
    batch = tc.TensorBatch(outs)
    scale = torch.from_numpy((np.random.default_rng(3).random((len(shapes), P)) * 0.5 + 0.5).astype(np.float32)).to(dev)
    ss = torch.zeros(n, device=dev)
    tc.batch_decompress_decode_batch(batch, di, dv, k, scale=scale, use_dct=use_dct, sumsq=ss)
    b0 = 0
    sc = scale.cpu().numpy()
    for t, (s, cnt) in enumerate(zip(shapes, counts)):
        Y, X = s[0] // 64, s[1] // 64
        sl = slice(b0, b0 + cnt)
        # the oracle's scatter on the concatenation, every peer's values times its factor for this tensor
        # and the exact 2^-5 the device folds into it when a transform follows
        cat_i = np.concatenate([i[sl] for i in idxs], axis=1)
        cat_v = np.concatenate([v[sl] * (sc[t, p] * np.float32(1 / 32 if use_dct else 1)) for p, v in enumerate(vals)],
                               axis=1).astype(np.float32)
        dense = orc.scatter_rows(cat_i, cat_v, 4096, mean=True).reshape(Y, X, 64, 64)
        got = outs[t].cpu().numpy()
        if use_dct:
            want = orc.decode2d(dense * np.float32(32))
            assert relerr(got, want) <= TOL, t
        else:
            want = orc.decode2d(dense, use_dct=False)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), t
        per_chunk = (want.reshape(Y, 64, X, 64).astype(np.float64) ** 2).sum((1, 3)).reshape(-1)
        assert np.allclose(ss[sl].cpu().numpy(), per_chunk, rtol=1e-4), t
        b0 += cnt


@pytest.mark.parametrize("use_dct", [True, False])
def test_error_feedback_subtract_with_repeats(dev, use_dct):
    # tplr_ef_subtract_batch: ef <- ef - decode(decompress(payload)) (src/tplr/neurons.py:162-171) on a payload
    # whose rows repeat indices; the rows that do must not be subtracted twice
    lib = _lib.load()
    k = 32
    shapes = [(64 * 40, 64 * 60), (64 * 30, 64 * 30)]
    counts = [(s[0] // 64) * (s[1] // 64) for s in shapes]
    n = sum(counts)
    idxs, vals = peers_with_repeats(1, 1, n, k, 99, every=3)
    rng = np.random.default_rng(5)
    efs = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    d_ef = [torch.from_numpy(e).to(dev) for e in efs]
    batch = tc.TensorBatch(d_ef)
    di, dv = on_device(idxs, vals, dev)
    with tc._on(dev):
        st = lib.tplr_ef_subtract_batch(tc._ptr(di[0]), tc._ptr(dv[0]), k, tc._ptr(batch.table), len(batch), n,
                                        int(use_dct), tc._stream(dev))
    assert st == 0
    b0 = 0
    for t, (s, cnt) in enumerate(zip(shapes, counts)):
        Y, X = s[0] // 64, s[1] // 64
        dense = orc.scatter_rows(idxs[0][b0:b0 + cnt], vals[0][b0:b0 + cnt], 4096, mean=True).reshape(Y, X, 64, 64)
        want = efs[t] - orc.decode2d(dense, use_dct=use_dct)
        got = d_ef[t].cpu().numpy()
        if use_dct:
            assert np.abs(got - want).max() <= TOL * max(np.abs(want).max(), np.abs(orc.decode2d(dense)).max()), t
        else:
            assert np.array_equal(got, want), t
        b0 += cnt
