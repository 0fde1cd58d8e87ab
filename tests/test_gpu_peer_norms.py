"""The peers' norms kept as one float per payload row (tplr_row_sumsq, tplr_clip_scales_rows, PeerNorms):
the row figures against a numpy replay of their fixed addition order, the clip factors against the oracle's
(src/tplr/compress.py:526-556) and arrival-time figures against figures taken at aggregate time.  Needs an MI355X.
"""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import codec as orc  # noqa: E402  (the checker)
import templar_amd.compress as tc  # noqa: E402
from templar_amd import _lib  # noqa: E402
import workloads  # noqa: E402


def t3(shape, seed, row_scale=False):
    return workloads.student_t3(shape, seed, row_scale=row_scale)


def tree_rows(v: np.ndarray) -> np.ndarray:
    """Row sums of squares in the kernel's order: squares in the next power of two of lanes, lane j adds lane j ^ off."""
    n, k = v.shape
    w = 2
    while w < k and w < 64:
        w *= 2
    x = np.zeros((n, w), np.float32)
    if k <= 64:
        x[:, :k] = v * v
    else:  # lane j first adds the squares of values j, j + 64, ... with fused multiply-adds
        for j in range(64):
            acc = np.zeros(n, np.float64)
            for e in range(j, k, 64):
                acc = (v[:, e].astype(np.float64) * v[:, e].astype(np.float64) + acc).astype(np.float32).astype(np.float64)
            x[:, j] = acc.astype(np.float32)
    lanes = np.arange(w)
    off = w // 2
    while off:
        x = x + x[:, lanes ^ off]
        off //= 2
    return x[:, 0].copy()


@pytest.mark.parametrize("k", [1, 2, 6, 16, 32, 48, 64, 128, 200])
def test_row_sums_of_squares_in_their_fixed_order(dev, k):
    lib = _lib.load()
    P = 3
    for n in (1, 77, 1000, 4099):
        vals = [t3((n, k), 40 + 7 * p + k, row_scale=True).contiguous() for p in range(P)]
        d_vals = [v.to(dev) for v in vals]
        # (peer 1's values start four bytes off a 16-byte boundary: the kernel with 4-byte loads serves the launch)
        if n == 77:
            shifted = torch.empty(n * k + 1, device=dev)
            shifted[1:].copy_(d_vals[1].reshape(-1))
            d_vals[1] = shifted[1:].view(n, k)
            assert d_vals[1].data_ptr() % 16 == 4
        outs = [torch.full((n,), float("nan"), device=dev) for _ in range(P)]
        vp = (C.c_void_p * P)(*[v.data_ptr() for v in d_vals])
        op = (C.c_void_p * P)(*[o.data_ptr() for o in outs])
        assert lib.tplr_row_sumsq(vp, P, k, n, op, None) == 0
        torch.cuda.synchronize()
        for v, o in zip(vals, outs):
            got, want = o.cpu().numpy(), tree_rows(v.numpy())
            if k <= 64:
                assert np.array_equal(got, want), (k, n)
            else:  # the replay's multiply-add rounds twice where the hardware's rounds once
                assert np.allclose(got, want, rtol=3e-7, atol=0)
            exact = (v.numpy().astype(np.float64) ** 2).sum(1)
            assert np.allclose(got, exact, rtol=2e-6, atol=0)


def test_row_sums_argument_checks(dev):
    lib = _lib.load()
    v = torch.ones(64, device=dev)
    o = torch.empty(2, device=dev)
    vp, op = (C.c_void_p * 1)(v.data_ptr()), (C.c_void_p * 1)(o.data_ptr())
    none = (C.c_void_p * 1)(None)
    assert lib.tplr_row_sumsq(vp, 1, 0, 2, op, None) == _lib.TPLR_E_BADARG
    assert lib.tplr_row_sumsq(vp, 1, 4097, 2, op, None) == _lib.TPLR_E_BADARG
    assert lib.tplr_row_sumsq(none, 1, 32, 2, op, None) == _lib.TPLR_E_BADARG
    assert lib.tplr_row_sumsq(vp, 1, 32, 2, none, None) == _lib.TPLR_E_BADARG
    assert lib.tplr_row_sumsq(vp, 129, 32, 2, op, None) == _lib.TPLR_E_TOOMANY
    assert lib.tplr_row_sumsq(vp, 1, 32, 0, op, None) == 0
    assert lib.tplr_clip_scales_rows(op, 1, None, 1, 1, None, None, None, None) == _lib.TPLR_E_BADARG


def _window(dev, k, P):
    shapes2 = [(128, 192), (64, 64), (512, 1024), (2048, 2048), (64, 3072)]
    shapes1 = [(2048,), (64,), (8192,), (192,)]
    g2 = [t3(s, 700 + i, row_scale=True).to(dev) for i, s in enumerate(shapes2)]
    g1 = [t3(s, 800 + i).to(dev) for i, s in enumerate(shapes1)]
    b2, b1 = tc.TensorBatch(g2), tc.RowBatch(g1)
    pay2, pay1 = [], []
    for p in range(P):
        o2 = [0.5 * g + t3(tuple(g.shape), 9100 + 10 * p + i, row_scale=True).to(dev) * (1 + p) for i, g in enumerate(g2)]
        o1 = [0.5 * g + t3(tuple(g.shape), 9300 + 10 * p + i).to(dev) * (1 + p) for i, g in enumerate(g1)]
        pay2.append(tc.encode_compress_batch(tc.TensorBatch(o2), k))
        pay1.append(tc.encode_compress_rows_batch(tc.RowBatch(o1), k))
    return b2, b1, pay2, pay1


@pytest.mark.parametrize("k,P", [(32, 5), (64, 4), (16, 15), (32, 1)])
def test_clip_factors_from_row_figures(dev, k, P):
    b2, b1, pay2, pay1 = _window(dev, k, P)
    v2, v1 = [v for _, v in pay2], [v for _, v in pay1]
    norms = tc.PeerNorms([b2, b1], max_peers=P + 2)
    for p in range(P):  # as the payloads arrive, peer by peer, a part at a time
        norms.arrived(p, [v2[p], None])
        norms.arrived(p, [None, v1[p]])
    (s2, s1), (m2, m1) = norms.clip_scales(P, return_median=True)
    assert s2.shape == (len(b2), P) and s1.shape == (len(b1), P) and m2.shape == (len(b2),) and m1.shape == (len(b1),)
    # the same bits as the factors taken from the values at aggregate time
    f2, fm2 = tc.peer_clip_scales_batch(b2, v2, k, return_median=True)
    f1 = tc.peer_clip_scales_batch(b1, v1, k)
    assert torch.equal(s2, f2) and torch.equal(s1, f1) and torch.equal(m2, fm2)
    # and the oracle's factors on the norms taken in double
    for batch, vals, sc, med in ((b2, v2, s2, m2), (b1, v1, s1, m1)):
        for i in range(len(batch)):
            nr = np.array([np.sqrt((batch.payload_slice(i, pay2[0][0], vals[p], k)[1].double() ** 2).sum().item())
                           for p in range(P)], np.float32)
            want_med, want = orc.clip_scales(nr)
            assert np.allclose(sc[i].cpu().numpy(), want, rtol=2e-6)
            assert np.isclose(float(med[i]), float(want_med), rtol=2e-6)
    # a second, narrower window on the same object
    (t2, t1) = norms.clip_scales(max(1, P - 1))
    assert torch.equal(t2, tc.peer_clip_scales_batch(b2, v2[:max(1, P - 1)], k))
    # the aggregate with ready factors is the aggregate that takes its own
    outs_a = [torch.full_like(t, float("nan")) for t in b2.tensors]
    outs_b = [torch.full_like(t, float("nan")) for t in b2.tensors]
    (s2, s1) = norms.clip_scales(P)
    tc.batch_decompress_decode_batch(tc.TensorBatch(outs_a), [i for i, _ in pay2], v2, k, scale=s2)
    tc.batch_decompress_decode_batch(tc.TensorBatch(outs_b), [i for i, _ in pay2], v2, k, clip_norm=True)
    assert all(torch.equal(a, b) for a, b in zip(outs_a, outs_b))
    r_a = [torch.full_like(t, float("nan")) for t in b1.tensors]
    r_b = [torch.full_like(t, float("nan")) for t in b1.tensors]
    tc.batch_decompress_decode_rows_batch(tc.RowBatch(r_a), [i for i, _ in pay1], v1, min(k, 64), scale=s1)
    tc.batch_decompress_decode_rows_batch(tc.RowBatch(r_b), [i for i, _ in pay1], v1, min(k, 64))
    assert all(torch.equal(a, b) for a, b in zip(r_a, r_b))


def test_non_finite_values_reach_the_factors_as_in_torch(dev):
    # torch.median over norms with a NaN is NaN (every factor of that parameter NaN); an infinite norm gives factor 0
    k, P = 32, 4
    b2, _, pay2, _ = _window(dev, k, P)
    v2 = [v.clone() for _, v in pay2]
    v2[1][0, 3] = float("nan")                    # parameter 0, peer 1
    v2[2][b2.offsets[2] + 5, 0] = float("inf")    # parameter 2, peer 2
    sc = tc.peer_clip_scales_batch(b2, v2, k).cpu().numpy()
    assert np.isnan(sc[0]).all()
    assert sc[2][2] == 0.0 and np.isfinite(sc[2]).all()
    for i in range(len(b2)):
        nr = np.array([float(torch.linalg.vector_norm(b2.payload_slice(i, pay2[0][0], v2[p], k)[1].double()))
                       for p in range(P)], np.float32)
        _, want = orc.clip_scales(nr)
        assert np.allclose(sc[i], want, rtol=2e-6, equal_nan=True)


def test_staged_window_leaves_the_row_figures(dev):
    k, P = 32, 3
    b2, b1, pay2, pay1 = _window(dev, k, P)
    norms = tc.PeerNorms([b2, b1], max_peers=P)
    stage = tc.PayloadStage(b2, k, P, quantized=False, norms=norms)
    T = len(b2)
    sl = [[b2.payload_slice(i, pay2[p][0], pay2[p][1], k) for p in range(P)] for i in range(T)]
    for host in (False, True):
        norms.row_sumsq.fill_(float("nan"))
        idxs = [[(a.cpu() if host else a) for a, _ in row] for row in sl]
        vals = [[(v.cpu() if host else v) for _, v in row] for row in sl]
        si, sv = stage.load(idxs, vals)
        for p in range(P):
            norms.arrived(p, [None, pay1[p][1]])
        s2, s1 = norms.clip_scales(P)
        assert torch.equal(s2, tc.peer_clip_scales_batch(b2, [v for _, v in pay2], k))
        assert torch.equal(s1, tc.peer_clip_scales_batch(b1, [v for _, v in pay1], k))
    with pytest.raises(ValueError):
        tc.PayloadStage(b2, k, P, quantized=False, norms=tc.PeerNorms([b1, b2], max_peers=P))


def test_peer_norms_seeded_sweep(dev):
    # thirty draws of row counts, row lengths, peer counts and alignments: the row figures bit for bit against the
    # replay of their order, the factors against the oracle's on norms taken in double
    rng = np.random.default_rng(77)
    lib = _lib.load()
    for draw in range(30):
        k = int(rng.choice([2, 4, 6, 8, 12, 16, 24, 32, 40, 64]))
        P = int(rng.integers(1, 9))
        rows = [int(rng.integers(1, 40)) for _ in range(int(rng.integers(1, 6)))]
        n = sum(rows)
        off = int(rng.integers(0, 4))  # floats past a 16-byte boundary
        vals = [t3((n, k), 1000 * draw + p, row_scale=True) * float(10.0 ** rng.uniform(-6, 3)) for p in range(P)]
        bufs = [torch.empty(n * k + off, device=dev) for _ in range(P)]
        d_vals = []
        for b, v in zip(bufs, vals):
            b[off:].copy_(v.reshape(-1))
            d_vals.append(b[off:].view(n, k))
        outs = [torch.empty(n, device=dev) for _ in range(P)]
        vp = (C.c_void_p * P)(*[v.data_ptr() for v in d_vals])
        op = (C.c_void_p * P)(*[o.data_ptr() for o in outs])
        assert lib.tplr_row_sumsq(vp, P, k, n, op, None) == 0
        for v, o in zip(vals, outs):
            assert np.array_equal(o.cpu().numpy(), tree_rows(v.numpy())), (draw, k, off)
        # clip factors of a row list cut into `rows`
        import numpy as _np
        desc = _np.zeros(len(rows), dtype=_np.dtype([("dense", "<u8"), ("ld", "<i8"), ("chunk_begin", "<i8"),
                                                     ("x_chunks", "<i4"), ("y_chunks", "<i4")]))
        begin = 0
        for i, r in enumerate(rows):
            desc[i] = (0, 64, begin, r, 1)
            begin += r
        table = torch.from_numpy(desc.view(_np.uint8).copy()).to(dev)
        S = int(rng.integers(1, 5))
        partial = torch.empty(len(rows) * P * S, dtype=torch.float64, device=dev)
        scale = torch.empty((len(rows), P), device=dev)
        med = torch.empty(len(rows), device=dev)
        assert lib.tplr_clip_scales_rows(op, P, table.data_ptr(), len(rows), S, partial.data_ptr(), scale.data_ptr(),
                                         med.data_ptr(), None) == 0
        begin = 0
        for i, r in enumerate(rows):
            nr = np.array([np.sqrt((v.numpy()[begin:begin + r].astype(np.float64) ** 2).sum()) for v in vals], np.float32)
            want_med, want = orc.clip_scales(nr)
            assert np.allclose(scale[i].cpu().numpy(), want, rtol=3e-6), (draw, i)
            assert np.isclose(float(med[i]), want_med, rtol=3e-6)
            begin += r
