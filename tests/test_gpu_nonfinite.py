"""Non-finite norms and values on the receive side, and the quantiser, against the reference's own
torch op sequence (oracle/torch_cpu_path.py) run on the CPU.

torch.median gives NaN as soon as one norm is NaN and torch.clamp keeps NaN
(src/tplr/compress.py:535, :553-556), so a peer whose values hold a NaN turns every coefficient any
peer sent into NaN: visible, and the device must show the same.  An infinite norm is the largest
norm; its peer's factor is 0.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import codec as orc  # noqa: E402  (the checker)
from oracle import torch_cpu_path as tcp  # noqa: E402
import templar_amd.compress as tc  # noqa: E402


def make_peers(P, Y, X, k, seed):
    rng = np.random.default_rng(seed)
    shared = rng.standard_normal((Y, X, 4096)).astype(np.float32)
    idxs, vals = [], []
    for p in range(P):
        g = (0.5 * shared + rng.standard_normal((Y, X, 4096)) * (1 + 0.3 * p)).astype(np.float32) * 1e-3
        i, v = orc.topk_rows(g, k)
        idxs.append(orc.pack12(i))
        vals.append(v.copy())
    return idxs, vals


def same_with_nans(got, want, rtol=0.0):
    got, want = np.asarray(got), np.asarray(want)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    fin = ~np.isnan(want)
    if rtol == 0.0:
        assert np.array_equal(got[fin], want[fin])
    else:
        assert np.array_equal(np.isinf(got[fin]), np.isinf(want[fin]))
        ok = np.isfinite(want[fin])
        scale = np.abs(want[fin][ok]).max() if ok.any() else 1.0
        assert np.abs(got[fin][ok] - want[fin][ok]).max() <= rtol * scale


@pytest.mark.parametrize("norms", [[float("nan"), 1.0], [1.0, float("nan")], [3.0, 1.0, float("nan"), 2.0, 9.0],
                                   [float("inf"), 1.0, 2.0, 5.0], [2.0, float("inf"), float("inf")],
                                   [float("nan"), float("inf"), 2.0, 1.0, 4.0]])
def test_given_block_norms_with_nan_and_inf(dev, norms):
    P, k, Y, X = len(norms), 32, 2, 2
    idxs, vals = make_peers(P, Y, X, k, 40 + P)
    bn = torch.tensor(norms)
    want = tcp.batch_decompress([torch.from_numpy(i) for i in idxs], [torch.from_numpy(v) for v in vals],
                                (Y, X, 64, 64), 4096, block_norms=bn).numpy()
    # (inf / inf is NaN too: two infinite norms make the median infinite)
    assert np.isnan(want).any() == bool(np.isnan(np.array(norms)).any() or np.isinf(np.array(norms)).sum() > 1)
    comp = tc.TopKCompressor()
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v).to(dev) for v in vals]
    for _ in range(3):  # the same answer every time
        got = comp.batch_decompress(torch.empty(1, device=dev), di, dv, (Y, X, 64, 64), 4096, block_norms=bn.to(dev))
        same_with_nans(got.cpu().numpy(), want)
    # the oracle agrees with torch here too
    same_with_nans(orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, block_norms=np.array(norms, np.float32)), want)


def test_block_norms_shorter_than_the_peer_list_raise(dev):
    idxs, vals = make_peers(3, 1, 1, 32, 5)
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v).to(dev) for v in vals]
    with pytest.raises(IndexError):
        tc.TopKCompressor().batch_decompress(torch.empty(1, device=dev), di, dv, (1, 1, 64, 64), 4096,
                                             block_norms=torch.ones(2, device=dev))


@pytest.mark.parametrize("bad", ["nan", "inf", "nan+inf"])
@pytest.mark.parametrize("P,k", [(5, 32), (15, 32), (20, 64)])
def test_non_finite_values_from_one_peer(dev, P, k, bad):
    # norms computed from the values, as batch_decompress does without block_norms (:531-534)
    Y, X = 2, 3
    idxs, vals = make_peers(P, Y, X, k, 70 + P + k)
    if "nan" in bad:
        vals[1][0, 1, 3] = np.nan
    if "inf" in bad:
        vals[P - 1][1, 0, 5] = np.inf
    want = tcp.batch_decompress([torch.from_numpy(i) for i in idxs], [torch.from_numpy(v) for v in vals],
                                (Y, X, 64, 64), 4096).numpy()
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v).to(dev) for v in vals]
    got = tc.TopKCompressor().batch_decompress(torch.empty(1, device=dev), di, dv, (Y, X, 64, 64), 4096)
    same_with_nans(got.cpu().numpy(), want, rtol=2e-6)
    # the whole-set form: per-tensor norms from the flat payload, two tensors
    outs = [torch.empty(64, 64 * 2, device=dev), torch.empty(64 * 2, 64 * 2, device=dev)]
    batch = tc.TensorBatch(outs)
    fi = [torch.from_numpy(orc.pack12(orc.unpack12(i, v.shape).reshape(-1, k))).to(dev) for i, v in zip(idxs, vals)]
    fv = [torch.from_numpy(v.reshape(-1, k)).to(dev) for v in vals]
    tc.batch_decompress_decode_batch(batch, fi, fv, k, use_dct=False)
    b0 = 0
    for t, o in enumerate(outs):
        Yt, Xt = o.shape[0] // 64, o.shape[1] // 64
        cnt = Yt * Xt
        ti = [torch.from_numpy(orc.pack12(orc.unpack12(i, v.shape).reshape(-1, k)[b0:b0 + cnt])) for i, v in zip(idxs, vals)]
        tv = [torch.from_numpy(v.reshape(-1, k)[b0:b0 + cnt].reshape(Yt, Xt, k)) for v in vals]
        want_t = tcp.batch_decompress(ti, tv, (Yt, Xt, 64, 64), 4096).numpy()
        same_with_nans(o.cpu().numpy(), orc.decode2d(want_t, use_dct=False), rtol=2e-6)
        b0 += cnt


def test_nan_value_through_the_fused_inverse_transform(dev):
    # a NaN coefficient makes its whole chunk NaN after the inverse DCT, and only that chunk
    # (an infinite one is not compared: a factorised transform and a dense product differ in where inf - inf appears)
    P, k, Y, X = 4, 32, 2, 3
    idxs, vals = make_peers(P, Y, X, k, 123)
    vals[2][1, 2, 7] = np.nan
    norms = torch.tensor([1.0, 2.0, 3.0, 4.0])
    dense = tcp.batch_decompress([torch.from_numpy(i) for i in idxs], [torch.from_numpy(v) for v in vals],
                                 (Y, X, 64, 64), 4096, block_norms=norms).numpy()
    want_nan = np.isnan(dense).any(axis=(2, 3))
    assert want_nan.sum() == 1 and want_nan[1, 2]
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v).to(dev) for v in vals]
    got = tc.batch_decompress_decode(di, dv, (Y, X, 64, 64), block_norms=norms.to(dev)).cpu().numpy()
    chunks = got.reshape(Y, 64, X, 64).transpose(0, 2, 1, 3)
    assert np.array_equal(np.isnan(chunks).all(axis=(2, 3)), want_nan)
    assert np.array_equal(np.isnan(chunks).any(axis=(2, 3)), want_nan)
    clean = np.where(np.isnan(dense), 0, dense)
    ref = orc.decode2d(clean).reshape(Y, 64, X, 64).transpose(0, 2, 1, 3)
    ok = ~want_nan
    assert np.abs(chunks[ok] - ref[ok]).max() <= 1e-5 * np.abs(ref[ok]).max()


def _audit_codes(v, q_a, shift_a, scale_a, q_b, shift_b, scale_b, n_bins):
    """Two runs of the quantiser whose shift and scale differ in their last bits may code an entry
    differently only if it sits on a bin boundary to within what those differences move it."""
    diff = np.flatnonzero(q_a.reshape(-1) != q_b.reshape(-1))
    if diff.size == 0:
        return 0
    x = v.reshape(-1)[diff].astype(np.float64)
    t = (x - float(shift_a)) / float(scale_a) + n_bins // 2
    slack = (abs(float(shift_a) - float(shift_b)) / float(scale_a)
             + np.abs(t) * abs(float(scale_a) - float(scale_b)) / float(scale_a)
             + 8 * np.finfo(np.float32).eps * (np.abs(t) + np.abs(x) / float(scale_a)))
    assert (np.abs(q_a.reshape(-1)[diff].astype(int) - q_b.reshape(-1)[diff].astype(int)) == 1).all()
    assert (np.abs(t - (np.floor(t) + 0.5)) <= slack).all(), (t, slack)
    return diff.size


@pytest.mark.parametrize("n_bins", [4, 256])
def test_device_quantiser_against_torch_op_sequence(dev, n_bins):
    # tplr_quantize_batch per parameter against the reference's torch ops on the CPU (:593-621)
    rng = np.random.default_rng(5 + n_bins)
    shapes = [(128, 64), (64, 192), (1024, 512), (64, 64)]
    k = 32
    batch = tc.TensorBatch([torch.zeros(s, device=dev) for s in shapes])
    parts = []
    for i, s in enumerate(shapes):
        rows = (s[0] // 64) * (s[1] // 64)
        parts.append((rng.standard_t(3, size=(rows, k)) * 10.0 ** (i - 3) + 0.01 * i).astype(np.float32))
    val = torch.from_numpy(np.concatenate(parts)).to(dev)
    codes, shift, scale, lookup = tc.quantize_batch(batch, val, k, n_bins, 6.0)
    b0 = 0
    for i, v in enumerate(parts):
        q_t, (shift_t, scale_t, off_t, lut_t, _) = tcp.quantize(torch.from_numpy(v), n_bins, 6.0)
        got_q = codes[b0:b0 + v.shape[0]].cpu().numpy()
        assert abs(float(shift[i]) - float(shift_t)) <= 4e-7 * max(abs(float(shift_t)), np.abs(v).max() / np.sqrt(v.size))
        assert abs(float(scale[i]) - scale_t) <= 1e-6 * scale_t
        n_diff = _audit_codes(v, q_t.numpy(), float(shift_t), scale_t, got_q, float(shift[i]), float(scale[i]), n_bins)
        assert n_diff <= max(2, v.size // 100)
        same = [b for b in np.unique(got_q) if (q_t.numpy() == b).sum() == (got_q == b).sum()]
        assert np.allclose(lookup[i].cpu().numpy()[same], lut_t.numpy()[same], rtol=1e-4, atol=1e-6 * np.abs(v).max())
        b0 += v.shape[0]


@pytest.mark.parametrize("n_bins", [4, 256])
def test_device_quantiser_ties_round_to_even(dev, n_bins):
    # exact halves (range 0: the scale falls back to exactly 1; dyadic symmetric values: the mean is exactly 0):
    # every code equals torch's
    comp = tc.TopKCompressor(use_quantization=True, quantization_bins=n_bins, quantization_range=0)
    half = np.arange(-n_bins // 2 - 3, n_bins // 2 + 4, dtype=np.float32) + np.float32(0.5)
    v = np.concatenate([half, -half, np.array([0.0, 0.25, -0.25, 0.75, -0.75, 0.0], np.float32)]).astype(np.float32)
    v = np.concatenate([v, np.zeros((-v.size) % 4, np.float32)])
    q_t, (shift_t, scale_t, _, lut_t, _) = tcp.quantize(torch.from_numpy(v), n_bins, 0.0)
    q, (shift, scale, half_bins, lut, dt) = comp._quantize_values(torch.from_numpy(v).to(dev))
    assert float(shift) == float(shift_t) == 0.0 and scale == scale_t == 1.0 and half_bins == n_bins // 2
    assert np.array_equal(q.cpu().numpy(), q_t.numpy())
    assert np.allclose(lut.cpu().numpy(), lut_t.numpy(), rtol=1e-6, atol=0)
    back = comp._dequantize_values(q, (shift, scale, half_bins, lut, dt))
    assert np.array_equal(back.cpu().numpy(), tcp.dequantize(q_t, (shift_t, scale_t, half_bins, lut_t, dt)).numpy())
