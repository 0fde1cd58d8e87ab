"""Parity of the HIP kernels (through the C ABI) against the CPU oracle.  Needs an MI355X.

Bars: bit-exact for packed bytes, index sets/order and gathered values on identical
coefficient inputs, and for scattered sums/means given identical clip factors; transforms
and reconstructions within 1e-5 of the tensor's largest magnitude (fp32 tolerance).
"""
import ctypes as C
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import codec as orc  # noqa: E402  (the checker)
import templar_amd.compress as tc  # noqa: E402
from templar_amd import _lib  # noqa: E402
import workloads  # noqa: E402

GOLD = os.path.join(os.path.dirname(__file__), "golden")
TOL = 1e-5


def t3(shape, seed, row_scale=False):
    return workloads.student_t3(shape, seed, row_scale=row_scale)


def relerr(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


# ---------------------------------------------------------------- pack / unpack
def test_pack_unpack_reference_vectors(dev):
    kats = json.load(open(os.path.join(GOLD, "reference_kats.json")))
    for case in kats["pack_roundtrip"]:
        idx = torch.tensor(case["indices"], dtype=torch.int64, device=dev)
        packed = tc.pack_12bit_indices(idx)
        assert packed.dtype == torch.uint8 and packed.device == idx.device
        assert packed.numel() == case["packed_len"]
        assert np.array_equal(packed.cpu().numpy(), orc.pack12(case["indices"]))
        back = tc.unpack_12bit_indices(packed, idx.shape)
        assert back.dtype == torch.int64 and torch.equal(back, idx)


@pytest.mark.parametrize("n", [2, 6, 8, 10, 100, 4098, 1 << 20])
def test_pack_unpack_random(dev, n):
    g = torch.Generator().manual_seed(n)
    idx = torch.randint(0, 4096, (n,), generator=g, dtype=torch.int64)
    packed = tc.pack_12bit_indices(idx.to(dev))
    assert np.array_equal(packed.cpu().numpy(), orc.pack12(idx.numpy()))
    assert torch.equal(tc.unpack_12bit_indices(packed, (n,)).cpu(), idx)
    # a view that starts at an odd byte offset
    buf = torch.zeros(packed.numel() + 1, dtype=torch.uint8, device=dev)
    buf[1:] = packed
    assert torch.equal(tc.unpack_12bit_indices(buf[1:], (n // 2, 2)).cpu().reshape(-1), idx)


def test_pack_errors(dev):
    with pytest.raises(ValueError, match="Number of indices must be even"):
        tc.pack_12bit_indices(torch.tensor([1, 2, 3], device=dev))
    with pytest.raises(ValueError, match="exceeds 12-bit limit"):
        tc.pack_12bit_indices(torch.tensor([0, 4096], device=dev))
    with pytest.raises(ValueError, match="Index 70000 exceeds"):
        tc.pack_12bit_indices(torch.tensor([5, 1, 70000, 3], device=dev))
    with pytest.raises(ValueError, match="Number of indices must be even"):
        tc.unpack_12bit_indices(torch.zeros(6, dtype=torch.uint8, device=dev), (3,))
    e = tc.pack_12bit_indices(torch.tensor([], dtype=torch.int64, device=dev))
    assert e.numel() == 0 and tc.unpack_12bit_indices(e, (0,)).numel() == 0


# ---------------------------------------------------------------- transforms
def test_dct2d_fixture(dev):
    z = np.load(os.path.join(GOLD, "codec_small.npz"))
    x = torch.from_numpy(z["x"]).to(dev)
    tr = tc.ChunkingTransformer(_Stub([x]), 64)
    coef = tr.encode(x, use_dct=True)
    assert coef.shape == (2, 3, 64, 64)
    assert relerr(coef.cpu().numpy(), z["coef"]) <= TOL
    back = tr.decode(coef, use_dct=True)
    assert back.shape == x.shape and relerr(back.cpu().numpy(), z["x"]) <= TOL
    dec = tr.decode(torch.from_numpy(z["coef"]).to(dev), use_dct=True)
    assert relerr(dec.cpu().numpy(), orc.decode2d(z["coef"])) <= TOL


class _Stub:
    """Anything with named_parameters() works as the `model` argument."""

    def __init__(self, tensors):
        self.t = tensors

    def named_parameters(self):
        from types import SimpleNamespace

        for i, t in enumerate(self.t):
            yield f"p{i}", SimpleNamespace(requires_grad=True, shape=t.shape, dtype=t.dtype, device=t.device)


@pytest.mark.parametrize("shape", [(64, 64), (192, 64), (64, 448), (512, 1024)])
def test_dct2d_random_and_strided(dev, shape):
    x = t3(shape, 11 + shape[0], row_scale=True)
    want = orc.encode2d(x.numpy())
    lib = _lib.load()
    xd = x.to(dev)
    R, Cc = shape
    out = torch.empty(want.shape, dtype=torch.float32, device=dev)
    st = lib.tplr_dct2d_fwd(tc._ptr(xd), R, Cc, Cc, tc._ptr(out), None)
    assert st == 0
    torch.cuda.synchronize()
    assert relerr(out.cpu().numpy(), want) <= TOL
    # input living inside a wider buffer (row stride > C)
    wide = torch.zeros(R, Cc + 64, device=dev)
    wide[:, 32:32 + Cc] = xd
    sub = wide[:, 32:32 + Cc]
    out2 = torch.empty_like(out)
    assert lib.tplr_dct2d_fwd(tc._ptr(sub), R, Cc, sub.stride(0), tc._ptr(out2), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    # inverse of the oracle's coefficients
    back = torch.empty(R, Cc, device=dev)
    assert lib.tplr_dct2d_inv(tc._ptr(torch.from_numpy(want).to(dev)), R, Cc, tc._ptr(back), Cc, None) == 0
    torch.cuda.synchronize()
    assert relerr(back.cpu().numpy(), x.numpy()) <= TOL


def test_dct1d_and_dense_chunks(dev):
    v = t3((2048,), 5)
    p2 = torch.randn(20, 30)
    tr = tc.ChunkingTransformer(_Stub([v.clone(), p2.clone(), torch.randn(100)]), 64)
    assert tr.shape_dict[2048] == 64 and tr.shape_dict[20] == 20 and tr.shape_dict[30] == 30 and tr.shape_dict[100] == 50
    e = tr.encode(v.to(dev), use_dct=True)
    assert e.shape == (32, 64)
    assert relerr(e.cpu().numpy(), orc.dct1d(v.numpy().reshape(32, 64))) <= TOL
    d = tr.decode(e, use_dct=True)
    assert d.shape == (2048,) and relerr(d.cpu().numpy(), v.numpy()) <= TOL
    # odd row count through the 1-D kernel (tail of a 64-vector group)
    lib = _lib.load()
    rows = torch.randn(70, 64)
    out = torch.empty(70, 64, device=dev)
    assert lib.tplr_dct1d(tc._ptr(rows.to(dev)), 70, 0, tc._ptr(out), None) == 0
    torch.cuda.synchronize()
    assert relerr(out.cpu().numpy(), orc.dct1d(rows.numpy())) <= TOL
    # chunk sizes other than 64 take the dense kernel
    e2 = tr.encode(p2.to(dev), use_dct=True)
    assert e2.shape == (1, 1, 20, 30)
    assert relerr(e2.cpu().numpy(), orc.encode2d(p2.numpy(), 20, 30)) <= TOL
    assert relerr(tr.decode(e2, use_dct=True).cpu().numpy(), p2.numpy()) <= TOL
    w = torch.randn(100)
    e3 = tr.encode(w.to(dev), use_dct=True)
    assert e3.shape == (2, 50) and relerr(e3.cpu().numpy(), orc.dct1d(w.numpy().reshape(2, 50))) <= TOL
    assert relerr(tr.decode(e3, use_dct=True).cpu().numpy(), w.numpy()) <= TOL


# ---------------------------------------------------------------- top-k on identical coefficients
def check_topk(rows_np, k, dev):
    rows = torch.from_numpy(rows_np).to(dev)
    idx12, val = tc._topk_rows(rows, k)
    torch.cuda.synchronize()
    want_i, want_v = orc.topk_rows(rows_np, k)
    got_i = orc.unpack12(idx12.cpu().numpy(), want_i.shape)
    assert np.array_equal(got_i, want_i)
    assert np.array_equal(idx12.cpu().numpy(), orc.pack12(want_i))
    assert np.array_equal(val.cpu().numpy().view(np.uint32), want_v.view(np.uint32))


def test_topk_fixture_bit_exact(dev):
    z = np.load(os.path.join(GOLD, "codec_small.npz"))
    idx12, val = tc._topk_rows(torch.from_numpy(z["coef"]).to(dev).reshape(-1, 4096), 32)
    assert np.array_equal(idx12.cpu().numpy(), z["idx12"])
    assert np.array_equal(val.cpu().numpy().reshape(z["val"].shape), z["val"])


@pytest.mark.parametrize("k", [2, 16, 32, 34, 64, 100, 128, 130, 256, 1000, 4096])
def test_topk_chunks_bit_exact(dev, k):
    rows = t3((48, 4096), 1000 + k).numpy()
    check_topk(rows, k, dev)


def test_topk_skewed_chunks(dev):
    # energy concentrated in a few tile rows: the per-lane bound is loose, the exact search runs
    rows = t3((16, 4096), 77).numpy().reshape(16, 64, 64)
    rows[:, :3, :] *= 1e4
    rows[5] = 0.0
    rows[6] = 1.5  # one value everywhere: all ties
    rows[7, 10:, :] = 0.0
    check_topk(rows.reshape(16, 4096), 32, dev)
    check_topk(rows.reshape(16, 4096), 64, dev)


@pytest.mark.parametrize("kind", ["normal", "few_levels", "heavy_tails_row_scaled", "sparse"])
def test_select_is_bit_exact_on_other_value_laws(dev, kind):
    # untransformed encode = select straight from the tensor: canonical order against the oracle for
    # every k the sort network serves (one key per lane, two keys per lane) and for tie-heavy inputs
    rng = np.random.default_rng(sum(map(ord, kind)))
    Y, X = 3, 5
    shape = (Y * 64, X * 64)
    if kind == "normal":
        x = rng.standard_normal(shape)
    elif kind == "few_levels":
        x = rng.integers(-3, 4, shape)  # seven distinct values: ties everywhere
    elif kind == "heavy_tails_row_scaled":
        x = rng.standard_t(2, shape) * np.exp(rng.standard_normal((shape[0], 1)))
    else:
        x = np.where(rng.random(shape) < 0.01, rng.standard_normal(shape), 0.0)
    x = x.astype(np.float32)
    chunks = x.reshape(Y, 64, X, 64).transpose(0, 2, 1, 3).reshape(Y * X, 4096)
    xt = torch.from_numpy(x).to(dev)
    for k in (2, 8, 32, 64, 128):
        idx, val, _, _ = tc.encode_compress(xt, k, use_dct=False)
        want_i, want_v = orc.topk_rows(chunks, k)
        assert np.array_equal(tc.unpack_12bit_indices(idx, val.shape).cpu().numpy().reshape(-1, k), want_i), (kind, k)
        assert np.array_equal(val.cpu().numpy().reshape(-1, k), want_v), (kind, k)


def test_topk_special_values(dev):
    rows = np.zeros((6, 4096), np.float32)
    rows[1, [5, 900, 17]] = [2.0, -2.0, 2.0]
    rows[1, 100] = np.nan
    rows[1, 4000] = -np.inf
    rows[1, 7] = -0.0
    rows[2] = np.float32(1e-42)  # denormals everywhere
    rows[2, 4095] = np.float32(3e-42)
    rows[3, :] = np.nan
    rows[4, ::2] = 1.0
    rows[4, 1::2] = -1.0
    rows[5] = np.linspace(-1, 1, 4096, dtype=np.float32)
    for k in (2, 32, 64, 200, 4096):
        rows_d = torch.from_numpy(rows).to(dev)
        idx12, val = tc._topk_rows(rows_d, k)
        want_i, want_v = orc.topk_rows(rows, k)
        got_i = orc.unpack12(idx12.cpu().numpy(), want_i.shape)
        assert np.array_equal(got_i, want_i)
        assert np.array_equal(val.cpu().numpy().view(np.uint32), want_v.view(np.uint32))


@pytest.mark.parametrize("k", [32, 64, 100])
def test_topk_candidates_at_the_limits_of_the_short_sort_keys(dev, k):
    # The candidates are sorted on 32-bit keys (magnitude above the threshold, slot) while their magnitudes span
    # fewer than eight (one key per lane) or four (two keys) binades, on 64-bit keys otherwise; the threshold is
    # the leading bits of the k-th largest lane statistic.  Rows built to sit on both sides of each limit; the
    # selection is the oracle's bit for bit in every case.
    rng = np.random.default_rng(4242 + k)
    base = (rng.standard_normal((12, 4096)) * 1e-3).astype(np.float32)
    rows = base.copy()
    rows[0, rng.choice(4096, 5, replace=False)] *= np.float32(2.0 ** 3)      # span of three binades: short keys
    rows[1, rng.choice(4096, 5, replace=False)] *= np.float32(2.0 ** 5)      # five: short keys only with one key per lane
    rows[2, rng.choice(4096, 5, replace=False)] *= np.float32(2.0 ** 9)      # nine: long keys
    rows[3, rng.choice(4096, 3, replace=False)] = np.float32(3e38)           # near the largest finite value
    rows[4, rng.choice(4096, 3, replace=False)] = np.nan                     # NaN candidates rank first
    rows[5, rng.choice(4096, 3, replace=False)] = -np.inf
    # magnitudes that differ only below the bits the threshold search looks at: many near-ties around the bound
    lvl = np.float32(2.5e-3)
    near = rng.choice(4096, 200, replace=False)
    rows[6, near] = (lvl * (1 + np.arange(200, dtype=np.float32) * np.float32(2.0 ** -20))) * rng.choice([-1, 1], 200)
    rows[7, near] = lvl                                                       # exact ties at the bound, index order decides
    rows[8] = np.abs(rows[8])
    rows[8, ::64] = np.float32(1.0)                                           # one large value per lane of the chunk layout
    rows[9, :64] = np.float32(1.0) + np.arange(64, dtype=np.float32) * np.float32(2.0 ** -23)   # all candidates in one lane
    rows[10] = np.float32(1e-30) * base[10] / np.float32(1e-3)                # tiny but normal magnitudes
    rows[11] = np.float32(1e-39)                                              # denormals: the compare may flush them
    rows[11, rng.choice(4096, 40, replace=False)] = np.float32(2e-39)
    check_topk(rows, k, dev)


@pytest.mark.parametrize("k", [2, 32, 64, 100, 128])
def test_topk_more_nans_than_candidate_slots(dev, k):
    # NaNs rank first (all of them tie, lowest index first) and a lane's maximum drops them, so the threshold
    # statistics do not see them: rows with more NaNs than the select has candidate slots (128), spread over the
    # lanes, in a few lanes only, positive and negative, with infinities and large values beside them.
    rng = np.random.default_rng(77 + k)
    rows = (rng.standard_normal((8, 4096)) * 1e-3).astype(np.float32)
    rows[0, rng.choice(4096, 129, replace=False)] = np.nan
    rows[1, rng.choice(4096, 300, replace=False)] = np.nan
    rows[2, rng.choice(4096, 1000, replace=False)] = np.nan
    rows[2, rng.choice(4096, 50, replace=False)] = np.inf
    rows[3, 64 * 5:64 * 9] = np.nan                                   # four lanes' rows entirely
    rows[4, rng.choice(4096, 200, replace=False)] = -np.nan
    rows[4, rng.choice(4096, 200, replace=False)] = np.nan
    rows[5, rng.choice(4096, 127, replace=False)] = np.nan            # one short of the slots
    rows[6, ::2] = np.nan
    rows[6, 1::2] = np.float32(3e38)
    rows[7, rng.choice(4096, 4000, replace=False)] = np.nan
    check_topk(rows, k, dev)
    # the fused encode without the transform takes the same select
    x = torch.from_numpy(rows.reshape(8, 64, 64).transpose(1, 0, 2).reshape(64, 8 * 64).copy()).to(dev)
    idx, val, _, _ = tc.encode_compress(x, k, use_dct=False)
    want_i, want_v = orc.topk_rows(rows, k)
    assert np.array_equal(tc.unpack_12bit_indices(idx, val.shape).cpu().numpy().reshape(-1, k), want_i)
    assert np.array_equal(val.cpu().numpy().reshape(-1, k).view(np.uint32), want_v.view(np.uint32))


@pytest.mark.parametrize("n,k", [(64, 32), (64, 64), (100, 10), (37, 6), (4095, 32), (2048, 128), (2, 2), (2048, 512),
                                 (300, 300), (4095, 4094)])
def test_topk_generic_rows(dev, n, k):
    rows = t3((9, n), n * 7 + k).numpy()
    rows[3] = 0.0
    check_topk(rows, k, dev)


# ---------------------------------------------------------------- fused encode
@pytest.mark.parametrize("shape,k", [((128, 192), 32), ((64, 64), 64), ((256, 128), 2), ((192, 320), 128)])
def test_fused_encode_equals_unfused(dev, shape, k):
    x = t3(shape, 31 + k, row_scale=True).to(dev)
    idx_f, val_f, xshape, totalk = tc.encode_compress(x, k, use_dct=True)
    tr = tc.ChunkingTransformer(_Stub([x]), 64)
    coef = tr.encode(x, use_dct=True)
    idx_u, val_u, xshape_u, totalk_u = tc.TopKCompressor().compress(coef, k)
    assert tuple(xshape) == tuple(xshape_u) and totalk == totalk_u == 4096
    assert torch.equal(idx_f, idx_u) and torch.equal(val_f, val_u)
    # selection on the device's own coefficients is exactly the oracle's selection
    want_i, want_v = orc.topk_rows(coef.cpu().numpy().reshape(-1, 4096), k)
    assert np.array_equal(idx_f.cpu().numpy(), orc.pack12(want_i))
    assert np.array_equal(val_f.cpu().numpy().reshape(-1, k), want_v)


@pytest.mark.parametrize("use_dct", [True, False])
def test_selections_larger_than_the_fused_select_holds(dev, use_dct):
    # k > 128: the chunked (transformed) tensor is written out and every chunk sorted whole.  Same canonical
    # payload as the oracle's selection on the device's coefficients, through the per-tensor and the whole-set
    # entry points; with every coefficient kept (k = 4096) decode(decompress(...)) gives the tensor back
    shapes = [(128, 192), (64, 64)]
    xs = [t3(s, 400 + i, row_scale=True).to(dev) for i, s in enumerate(shapes)]
    tr = tc.ChunkingTransformer(_Stub(xs), 64)
    for k in (130, 512, 4096):
        batch = tc.TensorBatch(xs)
        bi, bv = tc.encode_compress_batch(batch, k, use_dct=use_dct)
        for i, x in enumerate(xs):
            idx, val, xshape, totalk = tc.encode_compress(x, k, use_dct=use_dct)
            coef = tr.encode(x, use_dct=use_dct)
            want_i, want_v = orc.topk_rows(coef.cpu().numpy().reshape(-1, 4096), k)
            assert np.array_equal(idx.cpu().numpy(), orc.pack12(want_i)), (k, i)
            assert np.array_equal(val.cpu().numpy().reshape(-1, k).view(np.uint32), want_v.view(np.uint32)), (k, i)
            si, sv = batch.payload_slice(i, bi, bv, k)
            assert torch.equal(si, idx) and torch.equal(sv.reshape(val.shape), val)
            if k == 4096:
                back = tc.batch_decompress_decode([idx], [val], xshape, clip_norm=False, use_dct=use_dct)
                assert relerr(back.cpu().numpy(), x.cpu().numpy()) <= TOL


def near_tie_audit(x_np, idx12, val, k, tol=TOL):
    """End-to-end check against the oracle's own transform: every selected value within
    tolerance, and any chunk whose index set differs differs only in entries whose
    magnitudes are within tolerance of the k-th largest."""
    coef = orc.encode2d(x_np).reshape(-1, 4096)
    want_i, want_v = orc.topk_rows(coef, k)
    got_i = orc.unpack12(idx12, want_i.shape)
    scale = np.abs(coef).max()
    differing = 0
    for r in range(coef.shape[0]):
        a, b = set(got_i[r].tolist()), set(want_i[r].tolist())
        assert len(a) == k
        if a != b:
            differing += 1
            kth = np.abs(want_v[r]).min()
            for i in a ^ b:
                assert abs(abs(coef[r, i]) - kth) <= 4 * tol * scale, (r, i)
        got = val.reshape(-1, k)[r]
        assert np.abs(got - coef[r, got_i[r]]).max() <= tol * scale
    return differing, coef.shape[0]


def test_fused_encode_end_to_end_tolerance(dev):
    x = t3((512, 768), 4242, row_scale=True)
    idx12, val, _, _ = tc.encode_compress(x.to(dev), 32)
    diff, n = near_tie_audit(x.numpy(), idx12.cpu().numpy(), val.cpu().numpy(), 32)
    assert diff <= max(1, n // 20)


def test_no_dct_view_path(dev):
    # encode(use_dct=False) is a view; compress() then selects straight from the dense tensor
    x = t3((128, 256), 9).to(dev)
    tr = tc.ChunkingTransformer(_Stub([x]), 64)
    enc = tr.encode(x, use_dct=False)
    assert enc.data_ptr() == x.data_ptr() and enc.shape == (2, 4, 64, 64)
    idx12, val, xshape, totalk = tc.TopKCompressor().compress(enc, 32)
    want_i, want_v = orc.topk_rows(orc.encode2d(x.cpu().numpy(), use_dct=False).reshape(-1, 4096), 32)
    assert np.array_equal(idx12.cpu().numpy(), orc.pack12(want_i))
    assert np.array_equal(val.cpu().numpy().reshape(-1, 32), want_v)
    assert tuple(xshape) == (2, 4, 64, 64) and totalk == 4096
    dec = tr.decode(tc.TopKCompressor().decompress(x, idx12, val, xshape, totalk), use_dct=False)
    assert dec.shape == x.shape
    assert np.array_equal(dec.cpu().numpy(), orc.decode2d(orc.decompress(idx12.cpu().numpy(), val.cpu().numpy(),
                                                                         xshape, totalk), use_dct=False))


# ---------------------------------------------------------------- decode-aggregate
def make_peers(P, Y, X, k, seed):
    rng = np.random.default_rng(seed)
    shared = rng.standard_normal((Y, X, 4096)).astype(np.float32)
    idxs, vals = [], []
    for p in range(P):
        g = (0.5 * shared + rng.standard_normal((Y, X, 4096)) * (1 + 0.3 * p)).astype(np.float32) * 1e-3
        i, v = orc.topk_rows(g, k)
        idxs.append(orc.pack12(i))
        vals.append(v)
    return idxs, vals


@pytest.mark.parametrize("P,k", [(1, 32), (2, 32), (15, 32), (15, 64), (3, 2), (5, 128), (7, 20), (128, 4)])
def test_aggregate_dense_bit_exact(dev, P, k):
    Y, X = 2, 3
    idxs, vals = make_peers(P, Y, X, k, 100 * P + k)
    norms = np.array([orc.norm2(v) for v in vals], np.float32)
    want = orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, block_norms=norms)
    comp = tc.TopKCompressor()
    p = torch.empty(Y * 64, X * 64, device=dev)
    got = comp.batch_decompress(p, [torch.from_numpy(i).to(dev) for i in idxs], [torch.from_numpy(v).to(dev) for v in vals],
                                (Y, X, 64, 64), 4096, block_norms=torch.from_numpy(norms).to(dev))
    assert got.shape == (Y, X, 64, 64)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # norms computed on the device: same result to rounding of the clip factors
    got2 = comp.batch_decompress(p, [torch.from_numpy(i).to(dev) for i in idxs],
                                 [torch.from_numpy(v).to(dev) for v in vals], (Y, X, 64, 64), 4096)
    assert relerr(got2.cpu().numpy(), want) <= 1e-6
    # no clipping, plain sum
    want_sum = orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, clip_norm=False, mean=False)
    got_sum = tc._aggregate_chunks([torch.from_numpy(i).to(dev) for i in idxs], [torch.from_numpy(v).to(dev) for v in vals],
                                   None, Y, X, k, normalise=False, use_dct=False, mean=False)
    assert np.array_equal(got_sum.cpu().numpy(), want_sum)


def test_aggregate_normalise(dev):
    P, k, Y, X = 4, 32, 2, 2
    idxs, vals = make_peers(P, Y, X, k, 5)
    want = orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, normalise=True)
    got = tc.TopKCompressor().batch_decompress(torch.empty(1, device=dev), [torch.from_numpy(i).to(dev) for i in idxs],
                                               [torch.from_numpy(v).to(dev) for v in vals], (Y, X, 64, 64), 4096,
                                               normalise=True)
    assert relerr(got.cpu().numpy(), want) <= 1e-6
    assert np.array_equal(got.cpu().numpy() != 0, want != 0)


@pytest.mark.parametrize("P,k", [(1, 32), (15, 32), (15, 64), (20, 32), (24, 64), (31, 16)])
def test_aggregate_fused_with_inverse_dct(dev, P, k):
    Y, X = 3, 2
    idxs, vals = make_peers(P, Y, X, k, 9 * P + k)
    norms = np.array([orc.norm2(v) for v in vals], np.float32)
    want = orc.decode2d(orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, block_norms=norms))
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v).to(dev) for v in vals]
    ss = torch.zeros(Y * X, device=dev)
    got = tc.batch_decompress_decode(di, dv, (Y, X, 64, 64), block_norms=torch.from_numpy(norms).to(dev), sumsq=ss)
    assert got.shape == (Y * 64, X * 64)
    assert relerr(got.cpu().numpy(), want) <= TOL
    per_chunk = (want.reshape(Y, 64, X, 64).astype(np.float64) ** 2).sum((1, 3)).reshape(-1)
    assert np.allclose(ss.cpu().numpy(), per_chunk, rtol=1e-4)
    # the two-call form through the reference API gives the same tensor
    comp, tr = tc.TopKCompressor(), tc.ChunkingTransformer(_Stub([torch.empty(Y * 64, X * 64)]), 64)
    lazy = comp.batch_decompress(torch.empty(1, device=dev), di, dv, (Y, X, 64, 64), 4096,
                                 block_norms=torch.from_numpy(norms).to(dev), defer=True)
    assert torch.equal(tr.decode(lazy, use_dct=True), got)
    dense = comp.batch_decompress(torch.empty(1, device=dev), di, dv, (Y, X, 64, 64), 4096,
                                  block_norms=torch.from_numpy(norms).to(dev))
    assert relerr(tr.decode(dense, use_dct=True).cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("k", [2, 4, 6, 30, 32, 34, 62, 64])
@pytest.mark.parametrize("Y,X", [(1, 1), (1, 2), (1, 3), (3, 3)])
def test_aggregate_with_transform_short_payloads(dev, k, Y, X):
    """The kernel fetches packed indices four bytes at a time for groups of rows: the last rows of a payload, rows of
    three bytes (k = 2) and payloads of a single row must come out as any other (peers strided and not)."""
    for P, strided in ((1, True), (3, True), (3, False)):
        idxs, vals = make_peers(P, Y, X, k, 1000 * k + 10 * Y + X + P)
        want = orc.decode2d(orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, clip_norm=False))
        if strided:  # equally spaced in one allocation each, exactly sized: nothing behind the last row
            ibuf = torch.from_numpy(np.stack([i.reshape(-1) for i in idxs])).to(dev)
            vbuf = torch.from_numpy(np.stack([v.reshape(-1) for v in vals])).to(dev)
            di = [ibuf[p].view(Y * X, -1) for p in range(P)]
            dv = [vbuf[p].view(Y * X, k) for p in range(P)]
        else:
            di = [torch.from_numpy(i).to(dev) for i in idxs]
            dv = [torch.from_numpy(v).to(dev) for v in vals]
            di[-1] = torch.cat([torch.zeros(5, dtype=torch.uint8, device=dev), di[-1].reshape(-1)])[5:].view(Y * X, -1)
        got = tc.batch_decompress_decode(di, dv, (Y, X, 64, 64), clip_norm=False)
        assert relerr(got.cpu().numpy(), want) <= TOL, (P, strided)


def test_aggregate_with_transform_many_chunks_per_wave(dev):
    """More chunks than resident waves, so that every wave walks several index groups and ends inside one."""
    k, P = 32, 2
    Y, X = 4, 2100                               # 8400 chunks on some 2000 waves: ranges of four and five chunks
    g = torch.Generator(device=dev); g.manual_seed(5)
    idx = torch.rand((P, Y * X, 4096), device=dev, generator=g).topk(k, dim=-1).indices
    val = torch.randn((P, Y * X, k), device=dev, generator=g)
    di = [tc.pack_12bit_indices(idx[p].contiguous()) for p in range(P)]
    dv = [val[p].contiguous() for p in range(P)]
    got = tc.batch_decompress_decode(di, dv, (Y, X, 64, 64), clip_norm=False)
    dense = torch.zeros((Y * X, 4096), device=dev)
    cnt = torch.zeros((Y * X, 4096), device=dev)
    for p in range(P):
        dense.scatter_add_(1, idx[p], val[p])
        cnt.scatter_add_(1, idx[p], torch.ones_like(val[p]))
    dense = dense / cnt.clamp(min=1)
    want = orc.decode2d(dense.view(Y, X, 64, 64).cpu().numpy())
    assert relerr(got.cpu().numpy(), want) <= TOL


def test_scatter_rows_generic(dev):
    rng = np.random.default_rng(8)
    comp = tc.TopKCompressor()
    # 1-D tensor layout (x, w) = (32, 64), packed
    v = rng.standard_normal((32, 64)).astype(np.float32)
    i, vv = orc.topk_rows(v, 32)
    got = comp.decompress(torch.empty(1, device=dev), torch.from_numpy(orc.pack12(i)).to(dev), torch.from_numpy(vv).to(dev),
                          (32, 64), 64)
    assert np.array_equal(got.cpu().numpy(), orc.scatter_rows(i, vv, 64))
    # unpacked int64 indices with many duplicates: exact source-order sums
    idx = rng.integers(0, 50, size=(7, 300))
    val = (rng.standard_normal((7, 300)) * 10.0 ** rng.integers(-3, 4, size=(7, 300))).astype(np.float32)
    got = comp.decompress(torch.empty(1, device=dev), torch.from_numpy(idx).to(dev), torch.from_numpy(val).to(dev),
                          (7, 100), 100)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), orc.scatter_rows(idx, val, 100).view(np.uint32))
    with pytest.raises(RuntimeError, match="out of bounds"):
        comp.decompress(torch.empty(1, device=dev), torch.tensor([[3, 100]], device=dev), torch.ones(1, 2, device=dev),
                        (1, 100), 100)
    # batch form on a non-chunk layout
    P = 3
    payload = []
    for p in range(P):
        g = rng.standard_normal((32, 64)).astype(np.float32)
        ii, gv = orc.topk_rows(g, 32)
        payload.append((orc.pack12(ii), gv))
    norms = np.array([orc.norm2(v_) for _, v_ in payload], np.float32)
    want = orc.batch_decompress([a for a, _ in payload], [b for _, b in payload], (32, 64), 64, block_norms=norms)
    got = comp.batch_decompress(torch.empty(1, device=dev), [torch.from_numpy(a).to(dev) for a, _ in payload],
                                [torch.from_numpy(b).to(dev) for _, b in payload], (32, 64), 64,
                                block_norms=torch.from_numpy(norms).to(dev))
    assert np.array_equal(got.cpu().numpy(), want)


def test_clip_scales_and_norms(dev):
    lib = _lib.load()
    for norms in ([3.0, 1.0, 2.0, 10.0], [5.0], [2.0, 8.0], [1.0, 1.0, 4.0, 0.0, 9.0], list(np.linspace(0.1, 7, 128))):
        n = torch.tensor(norms, dtype=torch.float32, device=dev)
        s = torch.empty_like(n)
        m = torch.empty(1, device=dev)
        assert lib.tplr_clip_scales(tc._ptr(n), len(norms), 0, tc._ptr(s), tc._ptr(m), None) == 0
        med, want = orc.clip_scales(np.array(norms, np.float32))
        assert m.item() == np.float32(med) and np.array_equal(s.cpu().numpy(), want)
    vals = [torch.randn(1000 + 0 * p, device=dev) * (p + 1) for p in range(5)]
    ss = torch.empty(5, device=dev)
    ptrs = (C.c_void_p * 5)(*[v.data_ptr() for v in vals])
    assert lib.tplr_peer_sumsq(ptrs, 5, 1000, 1, tc._ptr(ss), None) == 0
    want = np.array([float((v.double() ** 2).sum()) for v in vals])
    assert np.allclose(ss.cpu().numpy(), want, rtol=1e-5)
    # in slices (ragged: 1000 values in 7 runs), and the clip factors from the partial sums
    ss7 = torch.empty((5, 7), device=dev)
    assert lib.tplr_peer_sumsq(ptrs, 5, 1000, 7, tc._ptr(ss7), None) == 0
    assert np.allclose(ss7.sum(dim=1).cpu().numpy(), want, rtol=1e-5)
    sc = torch.empty(5, device=dev)
    assert lib.tplr_clip_scales(tc._ptr(ss7), 5, 7, tc._ptr(sc), None, None) == 0
    _, want_sc = orc.clip_scales(np.sqrt(want).astype(np.float32))
    assert np.allclose(sc.cpu().numpy(), want_sc, rtol=2e-6)


def test_bad_arguments_are_rejected(dev):
    lib = _lib.load()
    x = torch.zeros(64, 64, device=dev)
    o = torch.zeros(4096, device=dev)
    b = torch.zeros(4096, dtype=torch.uint8, device=dev)
    assert lib.tplr_dct2d_fwd(tc._ptr(x), 64, 65, 65, tc._ptr(o), None) == _lib.TPLR_E_SHAPE
    assert lib.tplr_dct2d_fwd(None, 64, 64, 64, tc._ptr(o), None) == _lib.TPLR_E_BADARG
    assert lib.tplr_topk_pack(tc._ptr(o), 1, 4096, 33, tc._ptr(b), tc._ptr(o), None) == _lib.TPLR_E_BADARG
    assert lib.tplr_topk_pack(tc._ptr(o), 1, 5000, 32, tc._ptr(b), tc._ptr(o), None) == _lib.TPLR_E_TOOMANY
    assert lib.tplr_pack12(tc._ptr(o), 3, tc._ptr(b), None, None) == _lib.TPLR_E_ODD
    assert lib.tplr_encode_topk_pack(tc._ptr(x), 64, 64, 32, 32, 1, tc._ptr(b), tc._ptr(o), None) == _lib.TPLR_E_BADARG
    assert b"even" in lib.tplr_status_string(_lib.TPLR_E_ODD)


def test_calibration_copy(dev):
    lib = _lib.load()
    src = torch.arange(1 << 20, dtype=torch.float32, device=dev)
    dst = torch.zeros_like(src)
    assert lib.tplr_calib_copy(tc._ptr(src), tc._ptr(dst), src.numel() * 4, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(src, dst)
    assert lib.tplr_calib_copy(tc._ptr(src), tc._ptr(dst), 24, None) == _lib.TPLR_E_BADARG
    assert lib.tplr_calib_copy(tc._ptr(src), tc._ptr(dst), 0, None) == 0


# ---------------------------------------------------------------- persistent loops and batches
def test_persistent_encode_many_chunks_per_wave(dev):
    # 4608 chunks: more than one resident set of waves, so every wave walks several chunks
    x = t3((4608, 4096), 2024, row_scale=True).to(dev)
    idx_f, val_f, xshape, _ = tc.encode_compress(x, 32)
    tr = tc.ChunkingTransformer(_Stub([x]), 64)
    coef = tr.encode(x, use_dct=True)
    idx_u, val_u = tc._topk_rows(coef.reshape(-1, 4096), 32)
    assert torch.equal(idx_f, idx_u) and torch.equal(val_f.reshape(-1, 32), val_u)
    # spot-check chunks against the oracle's selection on the device coefficients
    rows = coef.reshape(-1, 4096)[::97].cpu().numpy()
    want_i, want_v = orc.topk_rows(rows, 32)
    got = orc.unpack12(idx_f.cpu().numpy(), (72 * 64, 32))[::97]
    assert np.array_equal(got, want_i)
    assert np.array_equal(val_f.reshape(-1, 32)[::97].cpu().numpy(), want_v)
    # and the decode side over the same number of chunks
    full = tc.batch_decompress_decode([idx_f], [val_f], xshape, clip_norm=False)
    dense = tc.TopKCompressor().decompress(x, idx_f, val_f, xshape, 4096)
    assert torch.equal(full, tr.decode(dense, use_dct=True))


def test_batch_encode_and_aggregate_match_per_tensor(dev):
    shapes = [(128, 192), (64, 64), (512, 1024), (1536, 2048), (64, 3072), (2048, 64)]
    k, P = 32, 4
    grads = [t3(s, 500 + i, row_scale=True).to(dev) for i, s in enumerate(shapes)]
    batch = tc.TensorBatch(grads)
    assert batch.total_chunks == sum((a // 64) * (b // 64) for a, b in shapes)
    idx12, val = tc.encode_compress_batch(batch, k)
    for i, g in enumerate(grads):
        want_i, want_v, xshape, _ = tc.encode_compress(g, k)
        got_i, got_v = batch.payload_slice(i, idx12, val, k)
        assert torch.equal(got_i, want_i) and torch.equal(got_v, want_v) and tuple(xshape) == batch.xshape(i)
    # P peers with flat payloads
    pay = []
    for p in range(P):
        pg = [0.5 * g + t3(tuple(g.shape), 9000 + 10 * p + i, row_scale=True).to(dev) * (1 + p)
              for i, g in enumerate(grads)]
        pay.append(tc.encode_compress_batch(tc.TensorBatch(pg), k))
    idxs, vals = [a for a, _ in pay], [b for _, b in pay]
    scale, med = tc.peer_clip_scales_batch(batch, vals, k, return_median=True)
    assert scale.shape == (len(shapes), P) and med.shape == (len(shapes),)
    assert torch.equal(scale, tc.peer_clip_scales_batch(batch, vals, k))
    for i in range(len(shapes)):
        norms = np.array([np.sqrt((batch.payload_slice(i, idxs[p], vals[p], k)[1].double() ** 2).sum().item())
                          for p in range(P)], np.float32)
        want_med, want = orc.clip_scales(norms)
        assert np.allclose(scale[i].cpu().numpy(), want, rtol=2e-6)
        # the validator's per-parameter clip norm (neurons/validator.py:3766-3768): torch.median, the lower middle
        assert np.isclose(float(med[i]), float(want_med), rtol=2e-6) and np.isclose(float(med[i]), np.sort(norms)[(P - 1) // 2], rtol=2e-6)
    outs = [torch.full(s, float("nan"), device=dev) for s in shapes]
    ss = torch.zeros(batch.total_chunks, device=dev)
    tc.batch_decompress_decode_batch(tc.TensorBatch(outs), idxs, vals, k, scale=scale, sumsq=ss)
    for i, o in enumerate(outs):
        sl = [batch.payload_slice(i, idxs[p], vals[p], k) for p in range(P)]
        y, x = batch.xshape(i)[:2]
        want = tc._aggregate_chunks([a.contiguous() for a, _ in sl], [b.contiguous() for _, b in sl],
                                    scale[i].contiguous(), y, x, k, normalise=False, use_dct=True)
        assert torch.equal(o, want)
        b0 = batch.offsets[i]
        per_chunk = (want.reshape(y, 64, x, 64).double() ** 2).sum((1, 3)).reshape(-1)
        assert torch.allclose(ss[b0:b0 + y * x].double(), per_chunk, rtol=1e-4)
    # dense-coefficient output of the batch kernel (no inverse transform)
    couts = [torch.empty(batch.xshape(i), device=dev) for i in range(len(shapes))]
    cb = tc.TensorBatch.__new__(tc.TensorBatch)
    # coefficient tensors are (Y, X, 64, 64): describe them by hand as contiguous chunk lists
    import numpy as _np
    desc = _np.zeros(len(shapes), dtype=_np.dtype([("dense", "<u8"), ("ld", "<i8"), ("chunk_begin", "<i8"),
                                                   ("x_chunks", "<i4"), ("y_chunks", "<i4")]))
    for i, c in enumerate(couts):
        desc[i] = (c.data_ptr(), 0, batch.offsets[i], c.shape[1], c.shape[0])
    cb.tensors, cb.total_chunks, cb.device, cb.offsets = couts, batch.total_chunks, dev, batch.offsets
    cb.table = torch.from_numpy(desc.view(_np.uint8).copy()).to(dev)
    tc.batch_decompress_decode_batch(cb, idxs, vals, k, scale=scale, use_dct=False)
    for i, c in enumerate(couts):
        sl = [batch.payload_slice(i, idxs[p], vals[p], k) for p in range(P)]
        want = orc.batch_decompress([a.cpu().numpy() for a, _ in sl], [b.cpu().numpy() for _, b in sl],
                                    batch.xshape(i), 4096, clip_norm=False)  # unclipped reference for the pattern
        assert np.array_equal(c.cpu().numpy() != 0, want != 0)


# ---------------------------------------------------------------- miner side: error-feedback step
@pytest.mark.parametrize("use_dct,k,bins", [(True, 32, 0), (True, 64, 0), (False, 32, 0), (True, 32, 4), (False, 64, 256),
                                            (False, 64, 4), (False, 2, 0)])
def test_error_feedback_step_matches_reference_sequence(dev, use_dct, k, bins):
    # three tensors of different shapes, walked as one batch (src/tplr/neurons.py:147-171 per parameter)
    shapes = [(128, 192), (64, 64), (256, 128)]
    decay = 0.95
    efs = [t3(s, 400 + i, row_scale=True) for i, s in enumerate(shapes)]
    grads = [t3(s, 500 + i, row_scale=True) * 0.5 for i, s in enumerate(shapes)]
    d_ef = [e.clone().to(dev) for e in efs]
    d_gr = [g.to(dev) for g in grads]
    comp = tc.TopKCompressor(use_quantization=bins > 0, quantization_bins=bins or 256, quantization_range=6)
    eb, gb = tc.TensorBatch(d_ef), tc.TensorBatch(d_gr)
    idx12, val, quant = tc.error_feedback_step_batch(eb, gb, decay, k, use_dct=use_dct, compressor=comp)
    assert (quant is None) == (bins == 0)
    tr = tc.ChunkingTransformer(_Stub(d_ef), 64)
    for i, s in enumerate(shapes):
        # the accumulated momentum is exact: two roundings, as mul_ then add_
        acc = (efs[i] * decay) + grads[i]
        # selection on the device's own coefficients of that exact tensor, values bit-exact
        coef = tr.encode(acc.to(dev), use_dct=use_dct).cpu().numpy()
        ef_acc, want_i, want_v, want_new = orc.error_feedback_step(efs[i].numpy(), grads[i].numpy(), decay, k,
                                                                   use_dct=use_dct, quant_bins=bins, coef_override=coef)
        assert np.array_equal(ef_acc, acc.numpy())
        got_i, got_v = eb.payload_slice(i, idx12, val, k)
        assert np.array_equal(got_i.cpu().numpy(), want_i)
        assert np.array_equal(got_v.cpu().numpy(), want_v)
        # the error feedback left behind: within fp32 tolerance of the reference sequence
        got_new = d_ef[i].cpu().numpy()
        assert np.abs(got_new - want_new).max() <= TOL * np.abs(ef_acc).max()
        if not use_dct and bins == 0:
            # no transform, no quantiser: the sent entries are removed exactly, the rest untouched
            assert np.array_equal(got_new, want_new)
        if quant is not None:
            q, qp = quant[i]
            wq, wqp = orc.quantize(want_v, bins, 6.0)
            assert np.array_equal(q.cpu().numpy(), wq)


@pytest.mark.parametrize("use_dct,k,bins", [(True, 6, 4), (False, 10, 256), (False, 2, 4)])
def test_error_feedback_step_with_quantiser_for_a_topk_that_is_not_a_multiple_of_four(dev, use_dct, k, bins):
    # the whole-set quantiser kernels read values four at a time; other (even) k go parameter by parameter through
    # torch's device ops: the payload is the oracle's, the codes are the oracle's except where a sum rounded
    # differently moves a value across a bin edge, and what is subtracted is what the codes de-quantise to
    shapes = [(128, 192), (64, 64), (192, 128)]
    decay = 0.9
    efs = [t3(s, 700 + i, row_scale=True) for i, s in enumerate(shapes)]
    grads = [t3(s, 800 + i, row_scale=True) * 0.5 for i, s in enumerate(shapes)]
    d_ef = [e.clone().to(dev) for e in efs]
    comp = tc.TopKCompressor(use_quantization=True, quantization_bins=bins, quantization_range=6)
    eb, gb = tc.TensorBatch(d_ef), tc.TensorBatch([g.to(dev) for g in grads])
    idx12, val, quant = tc.error_feedback_step_batch(eb, gb, decay, k, use_dct=use_dct, compressor=comp)
    tr = tc.ChunkingTransformer(_Stub(d_ef), 64)
    for i, s in enumerate(shapes):
        acc = (efs[i] * decay) + grads[i]
        coef = tr.encode(acc.to(dev), use_dct=use_dct).cpu().numpy()
        _, want_i, want_v, _ = orc.error_feedback_step(efs[i].numpy(), grads[i].numpy(), decay, k, use_dct=use_dct,
                                                       quant_bins=0, coef_override=coef)
        got_i, got_v = eb.payload_slice(i, idx12, val, k)
        assert np.array_equal(got_i.cpu().numpy(), want_i) and np.array_equal(got_v.cpu().numpy(), want_v)
        q, qp = quant[i]
        wq, wqp = orc.quantize(want_v, bins, 6.0)
        assert (q.cpu().numpy() != wq).mean() <= 2e-3
        sent = orc.dequantize(q.cpu().numpy(), (float(qp[0]), qp[1], qp[2], qp[3].cpu().numpy()))
        y, x = s[0] // 64, s[1] // 64
        dense = orc.decompress(want_i, sent.reshape(y, x, k), (y, x, 64, 64), 4096)
        want_new = acc.numpy().astype(np.float64) - orc.decode2d(dense, use_dct=use_dct)
        assert np.abs(d_ef[i].cpu().numpy() - want_new).max() <= TOL * np.abs(acc.numpy()).max()


def test_error_feedback_null_round_and_equivalence_with_separate_calls(dev):
    shape = (192, 128)
    ef0 = t3(shape, 77, row_scale=True)
    gr = t3(shape, 78, row_scale=True)
    # fused step == the reference's call sequence through this module's own API, bitwise
    d_ef = ef0.clone().to(dev)
    eb, gb = tc.TensorBatch([d_ef]), tc.TensorBatch([gr.to(dev)])
    idx12, val, _ = tc.error_feedback_step_batch(eb, gb, 0.9, 32, use_dct=True)
    tr, comp = tc.ChunkingTransformer(_Stub([d_ef]), 64), tc.TopKCompressor()
    ref = ef0.clone().to(dev)
    ref.mul_(0.9)
    ref.add_(gr.to(dev))
    i2, v2, xshape, totalk = comp.compress(tr.encode(ref, use_dct=True), 32)
    ref.sub_(tr.decode(comp.decompress(ref, i2, v2, xshape, totalk), use_dct=True))
    assert torch.equal(idx12, i2.reshape(-1)) and torch.equal(val.reshape(v2.shape), v2)
    assert torch.equal(d_ef, ref)
    # null round: the momentum is cleared, the payload is that of zeros
    idx12, val, _ = tc.error_feedback_step_batch(eb, gb, 0.9, 32, use_dct=True, null_round=True)
    assert float(d_ef.abs().max()) == 0.0 and float(val.abs().max()) == 0.0
    assert np.array_equal(orc.unpack12(idx12.cpu().numpy(), (6, 32))[0], np.arange(32))


@pytest.mark.parametrize("k", [2, 32, 34, 64])
def test_error_feedback_step_in_one_launch_equals_its_two_launches(dev, k):
    # tplr_ef_step_batch (update, transform, select, payload, subtraction of the payload's reconstruction, every chunk
    # read once and written once) against tplr_ef_encode_topk_pack_batch followed by tplr_ef_subtract_batch: the same
    # payload and the same tensors bit for bit; ragged shapes and a strided view whose neighbours stay untouched
    shapes = [(128, 192), (64, 64), (320, 128)]
    base = t3((320, 512), 5)
    def fresh():
        big = base.clone().to(dev)
        return big, [t3(shapes[0], 1, row_scale=True).to(dev), t3(shapes[1], 2).to(dev), big[:, 128:256]]
    grads = [t3(s, 10 + i, row_scale=True).to(dev) for i, s in enumerate(shapes)]
    gb = tc.TensorBatch(grads)
    lib = _lib.load()
    res = []
    for fused in (False, True):
        big, efs = fresh()
        eb = tc.TensorBatch(efs)
        n = eb.total_chunks
        idx12 = torch.full((n * (k // 2) * 3,), 255, dtype=torch.uint8, device=dev)
        val = torch.full((n, k), float("nan"), device=dev)
        if fused:
            assert lib.tplr_ef_step_batch(eb.table.data_ptr(), gb.table.data_ptr(), len(eb), n, 0.9, k, idx12.data_ptr(),
                                          val.data_ptr(), None) == 0
        else:
            assert lib.tplr_ef_encode_topk_pack_batch(eb.table.data_ptr(), gb.table.data_ptr(), len(eb), n, 0.9, k, 1,
                                                      idx12.data_ptr(), val.data_ptr(), None) == 0
            assert lib.tplr_ef_subtract_batch(idx12.data_ptr(), val.data_ptr(), k, eb.table.data_ptr(), len(eb), n, 1,
                                              None) == 0
        torch.cuda.synchronize()
        res.append((idx12, val, [e.clone() for e in efs], big))
    (i0, v0, e0, b0), (i1, v1, e1, b1) = res
    assert torch.equal(i0, i1) and torch.equal(v0.view(torch.int32), v1.view(torch.int32))
    for a, b in zip(e0, e1):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    assert torch.equal(b1[:, :128], base.to(dev)[:, :128]) and torch.equal(b1[:, 256:], base.to(dev)[:, 256:])


@pytest.mark.parametrize("k,bins", [(64, 4), (32, 0), (16, 256)])
def test_own_payload_subtraction_writes_what_the_read_modify_write_leaves(dev, k, bins):
    # without the transform the step's own payload is subtracted by k stores per chunk (own - sent) instead of k
    # read-modify-writes (ef - sent): the same bits in every element, ragged shapes and strided tensors included
    shapes = [(128, 192), (64, 64), (320, 128)]
    big = torch.from_numpy(t3((320, 512), 5).numpy()).to(dev)
    efs = [t3(shapes[0], 1, row_scale=True).to(dev), t3(shapes[1], 2).to(dev), big[:, 128:256]]  # the last one a strided view
    grads = [t3(s, 10 + i, row_scale=True).to(dev) for i, s in enumerate(shapes)]
    eb, gb = tc.TensorBatch(efs), tc.TensorBatch(grads)
    n = eb.total_chunks
    lib = _lib.load()
    idx12 = torch.empty(n * (k // 2) * 3, dtype=torch.uint8, device=dev)
    val = torch.empty((n, k), dtype=torch.float32, device=dev)
    assert lib.tplr_ef_encode_topk_pack_batch(eb.table.data_ptr(), gb.table.data_ptr(), len(eb), n, 0.9, k, 0,
                                              idx12.data_ptr(), val.data_ptr(), None) == 0
    sent = val
    if bins:
        codes, shift, scale, lookup = tc.quantize_batch(eb, val, k, bins, 6.0)
        sent = tc.dequantize_batch(eb, codes.reshape(-1), None, k, tables=(lookup, shift))
    keep = [e.clone() for e in efs]
    assert lib.tplr_ef_subtract_batch(idx12.data_ptr(), sent.data_ptr(), k, eb.table.data_ptr(), len(eb), n, 0, None) == 0
    want = [e.clone() for e in efs]
    for e, b in zip(efs, keep):
        e.copy_(b)
    assert lib.tplr_ef_subtract_own_batch(idx12.data_ptr(), sent.data_ptr(), val.data_ptr(), k, eb.table.data_ptr(),
                                          len(eb), n, None) == 0
    torch.cuda.synchronize()
    for a, b in zip(efs, want):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    assert torch.equal(big[:, :128], torch.from_numpy(t3((320, 512), 5).numpy()).to(dev)[:, :128])  # neighbours of the view untouched


# ---------------------------------------------------------------- validator side: one peer's evaluation update
@pytest.mark.parametrize("use_dct", [True, False])
@pytest.mark.parametrize("k,repeats", [(32, False), (64, False), (2, False), (16, True)])
def test_one_peers_payload_applied_to_the_parameters_in_one_launch(dev, use_dct, k, repeats):
    # neurons/validator.py:3595-3737 per parameter: vals * clip, decompress, decode, p.data.sub_(decoded, alpha=...):
    # here one launch over three parameters (ragged shapes, one a strided view), alpha and the clip factors riding on
    # the values.  Without factors the call is tplr_ef_subtract_batch bit for bit.
    shapes = [(128, 192), (64, 64), (320, 128)]
    base = t3((320, 512), 5)
    def fresh():
        big = base.clone().to(dev)
        return big, [t3(shapes[0], 1, row_scale=True).to(dev), t3(shapes[1], 2).to(dev), big[:, 128:256]]
    rng = np.random.default_rng(900 + k)
    big, params = fresh()
    pb = tc.TensorBatch(params)
    n = pb.total_chunks
    idx = np.stack([rng.choice(4096, size=k, replace=False) for _ in range(n)]).astype(np.int64)
    if repeats:
        idx[::3, 1] = idx[::3, 0]          # a peer's row naming an entry twice: the mean of those entries
        idx[1::5, 2:6] = idx[1::5, 6:7]
    val = rng.standard_normal((n, k)).astype(np.float32)
    idx12 = torch.from_numpy(orc.pack12(idx)).to(dev).reshape(-1)
    d_val = torch.from_numpy(val).to(dev)
    alpha, clip = 0.0375, np.array([1.0, 0.3125, 0.77], np.float32)
    tc.apply_decoded_batch(pb, idx12, d_val, k, alpha=alpha, clip=torch.from_numpy(clip), use_dct=use_dct)
    torch.cuda.synchronize()
    row = 0
    for i, s in enumerate(shapes):
        rows = (s[0] // 64) * (s[1] // 64)
        sl = slice(row, row + rows)
        row += rows
        xshape = (s[0] // 64, s[1] // 64, 64, 64)
        dense = orc.decompress(orc.pack12(idx[sl]).reshape(xshape[0], xshape[1], -1),
                               (val[sl] * clip[i]).reshape(xshape[0], xshape[1], k), xshape, 4096)
        before = (base[:, 128:256] if i == 2 else t3(s, 1 + i, row_scale=(i == 0))).numpy()
        want = before.astype(np.float64) - alpha * orc.decode2d(dense, use_dct=use_dct).astype(np.float64)
        got = params[i].cpu().numpy()
        assert np.abs(got - want).max() <= TOL * max(1.0, np.abs(before).max())
        if not use_dct and not repeats:
            # untouched elements keep their bits; touched ones are one multiply and one subtraction
            flat = orc.encode2d(got, use_dct=False).reshape(rows, 4096)
            keep = orc.encode2d(before, use_dct=False).reshape(rows, 4096)
            mask = np.ones_like(flat, bool)
            np.put_along_axis(mask, idx[sl], False, axis=1)
            assert np.array_equal(flat[mask], keep[mask])
            sent = np.take_along_axis(keep, idx[sl], axis=1) - val[sl] * np.float32(np.float32(alpha) * clip[i])
            assert np.array_equal(np.take_along_axis(flat, idx[sl], axis=1), sent)
    assert torch.equal(big[:, :128], base.to(dev)[:, :128]) and torch.equal(big[:, 256:], base.to(dev)[:, 256:])
    # clip norms in place of ready factors (validator.py:3608-3612): min(1, clip_norm / (norm of the parameter's values + 1e-8))
    row, norms = 0, []
    for s in shapes:
        rows = (s[0] // 64) * (s[1] // 64)
        norms.append(np.sqrt((val[row:row + rows].astype(np.float64) ** 2).sum()))
        row += rows
    cn = np.array([norms[0] * 0.5, norms[1] * 2.0, norms[2] * 0.125], np.float32)   # clipped, not clipped, clipped
    want_clip = np.minimum(1.0, cn / (np.array(norms) + 1e-8)).astype(np.float32)
    big3, p3 = fresh()
    big4, p4 = fresh()
    tc.apply_decoded_batch(tc.TensorBatch(p3), idx12, d_val, k, alpha=alpha, clip_norm=torch.from_numpy(cn), use_dct=use_dct)
    tc.apply_decoded_batch(tc.TensorBatch(p4), idx12, d_val, k, alpha=alpha, clip=torch.from_numpy(want_clip), use_dct=use_dct)
    torch.cuda.synchronize()
    for a, b, f in zip(p3, p4, want_clip):
        assert float((a - b).abs().max()) <= 1e-6 * max(1.0, float(b.abs().max()))
    assert want_clip[1] == 1.0 and want_clip[0] < 0.51
    # no factors: the miner's subtraction, bit for bit
    lib = _lib.load()
    big1, p1 = fresh()
    big2, p2 = fresh()
    b1, b2 = tc.TensorBatch(p1), tc.TensorBatch(p2)
    tc.apply_decoded_batch(b1, idx12, d_val, k, use_dct=use_dct)
    assert lib.tplr_ef_subtract_batch(idx12.data_ptr(), d_val.data_ptr(), k, b2.table.data_ptr(), len(b2), n, int(use_dct),
                                      None) == 0
    torch.cuda.synchronize()
    for a, b in zip(p1, p2):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))


def test_one_peers_payload_update_rejects_what_it_cannot_serve(dev):
    params = [t3((64, 128), 3).to(dev)]
    pb = tc.TensorBatch(params)
    idx12 = torch.zeros(2 * 48, dtype=torch.uint8, device=dev)
    val = torch.zeros((2, 32), device=dev)
    with pytest.raises(ValueError):
        tc.apply_decoded_batch(pb, idx12.to(torch.int16), val, 32)
    with pytest.raises(RuntimeError):
        tc.apply_decoded_batch(pb, idx12[:-3], val, 32)
    with pytest.raises(IndexError):
        tc.apply_decoded_batch(pb, idx12, val, 32, clip=torch.ones(2))
    assert _lib.load().tplr_apply_decoded_batch(idx12.data_ptr(), val.data_ptr(), None, 128, pb.table.data_ptr(), 1, 2, 1,
                                                None, None) == _lib.TPLR_E_TOOMANY
    with pytest.raises(ValueError, match="on_nonfinite"):
        tc.apply_decoded_batch(pb, idx12, val, 32, on_nonfinite="skip")


@pytest.mark.parametrize("use_dct", [True, False])
@pytest.mark.parametrize("kind", ["nan", "inf", "overflow"])
def test_evaluation_update_refuses_a_non_finite_decoded_gradient(dev, use_dct, kind):
    # neurons/validator.py:3646-3660, :3677-3680: a decoded gradient with a NaN or an infinity is never subtracted
    # from the parameter and the peer is rejected with ValueError.  The launch leaves every chunk whose decoded
    # values are not all finite as it was, flags its parameter, and updates the rest exactly as without the test.
    shapes = [(128, 192), (64, 64), (256, 128)]
    k, alpha = 32, 0.25
    grads = [t3(s, 70 + i, row_scale=True).to(dev) for i, s in enumerate(shapes)]
    batch = tc.TensorBatch(grads)
    idx12, val = tc.encode_compress_batch(batch, k, use_dct=use_dct)
    clip = torch.tensor([1.0, 0.5, 1.0], device=dev)
    bad_row = batch.offsets[2] + 3  # chunk 3 of parameter 2
    if kind == "nan":
        val[bad_row, 5] = float("nan")
    elif kind == "inf":
        val[bad_row, 0] = float("-inf")
    else:  # finite in the payload and as a decoded gradient, infinite once alpha is on it
        val[bad_row, 7] = 3e38
        alpha = 1e3
    start = [torch.randn(s, device=dev) for s in shapes]
    # what the update is without the test
    plain = [p.clone() for p in start]
    assert tc.apply_decoded_batch(tc.TensorBatch(plain), idx12, val, k, alpha=alpha, clip=clip, use_dct=use_dct,
                                  on_nonfinite="ignore") is None
    assert not torch.isfinite(plain[2]).all()   # the poison the reference's check exists for
    # with it
    guarded = [p.clone() for p in start]
    flags = tc.apply_decoded_batch(tc.TensorBatch(guarded), idx12, val, k, alpha=alpha, clip=clip, use_dct=use_dct,
                                   on_nonfinite="flags")
    assert flags.tolist() == [0, 0, 1]
    assert torch.equal(guarded[0], plain[0]) and torch.equal(guarded[1], plain[1])
    y, x = 3 // (shapes[2][1] // 64), 3 % (shapes[2][1] // 64)
    mask = torch.zeros(shapes[2], dtype=torch.bool, device=dev)
    mask[64 * y:64 * y + 64, 64 * x:64 * x + 64] = True
    assert torch.equal(guarded[2][mask], start[2][mask])         # the offending chunk keeps its bits
    assert torch.equal(guarded[2][~mask], plain[2][~mask])       # every other chunk is updated as before
    assert all(torch.isfinite(p).all() for p in guarded)
    # the default raises as the reference does, and the opposite sign takes the update back
    raised = [p.clone() for p in start]
    with pytest.raises(ValueError, match="NaN/Inf"):
        tc.apply_decoded_batch(tc.TensorBatch(raised), idx12, val, k, alpha=alpha, clip=clip, use_dct=use_dct)
    assert all(torch.equal(a, b) for a, b in zip(raised, guarded))
    with pytest.raises(ValueError):
        tc.apply_decoded_batch(tc.TensorBatch(raised), idx12, val, k, alpha=-alpha, clip=clip, use_dct=use_dct)
    back = max(float((p - p0).abs().max()) / float(p0.abs().max()) for p, p0 in zip(raised, start))
    assert back <= TOL
    # a clean payload raises nothing and equals the unguarded update bit for bit
    val[bad_row] = 1e-3
    a = [p.clone() for p in start]
    b = [p.clone() for p in start]
    tc.apply_decoded_batch(tc.TensorBatch(a), idx12, val, k, alpha=0.25, clip=clip, use_dct=use_dct)
    tc.apply_decoded_batch(tc.TensorBatch(b), idx12, val, k, alpha=0.25, clip=clip, use_dct=use_dct, on_nonfinite="ignore")
    assert all(torch.equal(p, q) for p, q in zip(a, b))


# ---------------------------------------------------------------- validator side: index checks
def test_index_stats_match_reference_overlap(dev):
    rng = np.random.default_rng(21)
    P, k = 5, 32
    shapes = [(128, 192), (64, 128)]
    batch = tc.TensorBatch([torch.zeros(s, device=dev) for s in shapes])
    n = batch.total_chunks
    base = np.stack([rng.permutation(4096)[:k] for _ in range(n)])
    rows = []
    for p in range(P):
        own = np.stack([rng.permutation(4096)[:k] for _ in range(n)])
        keep = rng.random((n, k)) < 0.3 * p / P        # peers share more and more of `base`
        r = np.where(keep, base, own)
        # repair accidental repeats inside a row, then plant three real ones for peer 3
        for c in range(n):
            u, first = np.unique(r[c], return_index=True)
            if len(u) < k:
                spare = np.setdiff1d(np.arange(4096), u)[: k - len(u)]
                r[c, np.setdiff1d(np.arange(k), first)] = spare
        rows.append(r.astype(np.int64))
    rows[3][0, 5] = rows[3][0, 4]
    rows[3][7, 31] = rows[3][7, 0]
    rows[3][n - 1, 1] = rows[3][n - 1, 0]
    idxs = [torch.from_numpy(orc.pack12(r)).to(dev) for r in rows]
    pair, dup, top = tc.index_stats_batch(batch, idxs, k)
    assert pair.shape == (2, P, P)
    for t in range(2):
        b0, b1 = batch.offsets[t], (batch.offsets[t + 1] if t + 1 < len(shapes) else n)
        inter, frac = orc.index_overlap([r[b0:b1] for r in rows])
        assert np.array_equal(np.triu(pair[t].cpu().numpy(), 1), inter)
        assert np.array_equal(top[t].cpu().numpy(), [r[b0:b1].max() for r in rows])
    assert dup.sum(dim=0).cpu().tolist() == [0, 0, 0, 3, 0]
    counts = [(s[0] // 64) * (s[1] // 64) for s in shapes]
    fr = tc.overlap_fractions(pair, counts, k).cpu().numpy()
    inter_all, _ = orc.index_overlap(rows)
    assert np.allclose(np.triu(fr, 1), inter_all / (n * k))
    # rows that are not chunks: (rows, k) with k = 4, indices below 64; the reference's own known answers
    a = torch.from_numpy(orc.pack12(np.array([[0, 1, 2, 3]]))).to(dev)
    b = torch.from_numpy(orc.pack12(np.array([[2, 3, 4, 5]]))).to(dev)
    pair, dup, top = tc.index_stats_batch([1], [a, b, a], 4)
    assert pair[0].cpu().tolist() == [[0, 2, 4], [0, 0, 2], [0, 0, 0]] and top[0].cpu().tolist() == [3, 5, 3]
    assert orc.index_bounds(np.array([0, 1, 2, 3]), 64) is None


@pytest.mark.parametrize("P,k", [(2, 32), (15, 32), (32, 32), (7, 64), (31, 64), (3, 128), (9, 6)])
def test_index_stats_every_row_length_and_peer_count(dev, P, k):
    # k <= 32: two peers per wave instruction; k <= 64: one; longer rows: entry by entry
    rng = np.random.default_rng(1000 * P + k)
    counts = [37, 1, 90]
    n = sum(counts)
    shared = np.stack([rng.permutation(4096)[:k] for _ in range(n)])
    rows = []
    for p in range(P):
        own = np.stack([rng.permutation(4096)[:k] for _ in range(n)])
        r = np.where(rng.random((n, k)) < 0.4, shared, own)
        rows.append(r.astype(np.int64))  # may repeat an index inside a row: counted below
    rows[P - 1][n - 1, k - 1] = 4095
    idxs = [torch.from_numpy(orc.pack12(r)).to(dev) for r in rows]
    pair, dup, top = tc.index_stats_batch(counts, idxs, k)
    b0 = 0
    for t, cnt in enumerate(counts):
        part = [r[b0:b0 + cnt] for r in rows]
        want_dup = [sum(k - len(np.unique(row)) for row in r) for r in part]
        assert dup[t].cpu().tolist() == want_dup
        assert top[t].cpu().tolist() == [int(r.max()) for r in part]
        # shared entries of peers i < j, row by row, as sets (every repeat of peer i's entry counts once more)
        got = pair[t].cpu().numpy()
        for i in range(P):
            for j in range(i + 1, P):
                want = sum(int(np.isin(part[i][c], part[j][c]).sum()) for c in range(cnt))
                assert got[i, j] == want, (t, i, j)
        b0 += cnt


@pytest.mark.parametrize("bins", [4, 256, 7])
def test_quantize_batch_matches_oracle_per_parameter(dev, bins):
    # one launch over a flat payload against the oracle's quantiser (reference :582-621) run per parameter;
    # both carry their sums in double, so shift, scale, codes and bin means agree to the last bit
    rng = np.random.default_rng(77 + bins)
    shapes = [(128, 64), (64, 192), (1024, 512), (64, 64), (192, 128)]
    k = 32
    batch = tc.TensorBatch([torch.zeros(s, device=dev) for s in shapes])
    parts = []
    for i, s in enumerate(shapes):
        rows = (s[0] // 64) * (s[1] // 64)
        v = rng.standard_t(3, size=(rows, k)).astype(np.float32) * np.float32(10.0 ** (i - 3)) + np.float32(0.01 * i)
        parts.append(v)
    parts[3][:] = np.float32(0.25)  # a constant parameter: the scale falls back to 1
    val = torch.from_numpy(np.concatenate(parts)).to(dev)
    codes, shift, scale, lookup = tc.quantize_batch(batch, val, k, bins, 6.0)
    assert codes.shape == (batch.total_chunks, k) and codes.dtype == torch.uint8 and lookup.shape == (len(shapes), bins)
    b0 = 0
    for i, v in enumerate(parts):
        q, (sh, sc, half, lut) = orc.quantize(v, bins, 6.0)
        assert half == bins // 2
        assert float(shift[i]) == sh and float(scale[i]) == sc, (i, float(shift[i]), sh, float(scale[i]), sc)
        got_q = codes[b0:b0 + v.shape[0]].cpu().numpy()
        assert np.array_equal(got_q, q), (i, int((got_q != q).sum()))
        assert np.allclose(lookup[i].cpu().numpy(), lut, rtol=1e-6, atol=0)
        b0 += v.shape[0]
    assert float(scale[3]) == 1.0
    # what the receiving side rebuilds from it: lookup[code] + shift, per parameter
    back = tc.dequantize_batch(batch, codes.reshape(-1), [(shift[i], float(scale[i]), bins // 2, lookup[i], torch.float32)
                                                          for i in range(len(shapes))], k)
    b0 = 0
    for i, v in enumerate(parts):
        q, qp = orc.quantize(v, bins, 6.0)
        want = orc.dequantize(q, qp)
        got = back[b0:b0 + v.shape[0]].cpu().numpy()
        assert np.abs(got - want).max() <= 1e-6 * max(np.abs(want).max(), 1e-30)
        b0 += v.shape[0]


@pytest.mark.parametrize("bins", [4, 256])
def test_compressor_quantiser_on_the_device_matches_oracle(dev, bins):
    # TopKCompressor._quantize_values on device tensors (one launch) against the oracle, then through
    # compress -> decompress as the callers use it (src/tplr/neurons.py:157-166)
    comp = tc.TopKCompressor(use_quantization=True, quantization_bins=bins, quantization_range=6)
    rng = np.random.default_rng(5 + bins)
    for shape in [(2, 3, 32), (7, 64), (1, 4), (33, 1, 12)]:
        v = (rng.standard_normal(shape) * 0.02 + 0.003).astype(np.float32)
        q, (shift, scale, half, lut, dt) = comp._quantize_values(torch.from_numpy(v).to(dev))
        wq, (wshift, wscale, whalf, wlut) = orc.quantize(v, bins, 6.0)
        assert q.shape == v.shape and q.dtype == torch.uint8 and isinstance(scale, float) and dt == torch.float32
        assert float(shift) == wshift and scale == wscale and half == whalf
        assert np.array_equal(q.cpu().numpy(), wq) and np.allclose(lut.cpu().numpy(), wlut, rtol=1e-6, atol=0)
        back = comp._dequantize_values(q, (shift, scale, half, lut, dt))
        assert np.array_equal(back.cpu().numpy(), orc.dequantize(wq, (wshift, wscale, whalf, lut.cpu().numpy())))
    x = t3((128, 192), 404, row_scale=True).to(dev)
    enc = tc.ChunkingTransformer(_Stub([torch.empty(128, 192)]), 64).encode(x, use_dct=True)
    idx, qv, xshape, totalk, qp = comp.compress(enc, 32)
    dense = comp.decompress(x, idx, qv, xshape, totalk, qp)
    i2, v2, _, _ = tc.TopKCompressor().compress(enc, 32)
    wq, wqp = orc.quantize(v2.cpu().numpy(), bins, 6.0)
    want = orc.decompress(i2.cpu().numpy(), orc.dequantize(wq, wqp), xshape, totalk)
    assert torch.equal(i2, idx) and np.array_equal(qv.cpu().numpy(), wq)
    assert np.abs(dense.cpu().numpy() - want).max() <= 1e-6 * np.abs(want).max()


@pytest.mark.parametrize("bins", [4, 256])
def test_maybe_dequantize_values_one_launch_for_all_peers(dev, bins):
    # src/tplr/neurons.py:325: one parameter's uint8 values of P peers with their quant_params
    comp = tc.TopKCompressor(use_quantization=True, quantization_bins=bins, quantization_range=6)
    rng = np.random.default_rng(9 + bins)
    P, shape = 7, (3, 5, 32)
    host, codes, qps = [], [], []
    for p in range(P):
        v = (rng.standard_normal(shape) * (p + 1) * 1e-3 + 1e-4 * p).astype(np.float32)
        q, qp = orc.quantize(v, bins, 6.0)
        host.append((q, qp))
        codes.append(torch.from_numpy(q).to(dev))
        qps.append((torch.tensor(qp[0], device=dev), qp[1], qp[2], torch.from_numpy(qp[3]).to(dev), torch.float32))
    out = comp.maybe_dequantize_values(codes, qps, dev)
    assert len(out) == P
    for p in range(P):
        assert out[p].dtype == torch.float32 and out[p].shape == shape
        assert np.array_equal(out[p].cpu().numpy(), orc.dequantize(*host[p]))
        assert torch.equal(out[p], comp._dequantize_values(codes[p], qps[p]))
    # payloads still on the host, and shapes the one-launch form does not take: same results
    out_h = comp.maybe_dequantize_values([c.cpu() for c in codes], [(a.cpu(), b, c, d.cpu(), e) for a, b, c, d, e in qps], dev)
    assert all(torch.equal(a, b) and a.device == out[0].device for a, b in zip(out_h, out))
    odd = [c.reshape(-1)[:30] for c in codes]  # 30 codes: not a multiple of 4
    out_o = comp.maybe_dequantize_values(odd, qps, dev)
    assert all(torch.equal(a, b.reshape(-1)[:30]) for a, b in zip(out_o, out))
    with pytest.raises(IndexError):
        comp.maybe_dequantize_values(codes, qps[:-1] + [None], dev)


def test_dequantize_batch_matches_per_parameter_reference_path(dev):
    rng = np.random.default_rng(31)
    shapes = [(128, 64), (64, 192), (192, 128)]
    k = 32
    batch = tc.TensorBatch([torch.zeros(s, device=dev) for s in shapes])
    for bins in (4, 256):
        comp = tc.TopKCompressor(use_quantization=True, quantization_bins=bins, quantization_range=6)
        codes, qps, want = [], [], []
        for i, s in enumerate(shapes):
            y, x = s[0] // 64, s[1] // 64
            v = torch.from_numpy(rng.standard_normal((y, x, k)).astype(np.float32) * (i + 1) + i).to(dev)
            q, qp = comp._quantize_values(v)
            codes.append(q.reshape(-1))
            qps.append(qp)
            # the reference's arithmetic on the oracle side: lookup[code] + shift
            want.append(orc.dequantize(q.cpu().numpy(), (float(qp[0]), qp[1], qp[2], qp[3].cpu().numpy())))
            assert torch.equal(comp._dequantize_values(q, qp).cpu(), torch.from_numpy(want[-1]))
        got = tc.dequantize_batch(batch, torch.cat(codes), qps, k)
        assert got.shape == (batch.total_chunks, k)
        assert np.array_equal(got.cpu().numpy().reshape(-1), np.concatenate([w.reshape(-1) for w in want]))


def test_aggregate_without_transform_writes_the_gradient_layout(dev):
    # use_dct=False (templar's default hparams): batch_decompress + decode is scatter-mean + re-layout
    P, k, Y, X = 20, 64, 3, 5
    idxs, vals = make_peers(P, Y, X, k, 77)
    norms = np.array([orc.norm2(v) for v in vals], np.float32)
    dense = orc.batch_decompress(idxs, vals, (Y, X, 64, 64), 4096, block_norms=norms)
    want = orc.decode2d(dense, use_dct=False)
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v).to(dev) for v in vals]
    bn = torch.from_numpy(norms).to(dev)
    got = tc.batch_decompress_decode(di, dv, (Y, X, 64, 64), block_norms=bn, use_dct=False)
    assert got.shape == (Y * 64, X * 64)
    assert np.array_equal(got.cpu().numpy(), want)
    # through the reference-shaped calls: deferred scatter, then decode
    comp, tr = tc.TopKCompressor(), tc.ChunkingTransformer(_Stub([torch.empty(Y * 64, X * 64)]), 64)
    lazy = comp.batch_decompress(torch.empty(1, device=dev), di, dv, (Y, X, 64, 64), 4096, block_norms=bn, defer=True)
    assert torch.equal(tr.decode(lazy, use_dct=False), got)
    eager = comp.batch_decompress(torch.empty(1, device=dev), di, dv, (Y, X, 64, 64), 4096, block_norms=bn)
    assert np.array_equal(eager.cpu().numpy(), dense)
    assert torch.equal(tr.decode(eager, use_dct=False), got)
    # into a view with a row stride, and the batch form with row-major descriptors
    wide = torch.full((Y * 64, X * 64 + 128), -1.0, device=dev)
    tc.batch_decompress_decode(di, dv, (Y, X, 64, 64), block_norms=bn, use_dct=False, out=wide[:, 64:64 + X * 64])
    assert torch.equal(wide[:, 64:64 + X * 64], got) and float(wide[:, :64].max()) == -1.0
    outb = torch.empty(Y * 64, X * 64, device=dev)
    flat_i = [i.reshape(-1) for i in di]
    flat_v = [v.reshape(-1, k) for v in dv]
    scale = tc._peer_scales(dv, bn, dev).reshape(1, P)  # the same clip factors as above
    tc.batch_decompress_decode_batch(tc.TensorBatch([outb]), flat_i, flat_v, k, scale=scale, use_dct=False)
    assert torch.equal(outb, got)
    # its own norms (partial sums added in another order) agree to rounding
    tc.batch_decompress_decode_batch(tc.TensorBatch([outb]), flat_i, flat_v, k, use_dct=False)
    assert float((outb - got).abs().max()) <= 1e-6 * float(got.abs().max())



# ---------------------------------------------------------------- a gathered window as flat buffers
@pytest.mark.parametrize("quantized,where,k", [(True, "cpu", 32), (False, "cpu", 32), (True, "cuda", 32), (True, "cpu", 6),
                                               (True, "cuda", 10)])
def test_payload_stage_equals_per_parameter_path(dev, quantized, where, k):
    # the reference's per-parameter lists (src/tplr/comms.py:1938-1963) of P peers, staged flat and
    # aggregated in one launch, against the per-parameter calls of src/tplr/neurons.py:309-367
    shapes = [(128, 192), (64, 64), (256, 128), (64, 320)]
    P = 5
    comp = tc.TopKCompressor(use_quantization=quantized, quantization_bins=256, quantization_range=6)
    tr = tc.ChunkingTransformer(_Stub([torch.empty(s) for s in shapes]), 64)
    idxs, vals, qps = [[] for _ in shapes], [[] for _ in shapes], [[] for _ in shapes]
    for i, s in enumerate(shapes):
        for p in range(P):
            g = t3(s, 4000 + 17 * p + i, row_scale=True).to(dev) * (1 + p)
            out = comp.compress(tr.encode(g, use_dct=True), k)
            idxs[i].append(out[0].to(where))
            vals[i].append(out[1].to(where))
            if quantized:
                sh, sc, off, lut, dt = out[4]
                qps[i].append((sh.to(where), sc, off, lut.to(where), dt))
    outs = [torch.empty(s, device=dev) for s in shapes]
    batch = tc.TensorBatch(outs)
    stage = tc.PayloadStage(batch, k, 8, quantized=quantized)
    for rep in range(2):  # the second window reuses the buffers
        fi, fv = stage.load(idxs, vals, qps if quantized else None)
        assert len(fi) == len(fv) == P and fv[0].shape == (batch.total_chunks, k) and fv[0].dtype == torch.float32
        scale = tc.peer_clip_scales_batch(batch, fv, k)
        tc.batch_decompress_decode_batch(batch, fi, fv, k, scale=scale)
        for i, s in enumerate(shapes):
            di = [t.to(dev) for t in idxs[i]]
            dv = [t.to(dev) for t in vals[i]]
            if quantized:
                dv = comp.maybe_dequantize_values(dv, [tuple(q) for q in qps[i]], dev)
            # staged values are the reference's de-quantised values, bit for bit
            for p in range(P):
                gi, gv = batch.payload_slice(i, fi[p], fv[p], k)
                assert torch.equal(gi, di[p]) and torch.equal(gv, dv[p])
            y, x = batch.xshape(i)[:2]
            want = tc._aggregate_chunks([a.contiguous() for a in di], [b.contiguous() for b in dv], scale[i].contiguous(),
                                        y, x, k, normalise=False, use_dct=True)
            assert torch.equal(outs[i], want)
            # and the oracle's batch_decompress + decode on the same payloads (its own clip factors)
            ref = orc.decode2d(orc.batch_decompress([a.cpu().numpy() for a in di], [b.cpu().numpy() for b in dv],
                                                    batch.xshape(i), 4096), use_dct=True)
            assert np.abs(outs[i].cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()
    # off the device and back (neurons/validator.py:94-219): one copy each way
    keep_i, keep_v = [t.clone() for t in fi], [t.clone() for t in fv]
    stage.offload(P)
    torch.cuda.synchronize()
    stage.dev.zero_()
    if quantized:
        stage.values.zero_()
    ri, rv = stage.reload(P)
    assert all(torch.equal(a, b) for a, b in zip(ri, keep_i)) and all(torch.equal(a, b) for a, b in zip(rv, keep_v))
    with pytest.raises(ValueError):
        tc.PayloadStage(batch, k, 2, quantized=quantized).load(idxs, vals, qps if quantized else None)
    with pytest.raises(IndexError):
        stage.load(idxs[:-1], vals[:-1], qps[:-1] if quantized else None)


# ---------------------------------------------------------------- the 1-D parameters as one set
@pytest.mark.parametrize("use_dct", [True, False])
def test_row_batch_matches_per_parameter_calls_and_oracle(dev, use_dct):
    lengths = [64, 2048, 128, 768]
    P, k = 5, 32
    comp = tc.TopKCompressor()
    tr = tc.ChunkingTransformer(_Stub([torch.empty(n) for n in lengths]), 64)
    grads = [t3((n,), 70 + i).to(dev) * (i + 1) for i, n in enumerate(lengths)]
    rb = tc.RowBatch(grads)
    assert rb.total_rows == sum(n // 64 for n in lengths)
    idx12, val = tc.encode_compress_rows_batch(rb, k, use_dct=use_dct)
    for i, g in enumerate(grads):
        wi, wv, xshape, totalk = comp.compress(tr.encode(g, use_dct=use_dct), k)
        gi, gv = rb.payload_slice(i, idx12, val, k)
        assert torch.equal(gi, wi) and torch.equal(gv, wv) and totalk == 64 and tuple(xshape) == (lengths[i] // 64, 64)
    # P peers' flat payloads -> every parameter
    pay = []
    for p in range(P):
        pg = [0.5 * g + t3(tuple(g.shape), 500 + 10 * p + i).to(dev) * (1 + p) for i, g in enumerate(grads)]
        pay.append(tc.encode_compress_rows_batch(tc.RowBatch(pg), k, use_dct=use_dct))
    idxs, vals = [a for a, _ in pay], [b for _, b in pay]
    outs = [torch.full((n,), float("nan"), device=dev) for n in lengths]
    tc.batch_decompress_decode_rows_batch(tc.RowBatch(outs), idxs, vals, k, use_dct=use_dct)
    for i, n in enumerate(lengths):
        sl = [rb.payload_slice(i, idxs[p], vals[p], k) for p in range(P)]
        pi, pv = [a for a, _ in sl], [b for _, b in sl]
        norms = torch.stack([torch.norm(v, p=2) for v in pv])  # src/tplr/neurons.py:346
        dense = comp.batch_decompress(outs[i], pi, pv, (n // 64, 64), 64, block_norms=norms)
        want = tr.decode(dense, use_dct=use_dct)
        assert np.abs((outs[i] - want).cpu().numpy()).max() <= 1e-6 * float(want.abs().max())
        ref = orc.batch_decompress([a.cpu().numpy() for a in pi], [b.cpu().numpy() for b in pv], (n // 64, 64), 64)
        ref = orc.dct1d(ref, inverse=True) if use_dct else ref
        assert np.abs(outs[i].cpu().numpy() - ref.reshape(-1)).max() <= 1e-5 * np.abs(ref).max()
    # index statistics take the row batch as they take a chunk batch
    pair, dup, top = tc.index_stats_batch(rb, idxs, k)
    pair2, dup2, top2 = tc.index_stats_batch(rb.rows, idxs, k)
    assert torch.equal(pair, pair2) and torch.equal(dup, dup2) and torch.equal(top, top2) and int(top.max()) < 64
    # the same tensors as views of one flat buffer: read and written in place, same results
    flat_in = torch.cat(grads)
    views = list(flat_in.split(lengths))
    vb = tc.RowBatch(views)
    assert vb.flat is not None and vb.flat.data_ptr() == flat_in.data_ptr() and rb.flat is None
    i2, v2 = tc.encode_compress_rows_batch(vb, k, use_dct=use_dct)
    assert torch.equal(i2, idx12) and torch.equal(v2, val)
    flat_out = torch.full((sum(lengths),), float("nan"), device=dev)
    tc.batch_decompress_decode_rows_batch(tc.RowBatch(list(flat_out.split(lengths))), idxs, vals, k, use_dct=use_dct,
                                          validate=False)
    assert torch.equal(flat_out, torch.cat(outs))
    # an index beyond the row length: torch's scatter raises, so does the checked form
    bad = tc.pack_12bit_indices(torch.full((rb.total_rows, k), 64, dtype=torch.int64, device=dev).contiguous())
    with pytest.raises(RuntimeError):
        tc.batch_decompress_decode_rows_batch(tc.RowBatch(outs), [bad] + idxs[1:], vals, k, use_dct=use_dct)


@pytest.mark.parametrize("use_dct", [True, False])
@pytest.mark.parametrize("P,k", [(1, 2), (15, 32), (20, 64), (40, 16)])
def test_rows_decode_in_one_launch_equals_aggregate_then_transform(dev, P, k, use_dct):
    # tplr_decode_rows_batch (scatter-mean of every row, inverse transform, written into its tensor) against
    # tplr_aggregate_rows followed by tplr_dct1d: the same bits, for separately allocated vectors of ragged
    # lengths, more peers than one round of loads holds, and rows with repeated indices (added in entry order)
    rng = np.random.default_rng(7000 + 10 * P + k)
    lengths = [64, 2048, 128, 768, 64 * 65]
    R = sum(n // 64 for n in lengths)
    idxs, vals = [], []
    for p in range(P):
        sel = np.argsort(rng.random((R, 64)), axis=1)[:, :k].astype(np.int64)
        for r in range(p % 3, R, 5):
            sel[r, k - 1] = sel[r, 0]                      # a repeat inside the row
        idxs.append(tc.pack_12bit_indices(torch.from_numpy(sel).to(dev).reshape(-1)))
        vals.append(torch.from_numpy((rng.standard_t(3, size=(R, k)) * (1 + p)).astype(np.float32)).to(dev))
    one = [torch.full((n,), float("nan"), device=dev) for n in lengths]
    two = [torch.full((n,), float("nan"), device=dev) for n in lengths]
    tc.batch_decompress_decode_rows_batch(tc.RowBatch(one), idxs, vals, k, use_dct=use_dct)
    tc.batch_decompress_decode_rows_batch(tc.RowBatch(two), idxs, vals, k, use_dct=use_dct, two_step=True)
    for a, b in zip(one, two):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    # and against the oracle's scatter on the concatenation, tensor by tensor
    r0 = 0
    for i, n in enumerate(lengths):
        rows = n // 64
        pi = [orc.pack12(orc.unpack12(a.cpu().numpy(), (R, k)).reshape(R, k)[r0:r0 + rows]) for a in idxs]
        pv = [v.cpu().numpy()[r0:r0 + rows] for v in vals]
        ref = orc.batch_decompress(pi, pv, (rows, 64), 64)
        ref = orc.dct1d(ref, inverse=True) if use_dct else ref
        assert np.abs(one[i].cpu().numpy() - ref.reshape(-1)).max() <= 1e-5 * np.abs(ref).max(), i
        r0 += rows


@pytest.mark.parametrize("use_dct,bins,flat", [(True, 0, False), (True, 4, True), (False, 256, False), (False, 0, True)])
def test_error_feedback_step_for_the_1d_parameters(dev, use_dct, bins, flat):
    # src/tplr/neurons.py:147-171 per parameter, restated with the oracle's pieces on rows of 64
    lengths, k, decay = [128, 64, 1024], 32, 0.9
    efs = [t3((n,), 300 + i) for i, n in enumerate(lengths)]
    grads = [t3((n,), 310 + i) * 0.5 for i, n in enumerate(lengths)]
    if flat:
        fe, fg = torch.cat(efs).to(dev), torch.cat(grads).to(dev)
        d_ef, d_gr = list(fe.split(lengths)), list(fg.split(lengths))
    else:
        d_ef, d_gr = [e.clone().to(dev) for e in efs], [g.to(dev) for g in grads]
    comp = tc.TopKCompressor(use_quantization=bins > 0, quantization_bins=bins or 256, quantization_range=6)
    eb, gb = tc.RowBatch(d_ef), tc.RowBatch(d_gr)
    assert (eb.flat is not None) == flat
    idx12, val, quant = tc.error_feedback_step_rows_batch(eb, gb, decay, k, use_dct=use_dct, compressor=comp)
    assert (quant is None) == (bins == 0)
    for i, n in enumerate(lengths):
        acc = ((efs[i] * decay) + grads[i]).numpy()
        rows = acc.reshape(-1, 64)
        coef = orc.dct1d(rows) if use_dct else rows
        got_i, got_v = eb.payload_slice(i, idx12, val, k)
        # selection on the device's own coefficients (its transform differs from the oracle's in the last bits)
        dev_coef = tc.ChunkingTransformer(_Stub([torch.empty(n)]), 64).encode(torch.from_numpy(acc).to(dev), use_dct=use_dct)
        assert np.abs(dev_coef.cpu().numpy() - coef).max() <= TOL * np.abs(coef).max()
        want_i, want_v = orc.topk_rows(dev_coef.cpu().numpy(), k)
        assert np.array_equal(tc.unpack_12bit_indices(got_i, got_v.shape).cpu().numpy(), want_i)
        assert np.array_equal(got_v.cpu().numpy(), want_v)
        sent = want_v
        if bins:
            wq, wqp = orc.quantize(want_v, bins, 6.0)
            assert np.array_equal(quant[i][0].cpu().numpy(), wq) and quant[i][1][1] == wqp[1]
            sent = orc.dequantize(wq, wqp)
        dense = orc.decompress(orc.pack12(want_i), sent, (n // 64, 64), 64)
        recon = orc.dct1d(dense, inverse=True) if use_dct else dense
        want_new = acc - recon.reshape(-1)
        assert np.abs(d_ef[i].cpu().numpy() - want_new).max() <= TOL * np.abs(acc).max()
    if bins:
        # the payloads as a receiver holds them (per-parameter host lists) staged flat again
        T = len(lengths)
        h_idx = [[eb.payload_slice(i, idx12, val, k)[0].cpu()] for i in range(T)]
        h_val = [[quant[i][0].cpu()] for i in range(T)]
        h_qp = [[(quant[i][1][0].cpu(), quant[i][1][1], quant[i][1][2], quant[i][1][3].cpu(), torch.float32)] for i in range(T)]
        fi, fv = tc.PayloadStage(eb, k, 2, quantized=True).load(h_idx, h_val, h_qp)
        assert torch.equal(fi[0], idx12)
        for i in range(T):
            b0 = eb.offsets[i]
            want = orc.dequantize(quant[i][0].cpu().numpy(), (float(quant[i][1][0]), quant[i][1][1], quant[i][1][2],
                                                                quant[i][1][3].cpu().numpy()))
            assert np.array_equal(fv[0][b0:b0 + eb.rows[i]].cpu().numpy(), want)
    # a null round clears the error feedback and sends zeros
    i0, v0, _ = tc.error_feedback_step_rows_batch(eb, gb, decay, k, use_dct=use_dct, null_round=True)
    assert float(v0.abs().max()) == 0.0 and all(float(e.abs().max()) == 0.0 for e in d_ef)


# ---------------------------------------------------------------- under stream capture
def test_whole_set_calls_replay_from_a_captured_graph(dev):
    # the library allocates nothing and keeps no state: the whole-set launches can be recorded once
    # and replayed.  Three replays with new data in the same buffers, each against the eager calls.
    shapes = [(128, 192), (64, 64), (256, 128)]
    k, P = 32, 3
    grads = [torch.zeros(s, device=dev) for s in shapes]
    batch = tc.TensorBatch(grads)
    n = batch.total_chunks
    idx12 = torch.zeros(n * (k // 2) * 3, dtype=torch.uint8, device=dev)
    val = torch.zeros((n, k), device=dev)
    peer_idx = [torch.zeros_like(idx12) for _ in range(P)]
    peer_val = [torch.zeros_like(val) for _ in range(P)]
    outs = [torch.zeros(s, device=dev) for s in shapes]
    out_batch = tc.TensorBatch(outs)

    def fill(seed):
        for i, g in enumerate(grads):
            g.copy_(t3(tuple(g.shape), seed + i, row_scale=True).to(dev))
        for p in range(P):
            pg = [0.5 * g + t3(tuple(g.shape), seed + 100 * (p + 1) + i, row_scale=True).to(dev) for i, g in enumerate(grads)]
            a, b = tc.encode_compress_batch(tc.TensorBatch(pg), k)
            peer_idx[p].copy_(a)
            peer_val[p].copy_(b)

    def work():
        tc.encode_compress_batch(batch, k, idx12=idx12, val=val)
        tc.batch_decompress_decode_batch(out_batch, peer_idx, peer_val, k, clip_norm=True)

    fill(1)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        for _ in range(2):
            work()  # warm-up outside the capture (first-use occupancy queries, allocator pools)
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        work()
    for rep in range(3):
        fill(1000 * (rep + 2))
        work()  # eager
        torch.cuda.synchronize()
        want = (idx12.clone(), val.clone(), [o.clone() for o in outs])
        idx12.zero_(), val.zero_()
        for o in outs:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(idx12, want[0]) and torch.equal(val, want[1])
        assert all(torch.equal(a, b) for a, b in zip(outs, want[2]))


@pytest.mark.parametrize("P,k,repeats", [(15, 32, False), (1, 2, False), (20, 64, False), (3, 128, False), (40, 20, False),
                                          (15, 32, True), (5, 128, True)])
def test_sums_of_squares_of_the_summed_coefficients_from_the_payloads(dev, P, k, repeats):
    # tplr_aggregate_sumsq_batch against the oracle's dense scatter-sum, chunk by chunk: one and several rounds of
    # units, rows longer than a wave, clip factors, and repeated indices inside a row (atomic path)
    shapes = [(128, 192), (64, 64), (192, 64)]
    counts = [(a // 64) * (b // 64) for a, b in shapes]
    n = sum(counts)
    idxs, vals = make_peers(P, 1, n, k, 4000 + 10 * P + k)
    rng = np.random.default_rng(17 * P + k)
    if repeats:
        for p in range(P):
            ii = orc.unpack12(idxs[p], (n, k)).reshape(n, k).copy()
            for r in range(0, n, 2):
                ii[r, 1 + (p % (k - 1))] = ii[r, 0]          # a repeat inside one wave instruction
                if k > 64:
                    ii[r, 70] = ii[r, 3]                       # and one across two of them
            idxs[p] = orc.pack12(ii)
    batch = tc.TensorBatch([torch.empty(s, device=dev) for s in shapes])
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v.reshape(n, k)).to(dev) for v in vals]
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in di])
    vp = (C.c_void_p * P)(*[v.data_ptr() for v in dv])
    for scaled in (False, True):
        scale = rng.uniform(0.2, 1.0, size=(len(shapes), P)).astype(np.float32) if scaled else None
        dscale = torch.from_numpy(scale).to(dev) if scaled else None
        ss = torch.full((n,), -1.0, device=dev)
        st = _lib.load().tplr_aggregate_sumsq_batch(ip, vp, dscale.data_ptr() if scaled else None, P, k,
                                                    batch.table.data_ptr(), len(shapes), n, ss.data_ptr(), None)
        assert st == 0
        torch.cuda.synchronize()
        got = ss.cpu().numpy()
        b0 = 0
        for t, cnt in enumerate(counts):
            ti = [orc.pack12(orc.unpack12(i, (n, k)).reshape(n, k)[b0:b0 + cnt]) for i in idxs]
            tv = [(v.reshape(n, k)[b0:b0 + cnt] * (scale[t, p] if scaled else np.float32(1))).reshape(1, cnt, k)
                  for p, v in enumerate(vals)]
            dense = orc.batch_decompress(ti, tv, (1, cnt, 64, 64), 4096, clip_norm=False, mean=False).astype(np.float64)
            want = (dense.reshape(cnt, 4096) ** 2).sum(axis=1)
            assert np.abs(got[b0:b0 + cnt] - want).max() <= 1e-5 * want.max(), (t, scaled)
            b0 += cnt


@pytest.mark.parametrize("P,k,bins,staged", [(20, 64, 4, True), (15, 32, 4, False), (5, 64, 2, False), (8, 16, 3, True),
                                             (24, 4, 4, False), (3, 6, 4, False), (4, 10, 4, True)])
def test_aggregate_straight_from_four_bin_codes_equals_dequantise_then_aggregate(dev, P, k, bins, staged):
    # templar's own settings (hparams.json: quantization_bins 4, topk 64, use_dct false, 20 peers): the aggregate
    # picks every entry's value among its peer's four and the norms come from four counts - against
    # de-quantising every peer's payload first (src/tplr/neurons.py:325, :346) and the fp32 aggregate: the same
    # bits (sum mode, fixed factors), and with the clip factors from the counts within rounding of the norms;
    # against the oracle on the de-quantised values; rows with repeated indices; payloads equally spaced or not
    shapes = [(128, 192), (64, 64), (192, 128)]
    T = len(shapes)
    counts = [(a // 64) * (b // 64) for a, b in shapes]
    n = sum(counts)
    idxs, vals = make_peers(P, 1, n, k, 8000 + 10 * P + k)
    for p in range(0, P, 3):   # repeats inside a row
        ii = orc.unpack12(idxs[p], (n, k)).reshape(n, k).copy()
        ii[p % n, k - 1] = ii[p % n, 0]
        idxs[p] = orc.pack12(ii)
    batch = tc.TensorBatch([torch.empty(s, device=dev) for s in shapes])
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    codes, qps = [], [[None] * P for _ in range(T)]
    for p in range(P):
        c, shift, scale, lookup = tc.quantize_batch(batch, torch.from_numpy(vals[p].reshape(n, k)).to(dev), k, bins, 6.0)
        codes.append(c)
        for i in range(T):
            qps[i][p] = (shift[i].clone(), float(scale[i]), bins // 2, lookup[i].clone(), torch.float32)
    if staged:  # one buffer, the peers' payloads equally spaced (scalar addressing in the kernel)
        ib = torch.stack(di)
        cb = torch.stack([c.reshape(-1) for c in codes])
        di, codes = [ib[p] for p in range(P)], [cb[p].view(n, k) for p in range(P)]
    fp32 = [tc.dequantize_batch(batch, codes[p].reshape(-1), [qps[i][p] for i in range(T)], k) for p in range(P)]
    got = [torch.full(s, 7.0, device=dev) for s in shapes]
    want = [torch.full(s, 7.0, device=dev) for s in shapes]
    # fixed factors, both reduce modes: bit for bit
    fixed = torch.from_numpy(np.random.default_rng(P).uniform(0.3, 1.0, (T, P)).astype(np.float32)).to(dev)
    deq, nb = tc.dequantised_tables(qps, dev)
    assert nb == bins and deq.shape == (T, P, 4)
    lib = _lib.load()
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in di])
    cp = (C.c_void_p * P)(*[c.data_ptr() for c in codes])
    for mode in (_lib.REDUCE_MEAN, _lib.REDUCE_SUM):
        for sc in (fixed, None):
            st = lib.tplr_decode_aggregate_codes_batch(ip, cp, deq.data_ptr(), sc.data_ptr() if sc is not None else None, P, k,
                                                       tc.TensorBatch(got).table.data_ptr(), T, n, mode, None, None)
            assert st == 0
            tc.batch_decompress_decode_batch(tc.TensorBatch(want), di, fp32, k, scale=sc, clip_norm=False, use_dct=False,
                                             mean=mode == _lib.REDUCE_MEAN)
            for a, b in zip(got, want):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (mode, sc is None)
    # the whole call with clip factors from the counts
    tc.batch_decompress_decode_codes_batch(tc.TensorBatch(got), di, codes, qps, k)
    tc.batch_decompress_decode_batch(tc.TensorBatch(want), di, fp32, k, use_dct=False)
    b0 = 0
    for t, cnt in enumerate(counts):
        assert relerr(got[t].cpu().numpy(), want[t].cpu().numpy()) <= 1e-6, t
        ti = [orc.pack12(orc.unpack12(i, (n, k)).reshape(n, k)[b0:b0 + cnt]) for i in idxs]
        tv = [v.cpu().numpy()[b0:b0 + cnt].reshape(1, cnt, k) for v in fp32]
        Y, X = shapes[t][0] // 64, shapes[t][1] // 64
        ref = orc.batch_decompress(ti, tv, (1, cnt, 64, 64), 4096).reshape(Y, X, 64, 64).transpose(0, 2, 1, 3)
        assert relerr(got[t].cpu().numpy(), ref.reshape(shapes[t])) <= TOL, t
        b0 += cnt
    # with the statistics of the decoded parameters: the same tensors, their norms, means and finiteness
    st_out = [torch.full(s, 7.0, device=dev) for s in shapes]
    stt = tc.batch_decompress_decode_codes_batch(tc.TensorBatch(st_out), di, codes, qps, k, stats=True).cpu().numpy()
    for t, (a, b) in enumerate(zip(st_out, got)):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
        d = a.double()
        assert abs(stt[t, 0] - float(torch.linalg.vector_norm(d))) <= 1e-5 * float(torch.linalg.vector_norm(d))
        assert abs(stt[t, 1] - float(d.mean())) <= 1e-5 * float(d.abs().mean()) and stt[t, 2] == 1.0
    # a stage that keeps the codes hands them and its tables to the same call
    stage = tc.PayloadStage(batch, k, P, quantized=True)
    per_i = [[batch.payload_slice(i, di[p], fp32[p], k)[0].cpu() for p in range(P)] for i in range(T)]
    per_c = [[codes[p].reshape(-1)[batch.offsets[i] * k:(batch.offsets[i] + batch.payload_rows(i)) * k].cpu()
              for p in range(P)] for i in range(T)]
    si, sc = stage.load(per_i, per_c, qps, expand=False)
    staged_out = [torch.full(s, 7.0, device=dev) for s in shapes]
    tc.batch_decompress_decode_codes_batch(tc.TensorBatch(staged_out), si, sc, qps, k, tables=stage.tables)
    for a, b in zip(staged_out, got):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    # the settings the kernel does not take (here: the transform) de-quantise first: same call, same semantics
    tc.batch_decompress_decode_codes_batch(tc.TensorBatch(got), di, codes, qps, k, use_dct=True)
    tc.batch_decompress_decode_batch(tc.TensorBatch(want), di, fp32, k, use_dct=True)
    for a, b in zip(got, want):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    # a code the quantiser cannot have produced: the reference's lookup raises
    spoiled = [c.clone() for c in codes]
    spoiled[P - 1].view(-1)[5] = bins if bins < 4 else 9
    with pytest.raises(IndexError):
        tc.batch_decompress_decode_codes_batch(tc.TensorBatch(got), di, spoiled, qps, k)


@pytest.mark.parametrize("P,k,use_dct", [(15, 32, True), (20, 64, True), (3, 128, True), (15, 32, False), (40, 16, False)])
def test_aggregate_returns_norm_mean_and_finiteness_of_every_parameter(dev, P, k, use_dct):
    # what outer_step computes after decode with three passes over each dense gradient
    # (src/tplr/neurons.py:380-385 norm and mean, :411/:438 isfinite), here from two floats per chunk: against
    # numpy on the very tensors the launch wrote; every fast and generic instantiation
    shapes = [(128, 192), (64, 64), (256, 128), (64, 320)]
    counts = [(a // 64) * (b // 64) for a, b in shapes]
    n = sum(counts)
    idxs, vals = make_peers(P, 1, n, k, 6000 + 10 * P + k)
    # tensor 1: one peer sends a NaN; tensor 2: values near the top of the range (squares overflow, elements and
    # their sum stay finite); tensor 3: an infinity
    b = np.cumsum([0] + counts)
    vals[0].reshape(n, k)[b[1], 3] = np.nan
    for p in range(P):
        vals[p].reshape(n, k)[b[2]:b[3]] *= np.float32(1e36) / np.abs(vals[p].reshape(n, k)[b[2]:b[3]]).max()
    vals[P - 1].reshape(n, k)[b[3] + 2, 0] = np.inf
    outs = [torch.full(s, 3.0, device=dev) for s in shapes]
    batch = tc.TensorBatch(outs)
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v.reshape(n, k)).to(dev) for v in vals]
    scale = torch.full((len(shapes), P), 0.5, device=dev)
    st = tc.batch_decompress_decode_batch(batch, di, dv, k, scale=scale, use_dct=use_dct, stats=True).cpu().numpy()
    plain = [torch.full(s, 3.0, device=dev) for s in shapes]
    assert tc.batch_decompress_decode_batch(tc.TensorBatch(plain), di, dv, k, scale=scale, use_dct=use_dct) is None
    for t, o in enumerate(outs):
        got = o.cpu().numpy()
        assert np.array_equal(got.view(np.uint32), plain[t].cpu().numpy().view(np.uint32)), t  # the same launch otherwise
        finite = bool(np.isfinite(got).all())
        assert st[t, 2] == (1.0 if finite else 0.0), (t, st[t])
        assert finite == (t in (0, 2)), t
        if finite:
            g = got.astype(np.float64)
            assert abs(st[t, 0] - np.sqrt((g * g).sum())) <= 1e-5 * np.sqrt((g * g).sum()), (t, st[t])
            assert abs(st[t, 1] - g.mean()) <= 1e-5 * np.abs(g).mean(), (t, st[t])
        else:
            assert not np.isfinite(st[t, 0])


@pytest.mark.parametrize("two_pass", [False, True])
@pytest.mark.parametrize("use_dct", [True, False])
def test_aggregate_mean_over_peers_then_normalised_per_tensor(dev, use_dct, two_pass):
    # the benchmark's wording of the aggregation workload: scatter-sum, inverse transform, divide by the number
    # of peers, divide every tensor by its L2 norm - against the oracle, tensor by tensor; the norm taken from
    # the payloads before the one aggregate launch (the default) and from the dense result (two_pass)
    P, k = 15, 32
    shapes = [(128, 192), (64, 64), (256, 128)]
    counts = [(a // 64) * (b // 64) for a, b in shapes]
    n = sum(counts)
    idxs, vals = make_peers(P, 1, n, k, 321)
    outs = [torch.full(s, 3.0, device=dev) for s in shapes]
    batch = tc.TensorBatch(outs)
    di = [torch.from_numpy(i).to(dev) for i in idxs]
    dv = [torch.from_numpy(v.reshape(n, k)).to(dev) for v in vals]
    factor = tc.aggregate_mean_normalised_batch(batch, di, dv, k, use_dct=use_dct, two_pass=two_pass)
    b0 = 0
    for t, (shape, cnt) in enumerate(zip(shapes, counts)):
        Y, X = shape[0] // 64, shape[1] // 64
        ti = [orc.pack12(orc.unpack12(i, (n, k))[b0:b0 + cnt]) for i in idxs]
        tv = [v.reshape(n, k)[b0:b0 + cnt].reshape(Y, X, k) for v in vals]
        want = orc.aggregate_mean_normalised(ti, tv, (Y, X, 64, 64), 4096, use_dct=use_dct)
        got = outs[t].cpu().numpy()
        assert abs(float(np.sqrt((got.astype(np.float64) ** 2).sum())) - 1.0) <= 1e-5
        assert np.abs(got - want).max() <= TOL * np.abs(want).max(), t
        plain = orc.decode2d(orc.batch_decompress(ti, tv, (Y, X, 64, 64), 4096, clip_norm=False, mean=False), use_dct=use_dct)
        assert abs(float(factor[t]) * np.sqrt((plain.astype(np.float64) ** 2).sum()) / P - 1.0) <= 1e-5
        b0 += cnt


@pytest.mark.parametrize("use_dct", [True, False])
@pytest.mark.parametrize("k", [2, 16, 32, 64])
def test_rows_encode_in_one_launch_equals_transform_then_select(dev, k, use_dct):
    # tplr_encode_rows_batch (every 1-D parameter where it lies, one launch) against tplr_dct1d followed by
    # tplr_topk_pack on the concatenation: the same bytes, for separately allocated vectors of ragged lengths,
    # with ties, zeros, denormals, infinities and NaNs among the elements
    rng = np.random.default_rng(900 + k)
    lengths = [64, 128, 768, 2048, 64 * 65, 64 * 3, 64 * 130]
    host = []
    for j, n in enumerate(lengths):
        v = (rng.standard_t(3, size=n) * 10.0 ** (j % 3 - 2)).astype(np.float32)
        v[rng.integers(0, n, n // 8)] = 0.0
        v[rng.integers(0, n, n // 16)] = np.float32(0.5)      # exact ties, either sign
        v[rng.integers(0, n, n // 16)] = np.float32(-0.5)
        host.append(v)
    host[1][:64] = 0.0                       # an all-zero row
    host[2][5] = np.nan
    host[2][70] = -np.nan
    host[3][100] = np.inf
    host[3][101] = -np.inf
    host[4][64 * 64 + 3] = np.float32(1e-41)  # a denormal in the second group of a tensor
    vecs = [torch.from_numpy(v).to(dev) for v in host]  # separate allocations
    rb = tc.RowBatch(vecs)
    assert rb.flat is None and rb.total_groups == 1 + 1 + 1 + 1 + 2 + 1 + 3
    idx12, val = tc.encode_compress_rows_batch(rb, k, use_dct=use_dct)
    rows = torch.cat(vecs).reshape(-1, 64)
    lib = _lib.load()
    if use_dct:
        coef = torch.empty_like(rows)
        with tc._on(dev):
            assert lib.tplr_dct1d(tc._ptr(rows), rows.shape[0], 0, tc._ptr(coef), tc._stream(dev)) == 0
        rows = coef
    want_i, want_v = tc._topk_rows(rows, k)
    assert val.shape == want_v.shape == (rb.total_rows, k)
    assert torch.equal(idx12, want_i)
    got_v, ref_v = val.cpu().numpy(), want_v.cpu().numpy()
    assert np.array_equal(np.isnan(got_v), np.isnan(ref_v))  # (a NaN's payload bits are not compared)
    fin = ~np.isnan(ref_v)
    assert np.array_equal(got_v.view(np.uint32)[fin], ref_v.view(np.uint32)[fin])
    # and the oracle's selection on those coefficients
    oi, ov = orc.topk_rows(rows.cpu().numpy(), k)
    assert np.array_equal(idx12.cpu().numpy(), orc.pack12(oi))

