"""The outer step over a window in one launch (tplr_outer_step_batch, outer_step_batch) against the oracle's
restatement of src/tplr/neurons.py:341-447 with the plain SGD of neurons/trainer.py:128-130.  Needs an MI355X.

Bars: updated parameters within 1e-5 of the parameter's largest magnitude (the transform and the order in which lr
and the clip factor are applied differ in rounding), gradient norm within 1e-5, a parameter whose gradient is not
finite left bit for bit as it was, the fused launch equal to aggregate-then-subtract on the device within the
same tolerance.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import codec as orc  # noqa: E402  (the checker)
import templar_amd.compress as tc  # noqa: E402
import workloads  # noqa: E402

TOL = 1e-5


def t3(shape, seed, row_scale=False):
    return workloads.student_t3(shape, seed, row_scale=row_scale)


def _window(dev, shapes, k, P, use_dct=True, staged=False):
    base = [t3(s, 400 + i, row_scale=True).to(dev) for i, s in enumerate(shapes)]
    batch = tc.TensorBatch(base)
    stage = tc.PayloadStage(batch, k, P, quantized=False) if staged else None
    idxs, vals = [], []
    for p in range(P):
        own = [0.5 * g + t3(tuple(g.shape), 7000 + 10 * p + i, row_scale=True).to(dev) * (1 + 0.5 * p) for i, g in enumerate(base)]
        if staged:
            i12, v = stage.regions(p)
            tc.encode_compress_batch(tc.TensorBatch(own), k, use_dct=use_dct, idx12=i12, val=v)
        else:
            i12, v = tc.encode_compress_batch(tc.TensorBatch(own), k, use_dct=use_dct)
        idxs.append(i12)
        vals.append(v)
    return batch, idxs, vals, stage


def _check_against_oracle(batch, params, start, idxs, vals, k, lr, stats, skipped, use_dct, expect_skipped=()):
    assert sorted(skipped) == sorted(expect_skipped)
    P = len(vals)
    for t in range(len(batch)):
        sl = [batch.payload_slice(t, idxs[p], vals[p], k) for p in range(P)]
        xshape = batch.xshape(t)
        want, g_norm, g_mean, applied = orc.outer_step(
            start[t].cpu().numpy(), [a.cpu().numpy().reshape(xshape[0], xshape[1], -1) for a, _ in sl],
            [b.cpu().numpy() for _, b in sl], xshape, 4096, lr, use_dct=use_dct)
        got = params[t].cpu().numpy()
        assert applied == (t not in expect_skipped)
        if not applied:
            assert np.array_equal(got.view(np.int32), start[t].cpu().numpy().view(np.int32)), f"parameter {t} was touched"
            assert float(stats[t, 2]) == 0.0
            continue
        assert np.abs(got - want).max() <= TOL * np.abs(want).max(), (t, np.abs(got - want).max())
        assert float(stats[t, 2]) == 1.0
        assert np.isclose(float(stats[t, 0]), g_norm, rtol=2e-5), (t, float(stats[t, 0]), g_norm)
        assert abs(float(stats[t, 1]) - g_mean) <= 2e-5 * g_norm / np.sqrt(want.size) + 1e-12
        assert np.isclose(float(stats[t, 3]), g_norm ** 2, rtol=4e-5)


@pytest.mark.parametrize("P,k,staged", [(15, 32, True), (15, 32, False), (8, 64, True), (3, 16, False), (1, 32, True),
                                        (9, 4, True)])
def test_outer_step_in_one_launch_matches_the_reference_sequence(dev, P, k, staged):
    shapes = [(128, 192), (64, 64), (320, 128), (512, 256)]
    batch, idxs, vals, _ = _window(dev, shapes, k, P, staged=staged)
    gen = torch.Generator(device=dev).manual_seed(3)
    big = torch.randn((320, 512), device=dev, generator=gen)
    big0 = big.clone()
    start = [torch.randn(shapes[0], device=dev, generator=gen), torch.randn(shapes[1], device=dev, generator=gen),
             big[:, 128:256].clone(), torch.randn(shapes[3], device=dev, generator=gen)]
    params = [start[0].clone(), start[1].clone(), big[:, 128:256], start[3].clone()]   # one parameter a strided view
    lr = 0.4
    stats, skipped = tc.outer_step_batch(tc.TensorBatch(params), idxs, vals, k, lr)
    torch.cuda.synchronize()
    _check_against_oracle(batch, params, start, idxs, vals, k, lr, stats, skipped, True)
    assert torch.equal(big[:, :128], big0[:, :128]) and torch.equal(big[:, 256:], big0[:, 256:])  # around the view
    # with ready clip factors (noted on arrival) the same bits
    again = [s.clone() for s in start]
    norms = tc.PeerNorms([batch], P)
    for p in range(P):
        norms.arrived(p, [vals[p]])
    stats2, skipped2 = tc.outer_step_batch(tc.TensorBatch(again), idxs, vals, k, lr, scale=norms.clip_scales(P)[0])
    assert skipped2 == [] and all(torch.equal(a, b) for a, b in zip(again, [p.contiguous() for p in params]))
    assert torch.equal(stats, stats2)
    # and the opposite sign takes the step back
    tc.outer_step_batch(tc.TensorBatch(again), idxs, vals, k, -lr, stats=False)
    assert max(float((a - s).abs().max()) / float(s.abs().max()) for a, s in zip(again, start)) <= TOL


def test_outer_step_equals_aggregate_then_subtract_on_the_device(dev):
    shapes = [(256, 256), (128, 512), (64, 64)]
    k, P, lr = 32, 15, 0.25
    batch, idxs, vals, _ = _window(dev, shapes, k, P, staged=True)
    start = [torch.randn(s, device=dev) for s in shapes]
    params = [s.clone() for s in start]
    stats, skipped = tc.outer_step_batch(tc.TensorBatch(params), idxs, vals, k, lr)
    dense = [torch.empty(s, device=dev) for s in shapes]
    ref_stats = tc.batch_decompress_decode_batch(tc.TensorBatch(dense), idxs, vals, k, clip_norm=True, stats=True)
    assert skipped == []
    for p, s, g in zip(params, start, dense):
        want = s - lr * g
        assert float((p - want).abs().max()) <= TOL * float(want.abs().max())
    assert torch.allclose(stats[:, 0], ref_stats[:, 0], rtol=2e-5) and torch.allclose(stats[:, 3], ref_stats[:, 3], rtol=4e-5)
    assert torch.equal(stats[:, 2], ref_stats[:, 2])


@pytest.mark.parametrize("kind", ["nan", "inf", "nan_norm_other_parameter_fine"])
def test_a_parameter_with_a_non_finite_gradient_is_left_alone(dev, kind):
    # src/tplr/neurons.py:438-442: `if not torch.isfinite(p.grad).all(): p.grad = None; continue` - the whole
    # parameter keeps its bits, the others take their step
    shapes = [(128, 192), (256, 128), (64, 64)]
    k, P, lr = 32, 5, 0.4
    batch, idxs, vals, _ = _window(dev, shapes, k, P, staged=True)
    row = batch.offsets[1] + 2
    if kind == "nan":
        vals[3][row, 4] = float("nan")
    elif kind == "inf":
        vals[0][row, 0] = float("inf")
    else:
        vals[2][row, 9] = float("nan")
    start = [torch.randn(s, device=dev) for s in shapes]
    params = [s.clone() for s in start]
    stats, skipped = tc.outer_step_batch(tc.TensorBatch(params), idxs, vals, k, lr)
    _check_against_oracle(batch, params, start, idxs, vals, k, lr, stats, skipped, True, expect_skipped=[1])


@pytest.mark.parametrize("P,k,use_dct", [(20, 32, True), (4, 32, False), (4, 128, True)])
def test_settings_outside_the_fused_launch_take_the_reference_route(dev, P, k, use_dct):
    shapes = [(128, 128), (64, 192)]
    batch, idxs, vals, _ = _window(dev, shapes, k, P, use_dct=use_dct)
    start = [torch.randn(s, device=dev) for s in shapes]
    params = [s.clone() for s in start]
    stats, skipped = tc.outer_step_batch(tc.TensorBatch(params), idxs, vals, k, 0.1, use_dct=use_dct)
    _check_against_oracle(batch, params, start, idxs, vals, k, 0.1, stats, skipped, use_dct)


def test_outer_step_argument_checks(dev):
    import ctypes as C
    from templar_amd import _lib
    shapes = [(64, 128)]
    batch, idxs, vals, _ = _window(dev, shapes, 32, 2)
    params = tc.TensorBatch([torch.zeros(shapes[0], device=dev)])
    with pytest.raises(ValueError):
        tc.outer_step_batch(params, idxs, vals, 32, 0.0)
    with pytest.raises(RuntimeError):
        tc.outer_step_batch(params, idxs, [v[:1] for v in vals], 32, 0.1)
    with pytest.raises(ValueError):
        tc.outer_step_batch(params, idxs, vals, 32, 0.1, scale=torch.ones(3, 3, device=dev))
    lib = _lib.load()
    ip = (C.c_void_p * 2)(*[i.data_ptr() for i in idxs])
    vp = (C.c_void_p * 2)(*[v.data_ptr() for v in vals])
    t = params.table.data_ptr()
    assert lib.tplr_outer_step_batch(ip, vp, None, 16, 32, t, 1, 2, None, None, None, None) == _lib.TPLR_E_TOOMANY
    assert lib.tplr_outer_step_batch(ip, vp, None, 2, 128, t, 1, 2, None, None, None, None) == _lib.TPLR_E_TOOMANY
    assert lib.tplr_outer_step_batch(ip, vp, None, 2, 2, t, 1, 2, None, None, None, None) == _lib.TPLR_E_BADARG
    assert lib.tplr_outer_step_batch(ip, vp, None, 2, 32, t, 1, 2, vals[0].data_ptr(), None, None, None) == _lib.TPLR_E_BADARG
    assert lib.tplr_outer_step_batch(None, vp, None, 2, 32, t, 1, 2, None, None, None, None) == _lib.TPLR_E_BADARG


@pytest.mark.parametrize("use_dct", [True, False])
def test_outer_step_of_the_one_dimensional_parameters(dev, use_dct):
    # the norm vectors of a model: rows of 64, the same reference lines; oracle = its batch_decompress (pinned
    # against torch) + the 64-point inverse transform (pinned against scipy) + the SGD line
    lengths = [64, 2048, 128, 768]
    P, k, lr = 5, 32, 0.4
    base = [t3((n,), 70 + i).to(dev) * (i + 1) for i, n in enumerate(lengths)]
    rb = tc.RowBatch(base)
    pay = []
    for p in range(P):
        pg = [0.5 * g + t3(tuple(g.shape), 500 + 10 * p + i).to(dev) * (1 + p) for i, g in enumerate(base)]
        pay.append(tc.encode_compress_rows_batch(tc.RowBatch(pg), k, use_dct=use_dct))
    idxs, vals = [a for a, _ in pay], [b.clone() for _, b in pay]
    vals[1][rb.offsets[2], 3] = float("nan")        # parameter 2 gets a poisoned gradient
    start = [torch.randn(n, device=dev) for n in lengths]
    params = [s.clone() for s in start]
    stats, skipped = tc.outer_step_rows_batch(tc.RowBatch(params), idxs, vals, k, lr, use_dct=use_dct)
    assert skipped == [2] and float(stats[2, 2]) == 0.0
    assert torch.equal(params[2].view(torch.int32), start[2].view(torch.int32))
    for i, n in enumerate(lengths):
        if i == 2:
            continue
        sl = [rb.payload_slice(i, idxs[p], vals[p], k) for p in range(P)]
        ref = orc.batch_decompress([a.cpu().numpy() for a, _ in sl], [b.cpu().numpy() for _, b in sl], (n // 64, 64), 64)
        grad = (orc.dct1d(ref, inverse=True) if use_dct else ref).reshape(-1)
        want = start[i].cpu().numpy() - np.float32(lr) * grad
        assert np.abs(params[i].cpu().numpy() - want).max() <= TOL * np.abs(want).max()
        assert np.isclose(float(stats[i, 0]), np.sqrt((grad.astype(np.float64) ** 2).sum()), rtol=2e-5)
        assert abs(float(stats[i, 1]) - grad.astype(np.float64).mean()) <= 2e-5 * np.abs(grad).max()
        assert float(stats[i, 2]) == 1.0
    # ready clip factors give the same bits
    again = [s.clone() for s in start]
    norms = tc.PeerNorms([rb], P)
    for p in range(P):
        norms.arrived(p, [vals[p]])
    tc.outer_step_rows_batch(tc.RowBatch(again), idxs, vals, k, lr, use_dct=use_dct, scale=norms.clip_scales(P)[0], stats=False)
    assert all(torch.equal(a.view(torch.int32), b.view(torch.int32)) for a, b in zip(again, params))


def _codes_window(dev, shapes, k, P, bins=4):
    """P peers' staged 4-bin payloads of untransformed chunks: (batch, idxs, codes, quant_params, fp32 values)."""
    base = [t3(s, 300 + i, row_scale=True).to(dev) for i, s in enumerate(shapes)]
    batch = tc.TensorBatch(base)
    T, n = len(shapes), batch.total_chunks
    stage = tc.PayloadStage(batch, k, P, quantized=True)
    idxs, codes, qps, fp32 = [], [], [[None] * P for _ in range(T)], []
    for p in range(P):
        own = [0.5 * g + t3(tuple(g.shape), 6000 + 10 * p + i, row_scale=True).to(dev) * (1 + 0.3 * p) for i, g in enumerate(base)]
        i12, c = stage.regions(p)
        idx_p, val_p = tc.encode_compress_batch(tc.TensorBatch(own), k, use_dct=False)
        cc, shift, scale, lookup = tc.quantize_batch(batch, val_p, k, bins, 6.0)
        i12.copy_(idx_p)
        c.copy_(cc)
        for i in range(T):
            qps[i][p] = (shift[i].clone(), float(scale[i]), bins // 2, lookup[i].clone(), torch.float32)
        idxs.append(i12)
        codes.append(c)
        fp32.append(tc.dequantize_batch(batch, c.reshape(-1), [qps[i][p] for i in range(T)], k))
    return batch, idxs, codes, qps, fp32


@pytest.mark.parametrize("P,k", [(20, 64), (15, 32), (4, 64), (24, 32)])
def test_outer_step_straight_from_four_bin_codes(dev, P, k):
    # templar's own settings (hparams.json: 4-bin quantiser, use_dct false, top-k 64, 20 peers): against the oracle's
    # outer step on the de-quantised values, and against the same call's reference route on the device
    shapes = [(128, 192), (64, 64), (256, 256), (192, 128)]
    batch, idxs, codes, qps, fp32 = _codes_window(dev, shapes, k, P)
    start = [torch.randn(s, device=dev) for s in shapes]
    params = [s.clone() for s in start]
    lr = 0.4
    stats, skipped = tc.outer_step_codes_batch(tc.TensorBatch(params), idxs, codes, qps, k, lr)
    _check_against_oracle(batch, params, start, idxs, fp32, k, lr, stats, skipped, False)
    # the reference route on the de-quantised values: the same tensors within rounding of the clip factors
    other = [s.clone() for s in start]
    stats2, skipped2 = tc.outer_step_batch(tc.TensorBatch(other), idxs, fp32, k, lr, use_dct=False)
    assert skipped2 == []
    for a, b in zip(params, other):
        assert float((a - b).abs().max()) <= 1e-6 * float(b.abs().max())
    assert torch.allclose(stats[:, 0], stats2[:, 0], rtol=2e-5)
    # payloads that are not a staged window take the other route inside the call: same result
    loose = [s.clone() for s in start]
    tc.outer_step_codes_batch(tc.TensorBatch(loose), [i.clone() for i in idxs], [c.clone() for c in codes], qps, k, lr, stats=False)
    for a, b in zip(loose, other):
        assert float((a - b).abs().max()) <= 1e-6 * float(b.abs().max())


def test_outer_step_from_codes_leaves_a_poisoned_parameter_alone(dev):
    shapes = [(128, 192), (256, 128), (64, 64)]
    k, P, lr = 64, 6, 0.3
    batch, idxs, codes, qps, fp32 = _codes_window(dev, shapes, k, P)
    # peer 2's table for parameter 1 carries an infinity (a corrupt quant_params tuple)
    sh, sc, off, lut, dt = qps[1][2]
    lut = lut.clone()
    lut[1] = float("inf")
    qps[1][2] = (sh, sc, off, lut, dt)
    fp32[2] = tc.dequantize_batch(batch, codes[2].reshape(-1), [qps[i][2] for i in range(len(shapes))], k)
    start = [torch.randn(s, device=dev) for s in shapes]
    params = [s.clone() for s in start]
    stats, skipped = tc.outer_step_codes_batch(tc.TensorBatch(params), idxs, codes, qps, k, lr)
    _check_against_oracle(batch, params, start, idxs, fp32, k, lr, stats, skipped, False, expect_skipped=[1])
    # a code past the quantiser's bins raises before anything is written
    spoiled = [c.clone() for c in codes]
    params = [s.clone() for s in start]
    stage = torch.stack([c.reshape(-1) for c in spoiled])
    stage[3, 17] = 9
    with pytest.raises(IndexError):
        tc.outer_step_codes_batch(tc.TensorBatch(params), idxs, [stage[p].view(-1, k) for p in range(P)], qps, k, lr)
    assert all(torch.equal(a, b) for a, b in zip(params, start))


def test_outer_step_seeded_sweep(dev):
    # twenty draws of shapes, peer counts, k, learning rates and layouts, each against the oracle
    rng = np.random.default_rng(2024)
    for draw in range(20):
        T = int(rng.integers(1, 5))
        shapes = [(64 * int(rng.integers(1, 5)), 64 * int(rng.integers(1, 5))) for _ in range(T)]
        P = int(rng.integers(1, 16))
        k = int(rng.choice([4, 8, 16, 32, 64]))
        lr = float(rng.choice([-1.0, 1.0]) * rng.uniform(0.01, 2.0))
        staged = bool(rng.integers(0, 2))
        batch, idxs, vals, _ = _window(dev, shapes, k, P, staged=staged)
        start = [torch.randn(s, device=dev) * float(rng.uniform(0.01, 10.0)) for s in shapes]
        params = [s.clone() for s in start]
        stats, skipped = tc.outer_step_batch(tc.TensorBatch(params), idxs, vals, k, lr)
        try:
            _check_against_oracle(batch, params, start, idxs, vals, k, lr, stats, skipped, True)
        except AssertionError as e:
            raise AssertionError(f"draw {draw}: shapes {shapes}, P {P}, k {k}, lr {lr}, staged {staged}: {e}") from e
