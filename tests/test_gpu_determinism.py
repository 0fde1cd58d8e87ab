"""Run twice, compare bytes: the whole-set encode, the 15-peer aggregate, the generic aggregate path for more
than 24 peers (floating-point atomics inside a wave's own tile), a payload with repeated indices (chunks done
again on the exact path), the clip factors from row figures and the one-launch miner step.  A result that
depended on the order in which waves or atomics happen to run would differ between two runs.  Needs an MI355X.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import templar_amd.compress as tc  # noqa: E402
import workloads  # noqa: E402


def _payloads(dev, grads, k, P, use_dct=True):
    out = []
    for p in range(P):
        own = [workloads.student_t3(tuple(g.shape), 5000 * (p + 1) + j, row_scale=True, device=dev).add_(g, alpha=0.5)
               for j, g in enumerate(grads)]
        out.append(tc.encode_compress_batch(tc.TensorBatch(own), k, use_dct=use_dct))
    return [i for i, _ in out], [v for _, v in out]


def _twice(run, outs):
    """run() writes into the tensors `outs`; both runs start from NaN-filled destinations."""
    snaps = []
    for _ in range(2):
        for o in outs:
            o.fill_(float("nan"))
        run()
        torch.cuda.synchronize()
        snaps.append([o.clone() for o in outs])
    for a, b in zip(*snaps):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), "two runs of the same launch differ"
    return snaps[0]


def test_whole_set_encode_twice(dev):
    grads = [g for g in workloads.gradient_set("cfg2_llama150m", device=dev) if g.dim() == 2]
    batch = tc.TensorBatch(grads)
    for k, use_dct in ((32, True), (64, False)):
        idx = torch.empty(batch.total_chunks * (k // 2) * 3, dtype=torch.uint8, device=dev)
        val = torch.empty((batch.total_chunks, k), device=dev)
        snaps = []
        for _ in range(2):
            idx.fill_(0xAB)
            val.fill_(float("nan"))
            tc.encode_compress_batch(batch, k, use_dct=use_dct, idx12=idx, val=val)
            torch.cuda.synchronize()
            snaps.append((idx.clone(), val.clone()))
        assert torch.equal(snaps[0][0], snaps[1][0]) and torch.equal(snaps[0][1].view(torch.int32), snaps[1][1].view(torch.int32))


@pytest.mark.parametrize("P,use_dct", [(15, True), (15, False), (30, True), (30, False), (3, True)])
def test_aggregate_twice(dev, P, use_dct):
    shapes = [(2048, 2048), (512, 1024), (64, 64), (3072, 768), (768, 3072)]
    grads = [workloads.student_t3(s, 60 + i, row_scale=True, device=dev) for i, s in enumerate(shapes)]
    k = 32
    idxs, vals = _payloads(dev, grads, k, P, use_dct)
    outs = [torch.empty_like(g) for g in grads]
    ob = tc.TensorBatch(outs)
    first = _twice(lambda: tc.batch_decompress_decode_batch(ob, idxs, vals, k, clip_norm=True, use_dct=use_dct), outs)
    assert all(torch.isfinite(o).all() for o in first)
    # the clip factors themselves, from the values and from row figures noted beforehand
    a = tc.peer_clip_scales_batch(ob, vals, k)
    b = tc.peer_clip_scales_batch(ob, vals, k)
    assert torch.equal(a, b)


@pytest.mark.parametrize("P", [4, 15, 40])
def test_aggregate_of_payloads_with_repeated_indices_twice(dev, P):
    # every fourth row of every peer names one coefficient twice: those chunks leave the fast path
    shapes = [(512, 512), (256, 1024)]
    grads = [workloads.student_t3(s, 90 + i, row_scale=True, device=dev) for i, s in enumerate(shapes)]
    k = 32
    idxs, vals = _payloads(dev, grads, k, P)
    n = sum((a // 64) * (b // 64) for a, b in shapes)
    for p in range(P):
        rows = tc.unpack_12bit_indices(idxs[p], (n, k))
        rows[::4, 1] = rows[::4, 0]
        idxs[p] = tc.pack_12bit_indices(rows.reshape(-1))
    outs = [torch.empty_like(g) for g in grads]
    ob = tc.TensorBatch(outs)
    _twice(lambda: tc.batch_decompress_decode_batch(ob, idxs, vals, k, clip_norm=True), outs)


def test_miner_step_twice(dev):
    shapes = [(1024, 2048), (512, 512), (64, 192)]
    grads = [workloads.student_t3(s, 30 + i, row_scale=True, device=dev) for i, s in enumerate(shapes)]
    ef0 = [workloads.student_t3(s, 130 + i, row_scale=True, device=dev) for i, s in enumerate(shapes)]
    gb = tc.TensorBatch(grads)
    snaps = []
    for _ in range(2):
        efs = [e.clone() for e in ef0]
        idx12, val, _ = tc.error_feedback_step_batch(tc.TensorBatch(efs), gb, 0.95, 32, use_dct=True)
        torch.cuda.synchronize()
        snaps.append((idx12.clone(), val.clone(), [e.clone() for e in efs]))
    assert torch.equal(snaps[0][0], snaps[1][0]) and torch.equal(snaps[0][1].view(torch.int32), snaps[1][1].view(torch.int32))
    assert all(torch.equal(a.view(torch.int32), b.view(torch.int32)) for a, b in zip(snaps[0][2], snaps[1][2]))


@pytest.mark.parametrize("P,k,use_dct", [(15, 32, True), (7, 16, True), (20, 32, True), (15, 32, False), (40, 32, True)])
def test_aggregate_does_not_depend_on_what_lds_held(dev, P, k, use_dct):
    """LDS keeps what the last kernel on a compute unit left.  The aggregate's fast scatter marks a slot it has
    claimed with an all-ones word, and lanes without an entry scatter to slots that are not cleared with the tile:
    if such a slot held all ones from an earlier kernel, every chunk was taken for one with a repeated index and done
    again on the exact path - the same result ten times slower.  Here every LDS word of the device is set to all
    ones (then to a NaN, then to zero) before the launch: results must be the same bits, and the launches after the
    all-ones fill must not take longer than after the zero fill."""
    from templar_amd import _lib
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    # (several chunks per wave: a wave's first chunk is scattered serially and never touches those slots)
    shapes = [(4096, 4096), (2048, 4096), (64, 64)]
    grads = [workloads.student_t3(s, 700 + i, row_scale=True, device=dev) for i, s in enumerate(shapes)]
    idxs, vals = _payloads(dev, grads, k, P, use_dct)
    outs = [torch.empty_like(g) for g in grads]
    ob = tc.TensorBatch(outs)
    scale = tc.peer_clip_scales_batch(ob, vals, k)
    run = lambda: tc.batch_decompress_decode_batch(ob, idxs, vals, k, scale=scale, use_dct=use_dct)
    snaps, times = [], {}
    for word in (0, -1, 0x7FC00000, 0):
        _lib.check(lib.tplr_debug_fill_lds(word, stream), "tplr_debug_fill_lds")
        for o in outs:
            o.fill_(float("nan"))
        run()
        torch.cuda.synchronize()
        snaps.append([o.clone() for o in outs])
        _lib.check(lib.tplr_debug_fill_lds(word, stream), "tplr_debug_fill_lds")
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(10):
            run()
        b.record()
        torch.cuda.synchronize()
        times[word] = a.elapsed_time(b)
    for s in snaps[1:]:
        for x, y in zip(snaps[0], s):
            assert torch.equal(x.view(torch.int32), y.view(torch.int32)), "the result depends on what LDS held"
    assert times[-1] < 2.0 * times[0] + 0.5, f"launches after an all-ones LDS take {times[-1]:.2f} ms against {times[0]:.2f} ms"


@pytest.mark.parametrize("k,use_dct", [(32, True), (64, True), (64, False), (8, False)])
def test_encode_and_miner_step_do_not_depend_on_what_lds_held(dev, k, use_dct):
    """The same for the send side: the staging buffer and the candidate slots of the select, and the miner step's
    tile, are written before they are read whatever LDS held."""
    from templar_amd import _lib
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    shapes = [(4096, 2048), (1024, 512), (64, 64)]
    grads = [workloads.student_t3(s, 800 + i, row_scale=True, device=dev) for i, s in enumerate(shapes)]
    batch = tc.TensorBatch(grads)
    snaps = []
    for word in (0, -1, 0x7FC00000):
        _lib.check(lib.tplr_debug_fill_lds(word, stream), "tplr_debug_fill_lds")
        idx, val = tc.encode_compress_batch(batch, k, use_dct=use_dct)
        efs = [torch.full_like(g, 0.25) for g in grads]
        _lib.check(lib.tplr_debug_fill_lds(word, stream), "tplr_debug_fill_lds")
        i2, v2, _ = tc.error_feedback_step_batch(tc.TensorBatch(efs), batch, 0.9, k, use_dct=use_dct)
        torch.cuda.synchronize()
        snaps.append([idx.clone(), val.view(torch.int32).clone(), i2.clone(), v2.view(torch.int32).clone()] +
                     [e.view(torch.int32).clone() for e in efs])
    for s in snaps[1:]:
        for x, y in zip(snaps[0], s):
            assert torch.equal(x, y), "the result depends on what LDS held"
