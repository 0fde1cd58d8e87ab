"""Full-size checks on the GPU: the 150M set (config 2), the 1B gradient set (294 144 chunks, benchmark
configurations 3 and 4) and the 72B block (config 5, k = 64, encode and 15-peer decode) through the batch
entry points of the C ABI; config 1 has a file of its own (tests/test_gpu_config1.py).

The CPU oracle cannot cover these sizes in test time, so the checks are properties that do not
depend on size (plus a strided sample that does go through the oracle):

  * selection: every row has k distinct indices < 4096, magnitudes in descending order, lowest
    index first on ties; fused encode == transform followed by select, bitwise, on the largest
    tensor; a strided sample of chunks equals the oracle's selection on the device's coefficients;
  * Parseval: the energy of the reconstruction of one payload equals the energy of its values
    (the transform is orthonormal), per chunk and in total;
  * mean of identical peers: P copies of one payload aggregate to the one-peer result (exactly
    for two peers, within a few ulp for more: sums of equal terms round);
  * linearity: the sum-mode aggregate of two different peers equals the sum of their one-peer
    decodes within fp32 tolerance;
  * round trip: encode(decode(payload)) selects the same index sets.
"""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import codec as orc  # noqa: E402  (the checker)
import templar_amd.compress as tc  # noqa: E402
import workloads  # noqa: E402

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")


def _set(name, dev):
    grads = [g for g in workloads.gradient_set(name, device=dev) if g.dim() == 2]
    return grads, workloads.CONFIGS[name]["k"]


def _check_rows(idx12, val, n, k):
    """Structure of a flat payload: distinct in-range indices, canonical order."""
    idx = tc.unpack_12bit_indices(idx12, (n, k))
    assert int(idx.max()) < 4096 and int(idx.min()) >= 0
    srt = idx.sort(dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all()), "duplicate index inside a row"
    mag = val.abs()
    assert bool((mag[:, :-1] >= mag[:, 1:]).all()), "magnitudes not descending"
    tie = mag[:, :-1] == mag[:, 1:]
    assert bool((idx[:, :-1][tie] < idx[:, 1:][tie]).all()), "ties not in index order"
    return idx


@pytest.mark.parametrize("name", ["cfg2_llama150m", "cfg3_llama1b", "cfg5_72b_block"])
def test_full_set_encode_properties(dev, name):
    grads, k = _set(name, dev)
    batch = tc.TensorBatch(grads)
    n = batch.total_chunks
    idx12, val = tc.encode_compress_batch(batch, k, use_dct=True)
    assert idx12.numel() == n * k * 3 // 2 and val.shape == (n, k)
    idx = _check_rows(idx12, val, n, k)

    # fused == transform then select, bitwise, on the largest tensor of the set
    big = max(range(len(grads)), key=lambda i: grads[i].numel())
    x = grads[big]

    class M:
        def named_parameters(self):
            from types import SimpleNamespace
            yield "w", SimpleNamespace(requires_grad=True, shape=tuple(x.shape), dtype=torch.float32, device=dev)

    tr = tc.ChunkingTransformer(M(), 64)
    coef = tr.encode(x, use_dct=True).reshape(-1, 4096)
    i_u, v_u = tc._topk_rows(coef, k)
    i_f, v_f = batch.payload_slice(big, idx12, val, k)
    assert torch.equal(i_f, i_u) and torch.equal(v_f.reshape(-1, k), v_u)

    # a strided sample of that tensor's chunks against the oracle's selection
    step = max(1, coef.shape[0] // 64)
    rows = coef[::step].cpu().numpy()
    want_i, want_v = orc.topk_rows(rows, k)
    b0 = batch.offsets[big]
    assert np.array_equal(idx[b0:b0 + coef.shape[0]][::step].cpu().numpy(), want_i)
    assert np.array_equal(v_u[::step].cpu().numpy(), want_v)
    # the selection is a top-k: nothing left out is larger than the smallest value kept
    kept = torch.zeros_like(coef, dtype=torch.bool).scatter_(1, idx[b0:b0 + coef.shape[0]], True)
    left = coef.abs().masked_fill(kept, 0.0).max(dim=1).values
    assert bool((left <= v_u.abs().min(dim=1).values).all())
    # transform tolerance on the sample, against the oracle's closed-form transform
    y, xx = x.shape[0] // 64, x.shape[1] // 64
    for g in range(0, coef.shape[0], step * 8):
        cy, cx = divmod(g, xx)
        blk = x[cy * 64:(cy + 1) * 64, cx * 64:(cx + 1) * 64].cpu().numpy()
        want = orc.encode2d(blk).reshape(-1)
        assert np.abs(coef[g].cpu().numpy() - want).max() <= TOL * np.abs(want).max()


def test_full_set_aggregate_properties(dev):
    grads, k = _set("cfg3_llama1b", dev)
    batch = tc.TensorBatch(grads)
    n = batch.total_chunks
    idx_a, val_a = tc.encode_compress_batch(batch, k, use_dct=True)
    # a second, different payload on the same shapes
    others = [workloads.student_t3(tuple(g.shape), 7000 + j, row_scale=True, device=dev) for j, g in enumerate(grads)]
    idx_b, val_b = tc.encode_compress_batch(tc.TensorBatch(others), k, use_dct=True)
    del others
    outs = [torch.empty_like(g) for g in grads]
    ob = tc.TensorBatch(outs)

    # one peer, no clip: Parseval per chunk and in total
    ss = torch.empty(n, device=dev)
    tc.batch_decompress_decode_batch(ob, [idx_a], [val_a], k, clip_norm=False, sumsq=ss)
    one = [o.clone() for o in outs]
    e_val = (val_a.double() ** 2).sum(dim=1)
    assert torch.allclose(ss.double(), e_val, rtol=1e-4, atol=1e-30)
    e_out = sum(float((o.double() ** 2).sum()) for o in one)
    assert abs(e_out - float(e_val.sum())) <= 1e-5 * float(e_val.sum())

    # P identical peers: the mean is the one-peer result (x + x halves back exactly; longer sums of
    # equal terms round, so 8 and 15 peers are held to a few ulp)
    for P in (2, 8, 15):
        tc.batch_decompress_decode_batch(ob, [idx_a] * P, [val_a] * P, k, clip_norm=False)
        for o, w in zip(outs, one):
            if P == 2:
                assert torch.equal(o, w)
            else:
                assert float((o - w).abs().max()) <= 1e-6 * float(w.abs().max()), f"P={P}"

    # clip factors of identical peers are min(1, n / (n + 1e-8)): 1 to within an ulp
    tc.batch_decompress_decode_batch(ob, [idx_a] * 4, [val_a] * 4, k, clip_norm=True)
    for o, w in zip(outs, one):
        assert float((o - w).abs().max()) <= 1e-6 * float(w.abs().max())

    # sum mode is linear: aggregate(a, b) == decode(a) + decode(b)
    tc.batch_decompress_decode_batch(ob, [idx_b], [val_b], k, clip_norm=False)
    two = [o.clone() for o in outs]
    tc.batch_decompress_decode_batch(ob, [idx_a, idx_b], [val_a, val_b], k, clip_norm=False, mean=False)
    for o, a, b in zip(outs, one, two):
        ref = a + b
        assert float((o - ref).abs().max()) <= TOL * float(ref.abs().max())

    # round trip: the reconstruction of a payload encodes to the same index sets
    idx_r, val_r = tc.encode_compress_batch(tc.TensorBatch(one), k, use_dct=True)
    ia = tc.unpack_12bit_indices(idx_a, (n, k)).sort(dim=1).values
    ir = tc.unpack_12bit_indices(idx_r, (n, k)).sort(dim=1).values
    same = (ia == ir).all(dim=1)
    # a row may differ only where the k-th and a dropped coefficient (a rounding-level zero) tie
    assert float(same.float().mean()) > 0.999
    assert float((val_r.abs().sum(dim=1) - val_a.abs().sum(dim=1)).abs().max()) <= 1e-4 * float(val_a.abs().sum(dim=1).max())


def test_full_set_error_feedback_step(dev):
    """src/tplr/neurons.py:147-171 over the whole 1B set in two launches.  Properties: the
    payload is that of the accumulated momentum (ef * decay + grad, bit-exact); what is left
    behind has (numerically) nothing at the sent coefficients and everything else untouched;
    energy splits between the payload and the remainder (Parseval)."""
    grads, k = _set("cfg3_llama1b", dev)
    efs = [workloads.student_t3(tuple(g.shape), 9000 + j, row_scale=True, device=dev) for j, g in enumerate(grads)]
    acc = [e * 0.95 + g for e, g in zip(efs, grads)]  # mul then add, as the reference does in place
    eb, gb = tc.TensorBatch(efs), tc.TensorBatch(grads)
    n = eb.total_chunks
    idx12, val, quant = tc.error_feedback_step_batch(eb, gb, 0.95, k, use_dct=True)
    assert quant is None
    want_i, want_v = tc.encode_compress_batch(tc.TensorBatch(acc), k, use_dct=True)
    assert torch.equal(idx12, want_i) and torch.equal(val, want_v)
    # energy: |acc|^2 = |payload|^2 + |remainder|^2 for an orthonormal transform
    e_acc = sum(float((a.double() ** 2).sum()) for a in acc)
    e_rem = sum(float((e.double() ** 2).sum()) for e in efs)
    e_pay = float((val.double() ** 2).sum())
    assert abs(e_acc - e_pay - e_rem) <= 1e-5 * e_acc
    # the remainder's coefficients: ~0 where sent, unchanged elsewhere (checked on the largest tensor)
    big = max(range(len(efs)), key=lambda i: efs[i].numel())

    class M:
        def named_parameters(self):
            from types import SimpleNamespace
            yield "w", SimpleNamespace(requires_grad=True, shape=tuple(efs[big].shape), dtype=torch.float32, device=dev)

    tr = tc.ChunkingTransformer(M(), 64)
    c_rem = tr.encode(efs[big], use_dct=True).reshape(-1, 4096)
    c_acc = tr.encode(acc[big], use_dct=True).reshape(-1, 4096)
    i_big, _ = eb.payload_slice(big, idx12, val, k)
    idx = tc.unpack_12bit_indices(i_big, (c_rem.shape[0], k))
    sent = torch.zeros_like(c_rem, dtype=torch.bool).scatter_(1, idx, True)
    top = float(c_acc.abs().max())
    assert float(c_rem[sent].abs().max()) <= TOL * top
    assert float((c_rem - c_acc)[~sent].abs().max()) <= TOL * top
    # without the transform the sent entries are removed exactly
    efs2 = [workloads.student_t3(tuple(g.shape), 9000 + j, row_scale=True, device=dev) for j, g in enumerate(grads[:8])]
    acc2 = [e * 0.95 + g for e, g in zip(efs2, grads[:8])]
    eb2 = tc.TensorBatch(efs2)
    i2, v2, _ = tc.error_feedback_step_batch(eb2, tc.TensorBatch(grads[:8]), 0.95, k, use_dct=False)
    for j, (e, a) in enumerate(zip(efs2, acc2)):
        ij, vj = eb2.payload_slice(j, i2, v2, k)
        y, x = a.shape[0] // 64, a.shape[1] // 64
        ch = a.reshape(y, 64, x, 64).permute(0, 2, 1, 3).reshape(y * x, 4096)
        ix = tc.unpack_12bit_indices(ij, (y * x, k))
        assert torch.equal(ch.gather(1, ix), vj.reshape(y * x, k))
        want = ch.scatter(1, ix, 0.0).reshape(y, x, 64, 64).permute(0, 2, 1, 3).reshape(a.shape)
        assert torch.equal(e, want)



@pytest.mark.parametrize("use_dct", [True, False])
def test_full_set_evaluation_update_properties(dev, use_dct):
    # neurons/validator.py:3595-3737 on the 1B set: p <- p - alpha * decode(decompress(vals * clip)), one launch.
    # Linearity gives size-independent checks: the update equals p - alpha * (the one-peer decode with the same clip
    # factors) within fp32 tolerance, and applying it again with -alpha brings the parameters back.
    grads, k = _set("cfg3_llama1b", dev)
    batch = tc.TensorBatch(grads)
    idx12, val = tc.encode_compress_batch(batch, k, use_dct=use_dct)
    del grads, batch
    gen = torch.Generator(device=dev).manual_seed(11)
    shapes = [tuple(s) for s in workloads.CONFIGS["cfg3_llama1b"]["shapes"] if len(s) == 2]
    params = [torch.randn(s, device=dev, generator=gen) * 0.02 for s in shapes]
    start = [p.clone() for p in params]
    pb = tc.TensorBatch(params)
    T = len(params)
    clip = torch.rand(T, device=dev, generator=gen) * 0.9 + 0.1
    alpha = 0.37
    tc.apply_decoded_batch(pb, idx12, val, k, alpha=alpha, clip=clip, use_dct=use_dct)
    dense = [torch.empty(s, device=dev) for s in shapes]
    tc.batch_decompress_decode_batch(tc.TensorBatch(dense), [idx12], [val], k, scale=clip.reshape(T, 1).contiguous(),
                                     use_dct=use_dct)
    worst = 0.0
    for p, p0, d in zip(params, start, dense):
        want = p0 - alpha * d
        worst = max(worst, float((p - want).abs().max()) / max(1e-30, float(want.abs().max())))
    assert worst <= TOL
    del dense
    tc.apply_decoded_batch(pb, idx12, val, k, alpha=-alpha, clip=clip, use_dct=use_dct)
    back = max(float((p - p0).abs().max()) / float(p0.abs().max()) for p, p0 in zip(params, start))
    assert back <= TOL
    if not use_dct:
        # without the transform only the k named positions of a chunk change
        tc.apply_decoded_batch(pb, idx12, val, k, alpha=alpha, clip=clip, use_dct=False)
        changed = sum(int((p != p0).sum()) for p, p0 in zip(params, start))
        assert changed <= pb.total_chunks * k


@pytest.mark.parametrize("P,k", [(20, 64), (15, 32), (12, 64)])
def test_full_size_index_statistics_against_bitmaps(dev, P, k):
    # the 1B set's 294 144 rows: every wave walks 144 rows, so the per-lane bit-plane counters are
    # summed in mid-run and at tensor boundaries.  Reference: one 4096-bit membership map per peer
    # and row built with torch.scatter_, shared entries = map_j gathered at peer i's indices.
    shapes = [s for s in workloads.CONFIGS["cfg3_llama1b"]["shapes"] if len(s) == 2]
    counts = [(a // 64) * (b // 64) for a, b in shapes]
    n = sum(counts)
    g = torch.Generator(device=dev)
    g.manual_seed(100 * P + k)
    base = torch.rand((n, 4096), device=dev, generator=g).topk(k, dim=-1).indices
    rows, packed = [], []
    for p in range(P):
        own = torch.rand((n, 4096), device=dev, generator=g).topk(k, dim=-1).indices
        # a varying share of `base`, column by column; entries repeated inside a row are allowed here
        # (both counts treat them alike: every copy in peer i counts, the other peer's set does not grow)
        keep = torch.rand((n, k), device=dev, generator=g) < (0.1 + 0.04 * p)
        r = torch.where(keep, base, own)
        rows.append(r)
        packed.append(tc.pack_12bit_indices(r.contiguous()))
        del own, keep
    pair, dup, top = tc.index_stats_batch(counts, packed, k)
    bounds = np.cumsum([0] + counts)
    seg = torch.zeros(n, dtype=torch.int64, device=dev)
    for t in range(len(counts)):
        seg[bounds[t]:bounds[t + 1]] = t
    maps = []
    for p in range(P):
        m = torch.zeros((n, 4096), dtype=torch.bool, device=dev)
        m.scatter_(1, rows[p], True)
        maps.append(m)
    want = torch.zeros((len(counts), P, P), dtype=torch.int64, device=dev)
    for i in range(P):
        for j in range(i + 1, P):
            per_row = maps[j].gather(1, rows[i]).sum(dim=1)
            want[:, i, j].index_add_(0, seg, per_row)
    assert torch.equal(torch.triu(pair, 1), want)
    for p in range(P):
        distinct = maps[p].sum(dim=1)
        want_dup = torch.zeros(len(counts), dtype=torch.int64, device=dev).index_add_(0, seg, k - distinct)
        assert torch.equal(dup[:, p], want_dup)
        want_top = torch.stack([rows[p][bounds[t]:bounds[t + 1]].max() for t in range(len(counts))])
        assert torch.equal(top[:, p].long(), want_top)


@pytest.mark.parametrize("name,use_dct,P,k", [("cfg3_llama1b", False, 15, 32), ("cfg3_llama1b", True, 15, 32),
                                              ("cfg3_llama1b", False, 20, 64), ("cfg3_llama1b", True, 20, 64),
                                              ("cfg3_llama1b", True, 31, 32), ("cfg2_llama150m", True, 15, 32),
                                              ("cfg2_llama150m", False, 15, 32), ("cfg5_72b_block", True, 15, 64)])
def test_full_set_aggregate_against_torch_scatter_reduce(dev, name, use_dct, P, k):
    # a whole set (the 1B set, the 150M set, the 72B block on its own shapes), every chunk: torch's own
    # scatter_reduce_(mean, include_self=False) on the concatenated payloads (the reference's op sequence,
    # src/tplr/compress.py:559-580, run on the GPU), then its einsum decode, against the one-launch aggregate
    from oracle import torch_cpu_path as tcp

    shapes = [s for s in workloads.CONFIGS[name]["shapes"] if len(s) == 2]
    counts = [(a // 64) * (b // 64) for a, b in shapes]
    n = sum(counts)
    g = torch.Generator(device=dev)
    g.manual_seed(4242 + P + k)
    base = torch.rand((n, 4096), device=dev, generator=g).topk(k, dim=-1).indices
    rows, packed, vals = [], [], []
    for p in range(P):
        own = torch.rand((n, 4096), device=dev, generator=g).topk(k, dim=-1).indices
        r = own.clone()
        r[:, : 4 + p] = base[:, : 4 + p]  # the peers agree on a growing part of every row ...
        clash = (r[:, 4 + p:, None] == base[:, None, : 4 + p]).any(-1)  # ... and must not repeat it in the rest
        keep_rows = ~clash.any(dim=1)  # rows whose own part repeats a shared index fall back to `own`
        r = torch.where(keep_rows[:, None], r, own)
        rows.append(r)
        packed.append(tc.pack_12bit_indices(r.contiguous()))
        vals.append(torch.randn((n, k), device=dev, generator=g) * (1 + p))
        del own, clash
    scale = torch.rand((len(shapes), P), device=dev, generator=g) * 0.5 + 0.5
    outs = [torch.full(s, float("nan"), device=dev) for s in shapes]
    tc.batch_decompress_decode_batch(tc.TensorBatch(outs), packed, vals, k, scale=scale, use_dct=use_dct)
    _, b = tcp.basis(64)
    b = b.to(dev)
    begin = 0
    worst = 0.0
    for t, (shape, cnt) in enumerate(zip(shapes, counts)):
        sl = slice(begin, begin + cnt)
        idx = torch.cat([r[sl] for r in rows], dim=1)
        val = torch.cat([vals[p][sl] * scale[t, p] for p in range(P)], dim=1)
        dense = torch.zeros((cnt, 4096), device=dev).scatter_reduce_(1, idx, val, reduce="mean", include_self=False)
        Y, X = shape[0] // 64, shape[1] // 64
        want = tcp.decode(dense.reshape(Y, X, 64, 64), b, b, use_dct=use_dct)
        err = (outs[t] - want).abs().max().item() / want.abs().max().item()
        worst = max(worst, err)
        assert err <= (TOL if use_dct else 2e-6), (t, shape, err)
        if not use_dct:
            # elements no peer sent are exactly zero (torch adds with atomics in no fixed order, so an
            # element whose contributions cancel may come out as 0 there and as a last-bit residue
            # here, or the other way round: the pattern is taken from the indices, not from the values)
            sent = torch.zeros((cnt, 4096), dtype=torch.bool, device=dev).scatter_(1, idx, True)
            sent = sent.reshape(Y, X, 64, 64).permute(0, 2, 1, 3).reshape(Y * 64, X * 64)
            assert float(outs[t][~sent].abs().max()) == 0.0
        begin += cnt
    assert worst > 0.0 or not use_dct


@pytest.mark.parametrize("name", ["cfg3_llama1b", "cfg2_llama150m", "cfg5_72b_block"])
def test_full_set_transform_and_selection_against_torch(dev, name):
    # every tensor of a set: the chunked transform against torch's einsum with the reference's
    # FFT-built basis (the reference's op sequence on the GPU), and the fused kernel's payload against
    # torch.topk on this library's own coefficients - magnitudes bit for bit, values gathered at the
    # selected indices bit for bit
    from oracle import torch_cpu_path as tcp

    grads, k = _set(name, dev)
    batch = tc.TensorBatch(grads)
    idx12, val = tc.encode_compress_batch(batch, k, use_dct=True)
    f, _ = tcp.basis(64)
    f = f.to(dev)
    worst = 0.0
    for i, x in enumerate(grads):
        class M:
            def named_parameters(self):
                from types import SimpleNamespace
                yield "w", SimpleNamespace(requires_grad=True, shape=tuple(x.shape), dtype=torch.float32, device=dev)

        coef = tc.ChunkingTransformer(M(), 64).encode(x, use_dct=True)
        ref = tcp.encode(x, 64, 64, f, f)
        err = (coef - ref).abs().max().item() / ref.abs().max().item()
        worst = max(worst, err)
        assert err <= TOL, (i, tuple(x.shape), err)
        rows = coef.reshape(-1, 4096)
        pi, pv = batch.payload_slice(i, idx12, val, k)
        pv = pv.reshape(-1, k)
        sel = tc.unpack_12bit_indices(pi, pv.shape)
        assert torch.equal(rows.gather(1, sel), pv)
        top = torch.topk(rows.abs(), k, dim=1, largest=True, sorted=True).values
        assert torch.equal(top, pv.abs())
    assert worst > 0.0


def _random_payloads(dev, n, P, k, seed):
    """P peers' flat payloads of n rows: k distinct indices per row, normal values growing with the peer."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    packed, vals = [], []
    for p in range(P):
        sel = torch.rand((n, 4096), device=dev, generator=g).topk(k, dim=-1).indices
        packed.append(tc.pack_12bit_indices(sel.contiguous()))
        vals.append(torch.randn((n, k), device=dev, generator=g) * (1 + p))
        del sel
    return packed, vals


def test_full_set_aggregate_from_four_bin_codes(dev):
    # templar's own settings on the 1B shapes (20 peers, k = 64, no transform, 4-bin quantiser), every chunk:
    # the aggregate straight from the codes of a staged window (wide loads) is bitwise the fp32 aggregate of the
    # de-quantised values with the same factors, and the whole call (norms from counts) agrees with de-quantise,
    # norms, aggregate within rounding of the clip factors
    P, k = 20, 64
    shapes = [s for s in workloads.CONFIGS["cfg3_llama1b"]["shapes"] if len(s) == 2]
    n = sum((a // 64) * (b // 64) for a, b in shapes)
    T = len(shapes)
    outs = [torch.empty(s, device=dev) for s in shapes]
    batch = tc.TensorBatch(outs)
    packed, vals = _random_payloads(dev, n, P, k, 99)
    ibuf = torch.stack(packed)
    cbuf = torch.empty((P, n, k), dtype=torch.uint8, device=dev)
    qps = [[None] * P for _ in range(T)]
    fp32 = []
    for p in range(P):
        c, shift, scale, lookup = tc.quantize_batch(batch, vals[p], k, 4, 6.0)
        cbuf[p].copy_(c)
        fp32.append(tc.dequantize_batch(batch, c.reshape(-1), None, k, tables=(lookup, shift)))
        for i in range(T):
            qps[i][p] = (shift[i], 1.0, 2, lookup[i], torch.float32)
    del vals, packed
    idxs, codes = [ibuf[p] for p in range(P)], [cbuf[p] for p in range(P)]
    tables = tc.dequantised_tables(qps, dev)
    want = [torch.empty(s, device=dev) for s in shapes]
    tc.batch_decompress_decode_codes_batch(batch, idxs, codes, qps, k, tables=tables)
    tc.batch_decompress_decode_batch(tc.TensorBatch(want), idxs, fp32, k, use_dct=False)
    for t, (a, b) in enumerate(zip(outs, want)):
        assert float((a - b).abs().max()) <= 1e-6 * float(b.abs().max()), t
    # fixed factors: bit for bit
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    scale = torch.rand((T, P), device=dev, generator=g) * 0.5 + 0.5
    import ctypes as C
    from templar_amd import _lib
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    cp = (C.c_void_p * P)(*[c.data_ptr() for c in codes])
    st = _lib.load().tplr_decode_aggregate_codes_batch(ip, cp, tables[0].data_ptr(), scale.data_ptr(), P, k,
                                                       batch.table.data_ptr(), T, n, _lib.REDUCE_MEAN, None, None)
    assert st == 0
    tc.batch_decompress_decode_batch(tc.TensorBatch(want), idxs, fp32, k, scale=scale, use_dct=False)
    for t, (a, b) in enumerate(zip(outs, want)):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), t


def test_full_set_normalised_mean_and_result_statistics(dev):
    # the 1B shapes, 15 peers, k = 32: the per-tensor norms taken from the payloads before the one aggregate launch
    # (orthonormal transform) give the tensors the literal order gives (aggregate, norms of the dense result,
    # scaling pass), every tensor of unit norm; and the statistics the aggregate leaves on its way are those of
    # the tensors it wrote
    P, k = 15, 32
    shapes = [s for s in workloads.CONFIGS["cfg3_llama1b"]["shapes"] if len(s) == 2]
    n = sum((a // 64) * (b // 64) for a, b in shapes)
    packed, vals = _random_payloads(dev, n, P, k, 123)
    one = [torch.empty(s, device=dev) for s in shapes]
    two = [torch.empty(s, device=dev) for s in shapes]
    f1 = tc.aggregate_mean_normalised_batch(tc.TensorBatch(one), packed, vals, k)
    f2 = tc.aggregate_mean_normalised_batch(tc.TensorBatch(two), packed, vals, k, two_pass=True)
    assert float(((f1 - f2).abs() / f2).max()) <= 1e-5
    for t, (a, b) in enumerate(zip(one, two)):
        assert float((a - b).abs().max()) <= TOL * float(b.abs().max()), t
        assert abs(float(torch.linalg.vector_norm(a.double())) - 1.0) <= 1e-5, t
    del two
    stats = tc.batch_decompress_decode_batch(tc.TensorBatch(one), packed, vals, k, stats=True)
    for t, a in enumerate(one):
        d = a.double()
        assert abs(float(stats[t, 0]) - float(torch.linalg.vector_norm(d))) <= 1e-5 * float(torch.linalg.vector_norm(d)), t
        assert abs(float(stats[t, 1]) - float(d.mean())) <= 1e-5 * float(d.abs().mean()), t
        assert float(stats[t, 2]) == 1.0


@pytest.mark.parametrize("P,k,chunks_y", [(20, 64, 70), (15, 32, 50), (7, 64, 33), (24, 32, 97)])
def test_codes_aggregate_wave_ranges_of_a_few_chunks(dev, P, k, chunks_y):
    # between the unit-test sizes (at most one chunk per wave) and the full sets (hundreds): wave ranges of one
    # to five chunks, where the pipeline's prologue, its two register sets and its tail all meet - the codes
    # aggregate of a staged window (wide loads) bit for bit against the fp32 aggregate of the de-quantised values
    import ctypes as C
    from templar_amd import _lib
    shapes = [(chunks_y * 64, 128 * 64), (64, 64), (3 * 64, 5 * 64)]
    T = len(shapes)
    n = sum((a // 64) * (b // 64) for a, b in shapes)
    outs = [torch.empty(s, device=dev) for s in shapes]
    want = [torch.empty(s, device=dev) for s in shapes]
    batch = tc.TensorBatch(outs)
    packed, vals = _random_payloads(dev, n, P, k, 1000 + P + k)
    ibuf, cbuf = torch.stack(packed), torch.empty((P, n, k), dtype=torch.uint8, device=dev)
    qps = [[None] * P for _ in range(T)]
    fp32 = []
    for p in range(P):
        c, shift, scale, lookup = tc.quantize_batch(batch, vals[p], k, 4, 6.0)
        cbuf[p].copy_(c)
        fp32.append(tc.dequantize_batch(batch, c.reshape(-1), None, k, tables=(lookup, shift)))
        for i in range(T):
            qps[i][p] = (shift[i], 1.0, 2, lookup[i], torch.float32)
    idxs, codes = [ibuf[p] for p in range(P)], [cbuf[p] for p in range(P)]
    deq, _ = tc.dequantised_tables(qps, dev)
    g = torch.Generator(device=dev)
    g.manual_seed(P)
    scale = torch.rand((T, P), device=dev, generator=g) * 0.5 + 0.5
    ip = (C.c_void_p * P)(*[i.data_ptr() for i in idxs])
    cp = (C.c_void_p * P)(*[c.data_ptr() for c in codes])
    for mode in (_lib.REDUCE_MEAN, _lib.REDUCE_SUM):
        for o in outs:
            o.fill_(float("nan"))
        st = _lib.load().tplr_decode_aggregate_codes_batch(ip, cp, deq.data_ptr(), scale.data_ptr(), P, k,
                                                           batch.table.data_ptr(), T, n, mode, None, None)
        assert st == 0
        tc.batch_decompress_decode_batch(tc.TensorBatch(want), idxs, fp32, k, scale=scale, use_dct=False,
                                         mean=mode == _lib.REDUCE_MEAN)
        for t, (a, b) in enumerate(zip(outs, want)):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (mode, t)


def test_codes_aggregate_seeded_sweep(dev):
    # forty seeded draws of (peers, k, bins, set of shapes, staged or separately allocated payloads): the aggregate
    # from codes bit for bit against the fp32 aggregate of the de-quantised values, both reduce modes; and the sums
    # of squares from the payloads against those of the dense sum-mode coefficients
    import ctypes as C
    from templar_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(20251)
    for draw in range(40):
        P = int(rng.integers(1, 25))
        k = int(rng.choice([4, 8, 16, 32, 64]))
        bins = int(rng.choice([2, 3, 4]))
        staged = bool(rng.integers(0, 2))
        shapes = [(int(rng.integers(1, 40)) * 64, int(rng.integers(1, 40)) * 64) for _ in range(int(rng.integers(1, 4)))]
        T = len(shapes)
        n = sum((a // 64) * (b // 64) for a, b in shapes)
        outs = [torch.empty(s, device=dev) for s in shapes]
        want = [torch.empty(s, device=dev) for s in shapes]
        batch = tc.TensorBatch(outs)
        packed, vals = _random_payloads(dev, n, P, k, 7000 + draw)
        qps = [[None] * P for _ in range(T)]
        fp32, codes = [], []
        for p in range(P):
            c, shift, scale, lookup = tc.quantize_batch(batch, vals[p], k, bins, 6.0)
            codes.append(c)
            fp32.append(tc.dequantize_batch(batch, c.reshape(-1), None, k, tables=(lookup, shift)))
            for i in range(T):
                qps[i][p] = (shift[i], 1.0, bins // 2, lookup[i], torch.float32)
        if staged:
            ibuf, cbuf = torch.stack(packed), torch.stack(codes)
            packed, codes = [ibuf[p] for p in range(P)], [cbuf[p] for p in range(P)]
        deq, _ = tc.dequantised_tables(qps, dev)
        g = torch.Generator(device=dev)
        g.manual_seed(draw)
        scale = torch.rand((T, P), device=dev, generator=g) * 0.5 + 0.5
        ip = (C.c_void_p * P)(*[i.data_ptr() for i in packed])
        cp = (C.c_void_p * P)(*[c.data_ptr() for c in codes])
        for mode in (_lib.REDUCE_MEAN, _lib.REDUCE_SUM):
            for o in outs:
                o.fill_(float("nan"))
            st = lib.tplr_decode_aggregate_codes_batch(ip, cp, deq.data_ptr(), scale.data_ptr(), P, k,
                                                       batch.table.data_ptr(), T, n, mode, None, None)
            assert st == 0, (draw, st)
            tc.batch_decompress_decode_batch(tc.TensorBatch(want), packed, fp32, k, scale=scale, use_dct=False,
                                             mean=mode == _lib.REDUCE_MEAN)
            for t, (a, b) in enumerate(zip(outs, want)):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (draw, P, k, bins, staged, mode, t)
        # `want` now holds the sum-mode coefficients (no transform): their sums of squares per chunk
        ss = torch.empty(n, device=dev)
        vp = (C.c_void_p * P)(*[v.data_ptr() for v in fp32])
        assert lib.tplr_aggregate_sumsq_batch(ip, vp, scale.data_ptr(), P, k, batch.table.data_ptr(), T, n,
                                              ss.data_ptr(), None) == 0
        b0 = 0
        for t, s in enumerate(shapes):
            Y, X = s[0] // 64, s[1] // 64
            d = want[t].double().reshape(Y, 64, X, 64).permute(0, 2, 1, 3).reshape(Y * X, 4096)
            ref = (d * d).sum(dim=1)
            got = ss[b0:b0 + Y * X].double()
            assert float((got - ref).abs().max()) <= 1e-5 * float(ref.max()), (draw, t)
            b0 += Y * X


def test_full_set_outer_step_properties(dev):
    # the 1B set, 15 peers: p <- p - lr * decode(aggregate) in one launch equals the aggregate written as dense
    # gradients followed by the subtraction (every element, fp32 tolerance), its statistics are those of the
    # aggregate launch, the opposite sign takes the step back, and a poisoned parameter keeps its bits while the
    # others take their step
    grads, k = _set("cfg3_llama1b", dev)
    P, lr = 15, 0.4
    batch = tc.TensorBatch(grads)
    stage = tc.PayloadStage(batch, k, P, quantized=False)
    idxs, vals = [], []
    for p in range(P):
        own = [workloads.student_t3(tuple(g.shape), 1000 * (p + 1) + j, row_scale=True, device=dev).add_(g, alpha=0.5)
               for j, g in enumerate(grads)]
        i12, v = stage.regions(p)
        tc.encode_compress_batch(tc.TensorBatch(own), k, idx12=i12, val=v)
        idxs.append(i12)
        vals.append(v)
        del own
    shapes = [tuple(g.shape) for g in grads]
    scale = tc.peer_clip_scales_batch(batch, vals, k)
    ref_stats = tc.batch_decompress_decode_batch(batch, idxs, vals, k, scale=scale, stats=True)   # dense gradients in `grads`
    gen = torch.Generator(device=dev).manual_seed(5)
    params = [torch.randn(s, device=dev, generator=gen) * 0.02 for s in shapes]
    pb = tc.TensorBatch(params)
    start3 = params[3].clone()
    stats, skipped = tc.outer_step_batch(pb, idxs, vals, k, lr, scale=scale)
    assert skipped == []
    gen = torch.Generator(device=dev).manual_seed(5)
    worst = 0.0
    for p, g, s in zip(params, grads, shapes):
        want = torch.randn(s, device=dev, generator=gen) * 0.02 - lr * g
        worst = max(worst, float((p - want).abs().max()) / float(want.abs().max()))
    assert worst <= TOL
    assert torch.allclose(stats[:, 0], ref_stats[:, 0], rtol=2e-5) and torch.equal(stats[:, 2], ref_stats[:, 2])
    assert torch.allclose(stats[:, 1], ref_stats[:, 1], rtol=1e-3, atol=1e-9)
    tc.outer_step_batch(pb, idxs, vals, k, -lr, scale=scale, stats=False)
    gen = torch.Generator(device=dev).manual_seed(5)
    back = 0.0
    for p, s in zip(params, shapes):
        p0 = torch.randn(s, device=dev, generator=gen) * 0.02
        back = max(back, float((p - p0).abs().max()) / float(p0.abs().max()))
    assert back <= TOL
    # one NaN in one peer's values of parameter 3
    keep = [p.clone() if i in (2, 3, 4) else None for i, p in enumerate(params)]
    vals[7][batch.offsets[3] + 11, 5] = float("nan")
    stats, skipped = tc.outer_step_batch(pb, idxs, vals, k, lr)
    assert skipped == [3] and float(stats[3, 2]) == 0.0
    assert torch.equal(params[3].view(torch.int32), keep[3].view(torch.int32))
    assert not torch.equal(params[2], keep[2]) and not torch.equal(params[4], keep[4])
    assert all(bool(torch.isfinite(p).all()) for p in params)
    del start3
