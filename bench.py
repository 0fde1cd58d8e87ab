#!/usr/bin/env python3
"""Benchmark of the gradient-codec hot path on one MI355X.

Workload (benchmark configurations 3 and 4): the LLaMA-style 1B gradient set
(16 layers, hidden 2048, intermediate 8192, vocab 32000; 115 two-dimensional tensors =
294 144 chunks of 64x64, plus 33 norm vectors), synthetic Student-t(df=3) x 1e-3 gradients
with log-normal row scales, chunk 64, top-k 32.

  step       = one encode + top-k + pack pass over the whole set (one fused launch for all
               2-D tensors, one more for all the norm vectors, each read where it is allocated);
               the same step is first repeated untimed for SETTLE_S seconds, then come the W
               warm-up steps and the K timed ones
  value      = algorithmic bytes of that pass / time, in GB/s (inputs resident in HBM)
  aggregate  = one 15-peer decode-aggregate pass over the same shapes (per-tensor, per-peer
               norms and clip factors, then one fused unpack + scatter-mean + inverse DCT launch),
               reported as ms and GB/s
  roofline   = the same figures against the 8 TB/s HBM peak, per kernel, from HIP events on
               the launch stream
  cpu_baseline = the reference's op sequence in torch on the host cores (oracle port), timed
               on a bounded sample of the same workload

Prints one JSON line.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

def measured_traffic(workload, k, use_dct, peers, kernel):
    """HBM bytes per launch of a whole-set kernel from hardware counters (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
    runs of `bench.py --profile ...`, scaled by the library's calibration copy): read from profiles/traffic.json,
    which `bench_profiles.py summarise` writes beside the summaries that give the commands.  None for a launch
    that has no entry there."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        return None
    from bench_profiles import traffic_key

    return table.get(traffic_key(workload, k, use_dct, peers, kernel))


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg3_llama1b", help="cfg1_2048x2048 | cfg2_llama150m | cfg3_llama1b | cfg5_72b_block")
    ap.add_argument("--peers", type=int, default=15)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--topk", type=int, default=0, help="top-k per chunk instead of the workload's own (templar runs 64)")
    ap.add_argument("--no-dct", action="store_true", help="chunks are selected and scattered untransformed (templar's use_dct=false)")
    ap.add_argument("--profile", choices=["encode", "aggregate", "miner", "copy", "calib", "fill", "read", "linfill", "outer"], default=None,
                    help="run only that phase's batched launches --steps times (for rocprofv3) and print nothing; "
                         "'copy' runs the library's calibration copy of 1 GiB instead (counter scaling); 'calib' / 'fill' "
                         "run the memory-only form of the aggregate kernel with / without its payload loads, 'read' the "
                         "memory-only form of the encode kernel, 'linfill' a fill of the aggregate's output bytes over a "
                         "linear address range (library kernel, then torch's fill_ and copy_ of the same size)")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="rough budget for the CPU baseline sample")
    return ap.parse_args()


SETTLE_S = 0.25  # see event_ms


def event_ms(fn, steps, warmup, settle=False):
    """`warmup` untimed calls, then exactly `steps` calls between two events on the current stream:
    (mean ms per call from the events, mean wall ms per call).  settle: the calls are first repeated,
    untimed, for SETTLE_S seconds - the clock governor of the device needs a few hundred launches after
    an idle spell (input generation, host work) to leave its idle clocks, far more than a warm-up of a
    handful of calls gives it, and a codec that runs every window runs at the settled clocks."""
    import torch

    if settle:
        t_end = time.perf_counter() + SETTLE_S
        while time.perf_counter() < t_end:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall


def launch_stats(fn, steps):
    """Per-call durations of `steps` further calls, each between its own pair of events on the current
    stream: (median, min, max) in ms.  The clock governor ramps for the first calls after idle; the
    spread shows whether a mean sits inside that ramp."""
    import torch

    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in pairs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in pairs)
    return round(t[len(t) // 2], 4), round(t[0], 4), round(t[-1], 4)


def fill_references(dev, n_bytes):
    """Reference points for a write of n_bytes on this device: (names, callables).  The library's linear fill
    (16 bytes per lane, grid-stride, one resident round of workgroups), the same with every wave walking a
    contiguous span, torch's fill_ (one 16-byte store per thread, workgroups dispatched in address order) and
    torch's copy_ of the same size (as many bytes read as written)."""
    import torch

    from templar_amd import _lib

    lib = _lib.load()
    buf = torch.empty(n_bytes // 4, dtype=torch.float32, device=dev)
    src = torch.ones(n_bytes // 4, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    names = ["library_linear_fill", "library_linear_fill_span_per_wave", "torch_fill_", "torch_copy_"]
    fns = [lambda: _lib.check(lib.tplr_calib_fill(buf.data_ptr(), n_bytes, 0, st), "tplr_calib_fill"),
           lambda: _lib.check(lib.tplr_calib_fill(buf.data_ptr(), n_bytes, 2, st), "tplr_calib_fill"),
           lambda: buf.fill_(1.0),
           lambda: buf.copy_(src)]
    return names, fns


def cpu_baseline(workload_name, k, peers, budget_s):
    """Reference op sequence on torch CPU (oracle/torch_cpu_path.py) on a bounded sample:
    one transformer layer's worth of the 1B set (4 x 2048x2048, 2 x 8192x2048, 2048x8192)
    for encode, 15 peers' payloads of one 2048x2048 tensor for aggregate, repeated until
    about `budget_s` seconds of CPU time are spent."""
    import torch

    import workloads
    from oracle import torch_cpu_path as tcp

    f, b = tcp.basis(64)
    if "cfg1" in workload_name:
        sample_shapes = [(2048, 2048)]
    else:
        sample_shapes = [(2048, 2048)] * 4 + [(8192, 2048)] * 2 + [(2048, 8192)]
    xs = [workloads.student_t3(s, 900 + i, row_scale=True) for i, s in enumerate(sample_shapes)]
    nbytes = workloads.encode_bytes(sample_shapes, k)

    def enc_pass():
        return [tcp.compress(tcp.encode(x, 64, 64, f, f), k) for x in xs]

    enc_pass()
    times = []
    t_begin = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_begin < 0.6 * budget_s and len(times) < 200):
        t0 = time.perf_counter()
        enc_pass()
        times.append(time.perf_counter() - t0)
    enc_s = sorted(times)[len(times) // 2]
    n_enc = len(times)

    # aggregate: `peers` payloads of the first sample tensor
    x0 = xs[0]
    ppay = []
    for p in range(peers):
        g = 0.5 * x0 + workloads.student_t3(x0.shape, 1000 * (p + 1), row_scale=True)
        ppay.append(tcp.compress(tcp.encode(g, 64, 64, f, f), k))
    idxs, vals = [a[0] for a in ppay], [a[1] for a in ppay]
    xshape, totalk = ppay[0][2], ppay[0][3]

    def agg_pass():
        norms = torch.stack([torch.norm(v, p=2) for v in vals])
        return tcp.decode(tcp.batch_decompress(idxs, vals, xshape, totalk, block_norms=norms), b, b)

    agg_pass()
    times = []
    t_begin = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_begin < 0.4 * budget_s and len(times) < 500):
        t0 = time.perf_counter()
        agg_pass()
        times.append(time.perf_counter() - t0)
    agg_s = sorted(times)[len(times) // 2]
    agg_bytes = workloads.aggregate_bytes([tuple(x0.shape)], k, peers)

    # the same op sequence through torch's own kernels on the GPU: what the reference does on this
    # device today (it synchronises in pack_12bit_indices, as the reference's .item() does)
    dev = torch.device("cuda:0")
    fd, bd = f.to(dev), b.to(dev)
    xs_d = [x.to(dev) for x in xs]
    idxs_d, vals_d = [i.to(dev) for i in idxs], [v.to(dev) for v in vals]

    def timed_gpu(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    enc_gpu_s = timed_gpu(lambda: [tcp.compress(tcp.encode(x, 64, 64, fd, fd), k) for x in xs_d], 5)
    agg_gpu_s = timed_gpu(lambda: tcp.decode(tcp.batch_decompress(
        idxs_d, vals_d, xshape, totalk, block_norms=torch.stack([torch.norm(v, p=2) for v in vals_d])), bd, bd), 10)
    same_ops = {"encode_GBps": round(nbytes / enc_gpu_s / 1e9, 2),
                "aggregate_GBps": round(agg_bytes / agg_gpu_s / 1e9, 2),
                "aggregate_ms_per_2048x2048": round(agg_gpu_s * 1e3, 3),
                "what": "the reference's torch op sequence on the same sample, run by torch's ROCm kernels on this GPU"}
    return {
        "value": round(nbytes / enc_s / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": f"encode+top-k+pack of one 1B-set layer {[list(s) for s in sample_shapes]} fp32 (k={k}), median of "
                  f"{n_enc} passes; {peers}-peer decode-aggregate of {list(x0.shape)}, median of {len(times)} passes; "
                  f"torch CPU ops in the reference's order",
        "aggregate_GBps": round(agg_bytes / agg_s / 1e9, 3),
        "aggregate_ms_per_2048x2048": round(agg_s * 1e3, 3),
        "encode_sample_s": round(enc_s, 4),
        "same_ops_on_this_gpu": same_ops,
    }


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}); every box in this build has one GPU and the "
              "path has no collective.  Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch

    import templar_amd.compress as tc
    import workloads
    from templar_amd import _lib as _lib_mod

    dev = torch.device("cuda:0")
    if args.profile == "copy":
        _lib = _lib_mod
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB
        dst = torch.empty_like(src)
        lib = _lib.load()
        event_ms(lambda: _lib.check(lib.tplr_calib_copy(src.data_ptr(), dst.data_ptr(), src.numel() * 4,
                                                        torch.cuda.current_stream().cuda_stream), "calib_copy"),
                 args.steps, args.warmup, settle=True)
        assert torch.equal(src, dst)
        return
    if args.profile == "linfill":
        n_out = workloads.chunks_2d(workloads.CONFIGS[args.workload]["shapes"]) * 16384
        for fn in fill_references(dev, n_out)[1]:
            event_ms(fn, args.steps, args.warmup, settle=True)
        return
    cfg = workloads.CONFIGS[args.workload]
    k, shapes = (args.topk or cfg["k"]), cfg["shapes"]
    P = args.peers
    DCT = not args.no_dct

    class Shapes:
        def named_parameters(self):
            from types import SimpleNamespace
            for i, s in enumerate(shapes):
                yield f"p{i}", SimpleNamespace(requires_grad=True, shape=tuple(s), dtype=torch.float32, device=dev)

    tr = tc.ChunkingTransformer(Shapes(), 64)
    comp = tc.TopKCompressor()

    # ---- inputs resident in HBM
    grads = workloads.gradient_set(args.workload, device=dev)
    two_d = [g for g in grads if g.dim() == 2]
    one_d = [g for g in grads if g.dim() == 1]
    batch = tc.TensorBatch(two_d)
    n_chunks = batch.total_chunks
    idx_buf = torch.empty(n_chunks * (k // 2) * 3, dtype=torch.uint8, device=dev)
    val_buf = torch.empty((n_chunks, k), dtype=torch.float32, device=dev)
    # the norm vectors (rows of 64 elements), every one an allocation of its own as in a model: one launch
    # reads them where they lie
    flat_1d = None
    rows_1d = tc.RowBatch(one_d) if one_d and all(g.numel() % 64 == 0 for g in one_d) else None
    if one_d and rows_1d is None:
        flat_1d = torch.cat(one_d)
    if rows_1d is not None:
        k1 = min(k, 64)
        idx_buf_1d = torch.empty(rows_1d.total_rows * (k1 // 2) * 3, dtype=torch.uint8, device=dev)
        val_buf_1d = torch.empty((rows_1d.total_rows, k1), dtype=torch.float32, device=dev)

    def encode2d_only():
        tc.encode_compress_batch(batch, k, use_dct=DCT, idx12=idx_buf, val=val_buf)

    def encode_pass():
        encode2d_only()
        if rows_1d is not None:
            tc.encode_compress_rows_batch(rows_1d, k, use_dct=DCT, idx12=idx_buf_1d, val=val_buf_1d)
        elif flat_1d is not None:
            comp.compress(tr.encode(flat_1d, use_dct=DCT), k)

    def encode_per_tensor():
        for g in two_d:
            tc.encode_compress(g, k, use_dct=DCT)

    def encode_reference_calls():  # the reference's own two calls per parameter, unchanged
        for g in two_d:
            comp.compress(tr.encode(g, use_dct=DCT), k)

    if flat_1d is not None:
        tr.shape_dict[flat_1d.shape[0]] = 64

    # ---- miner side (src/tplr/neurons.py:147-171): momentum update + encode, then subtract the
    # reconstruction, over the whole set in two launches; separate error-feedback tensors
    def miner_figures(steps, warmup):
        efs = [torch.zeros_like(g) for g in two_d]
        eb = tc.TensorBatch(efs)
        lib = _lib_mod.load()
        st = torch.cuda.current_stream(dev).cuda_stream
        k1 = lambda: _lib_mod.check(lib.tplr_ef_encode_topk_pack_batch(  # noqa: E731
            eb.table.data_ptr(), batch.table.data_ptr(), len(eb), n_chunks, 0.95, k, 1, idx_buf.data_ptr(),
            val_buf.data_ptr(), st), "ef_encode")
        k2 = lambda: _lib_mod.check(lib.tplr_ef_subtract_batch(  # noqa: E731
            idx_buf.data_ptr(), val_buf.data_ptr(), k, eb.table.data_ptr(), len(eb), n_chunks, 1, st), "ef_subtract")
        both = lambda: (k1(), k2())  # noqa: E731
        fused_ms = None
        if DCT:
            kf = lambda: _lib_mod.check(lib.tplr_ef_step_batch(  # noqa: E731
                eb.table.data_ptr(), batch.table.data_ptr(), len(eb), n_chunks, 0.95, k, idx_buf.data_ptr(),
                val_buf.data_ptr(), st), "ef_step")
            fused_ms, _ = event_ms(kf, steps, warmup, settle=True)
        ms_both, _ = event_ms(both, steps, warmup, settle=True)
        ms1, _ = event_ms(k1, steps, 1)
        ms2, _ = event_ms(k2, steps, 1)
        # the same step through the Python entry point with templar's 4-bin quantiser on
        # (hparams.json:59-60): + one quantise and one de-quantise launch over the payload
        q4 = tc.TopKCompressor(use_quantization=True, quantization_bins=4, quantization_range=6)
        _, ms_q = event_ms(lambda: tc.error_feedback_step_batch(eb, batch, 0.95, k, use_dct=DCT, compressor=q4),
                           max(3, steps // 4), 1)
        b1 = n_chunks * (2 * 16384 + 16384 + 11 * k // 2)
        b2 = n_chunks * (16384 + 11 * k // 2 + 16384)
        two = {"ms": round(ms_both, 4), "GBps": round((b1 + b2) / (ms_both * 1e-3) / 1e9, 2),
               "frac_of_hbm_peak": round((b1 + b2) / (ms_both * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
               "update_encode_ms": round(ms1, 4), "update_encode_bytes": b1,
               "subtract_decoded_ms": round(ms2, 4), "subtract_decoded_bytes": b2}
        if fused_ms is None:
            return {"what": "ef = ef*decay + grad, encode+top-k+pack, ef -= decode(payload): two launches over the set",
                    **two, "with_4bin_quantiser_wall_ms": round(ms_q, 4)}
        return {
            "what": "ef = ef*decay + grad, encode+top-k+pack, ef -= decode(payload) over the set in ONE launch (no quantiser "
                    "between the halves): every chunk read once and written once; `two_launches` is the same step as "
                    "update+encode and subtract-decoded launches, which a quantiser between them requires",
            "ms": round(fused_ms, 4), "bytes": b1, "GBps": round(b1 / (fused_ms * 1e-3) / 1e9, 2),
            "frac_of_hbm_peak": round(b1 / (fused_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "two_launches": two,
            "with_4bin_quantiser_wall_ms": round(ms_q, 4),
        }

    # ---- P peers' flat payloads for the aggregation side (peer p = 0.5 shared + own); built before anything is
    # timed: every input of the run is then resident, and the device has left its idle clocks
    # held as a staged window (PayloadStage: one device buffer, the peers' payloads equally spaced), the form
    # in which a gathered window reaches the aggregate
    idxs, vals, idxs_1d, vals_1d = [], [], [], []
    window = tc.PayloadStage(batch, k, P, quantized=False) if args.profile in (None, "aggregate", "calib", "fill", "outer") else None
    # the peers' norms as one float per payload row, noted when a peer's payload is in place (on arrival, in a
    # gather): the window's clip factors then take two small launches and no pass over the values
    norms = tc.PeerNorms([batch] + ([rows_1d] if rows_1d is not None else []), P) if window is not None else None
    for p in range(P if window is not None else 0):  # (a profile of another phase holds only that phase's launches)
        own = [workloads.student_t3(tuple(g.shape), 1000 * (p + 1) + j, row_scale=True, device=dev).add_(g, alpha=0.5)
               for j, g in enumerate(two_d)]
        i12, v = window.regions(p)
        tc.encode_compress_batch(tc.TensorBatch(own), k, use_dct=DCT, idx12=i12, val=v)
        torch.cuda.synchronize()
        idxs.append(i12)
        vals.append(v)
        del own
        if rows_1d is not None:  # the norm vectors' payloads, same recipe
            own = [workloads.student_t3(tuple(g.shape), 2000 * (p + 1) + j, row_scale=False, device=dev).add_(g, alpha=0.5)
                   for j, g in enumerate(one_d)]
            i12, v = tc.encode_compress_rows_batch(tc.RowBatch(own), k, use_dct=DCT)
            idxs_1d.append(i12)
            vals_1d.append(v)
        norms.arrived(p, [vals[p]] + ([vals_1d[p]] if rows_1d is not None else []))
    # every --profile run goes through the same settle phase as the timed run, so that the launches a profiler
    # sees last (the `steps` timed ones) run at the clocks the benchmark line is measured at
    if args.profile == "miner":
        miner_figures(args.steps, args.warmup)
        return
    if args.profile == "encode":
        event_ms(encode2d_only, args.steps, args.warmup, settle=True)
        return
    if args.profile == "read":
        lib_r = _lib_mod.load()
        st_r = torch.cuda.current_stream(dev).cuda_stream
        event_ms(lambda: _lib_mod.check(lib_r.tplr_calib_encode(batch.table.data_ptr(), len(batch), n_chunks, st_r),
                                        "tplr_calib_encode"), args.steps, args.warmup, settle=True)
        return
    if args.profile is None:
        enc_ms, enc_wall = event_ms(encode_pass, args.steps, args.warmup, settle=True)
    enc_bytes = workloads.encode_bytes(shapes, k)
    if args.profile is None:
        enc_spread = launch_stats(encode_pass, args.steps)
        enc2d_ms, _ = event_ms(encode2d_only, args.steps, 1)      # the fused 2-D kernel alone (dominant)
        enc2d_spread = launch_stats(encode2d_only, args.steps)
        # what the memory system alone needs to hand the kernel its input: the library's calibration kernel issues
        # the encode's row loads (same grid, ranges, instructions) and nothing else
        _lib_enc = _lib_mod.load()
        _st_enc = torch.cuda.current_stream(dev).cuda_stream
        enc_read_ms, _ = event_ms(lambda: _lib_mod.check(_lib_enc.tplr_calib_encode(
            batch.table.data_ptr(), len(batch), n_chunks, _st_enc), "tplr_calib_encode"), args.steps, 2)
        enc_pt_ms, _ = event_ms(encode_per_tensor, max(3, args.steps // 2), 1)
        enc_rc_ms, _ = event_ms(encode_reference_calls, 3, 1)
    enc2d_bytes = n_chunks * (16384 + 11 * k // 2)
    miner = miner_figures(max(3, args.steps // 2), 2) if k <= 64 and args.profile is None else None

    outs = two_d  # the gradients are not needed any more: decode into their storage
    out_batch = batch

    def aggregate_2d_pass():
        tc.batch_decompress_decode_batch(out_batch, idxs, vals, k, scale=norms.clip_scales(P)[0], use_dct=DCT)

    def aggregate_pass():
        # clip factors of every parameter from the row figures noted on arrival (two launches), the fused launch
        # over the 2-D set, one launch for the norm vectors
        scales = norms.clip_scales(P)
        tc.batch_decompress_decode_batch(out_batch, idxs, vals, k, scale=scales[0], use_dct=DCT)
        if rows_1d is not None:
            tc.batch_decompress_decode_rows_batch(rows_1d, idxs_1d, vals_1d, min(k, 64), scale=scales[1], use_dct=DCT,
                                                  validate=False)

    def aggregate_pass_norms_from_values():
        # the same pass when nothing was noted on arrival: the norms are taken from the values here (one more
        # pass over every peer's values per batch)
        tc.batch_decompress_decode_batch(out_batch, idxs, vals, k, clip_norm=True, use_dct=DCT)
        if rows_1d is not None:
            tc.batch_decompress_decode_rows_batch(rows_1d, idxs_1d, vals_1d, min(k, 64), clip_norm=True, use_dct=DCT,
                                                  validate=False)

    scale = tc.peer_clip_scales_batch(out_batch, vals, k)

    def aggregate_kernel_only():
        tc.batch_decompress_decode_batch(out_batch, idxs, vals, k, scale=scale, use_dct=DCT)

    # the reference's per-parameter form of the same payloads (lists of P tensors per parameter)
    per_param = []
    for i in range(len(out_batch)):
        sl = [out_batch.payload_slice(i, idxs[p], vals[p], k) for p in range(P)]
        per_param.append(([a for a, _ in sl], [b for _, b in sl], out_batch.xshape(i)))

    def aggregate_per_tensor():
        for i, (pi, pv, xs) in enumerate(per_param):
            tc.batch_decompress_decode(pi, pv, xs, out=outs[i], use_dct=DCT)

    def aggregate_reference_calls():  # batch_decompress then decode per parameter, unchanged
        for i, (pi, pv, xs) in enumerate(per_param):
            tr.decode(comp.batch_decompress(outs[i], pi, pv, xs, 4096, clip_norm=True), use_dct=DCT)

    # what the memory system alone needs for this launch's traffic: the library's calibration kernel issues the
    # aggregate's loads and stores (same grid, ranges, instructions) without the scatter and the transform
    lib_c = _lib_mod.load()
    ip_c = (ctypes.c_void_p * P)(*[i.data_ptr() for i in idxs])
    vp_c = (ctypes.c_void_p * P)(*[v.data_ptr() for v in vals])
    cur_stream = torch.cuda.current_stream(dev).cuda_stream

    def calib(n_peers):
        _lib_mod.check(lib_c.tplr_calib_aggregate(ip_c, vp_c, n_peers, k, int(DCT), out_batch.table.data_ptr(), len(out_batch),
                                                  n_chunks, cur_stream), "tplr_calib_aggregate")

    if args.profile in ("calib", "fill"):
        event_ms(lambda: calib(P if args.profile == "calib" else 0), args.steps, args.warmup, settle=True)
        return
    if args.profile == "aggregate":
        event_ms(aggregate_pass, args.steps, args.warmup, settle=True)
        return
    if args.profile == "outer":
        prm = tc.TensorBatch([torch.zeros_like(o) for o in outs])
        fac = (scale * 0.4).contiguous()
        flg = torch.zeros(len(prm), dtype=torch.int32, device=dev)
        pc_ = torch.empty((n_chunks, 2), dtype=torch.float32, device=dev)
        pt_ = torch.empty((len(prm), 4), dtype=torch.float32, device=dev)
        event_ms(lambda: _lib_mod.check(lib_c.tplr_outer_step_batch(
            ip_c, vp_c, fac.data_ptr(), P, k, prm.table.data_ptr(), len(prm), n_chunks, pc_.data_ptr(), pt_.data_ptr(),
            flg.data_ptr(), cur_stream), "tplr_outer_step_batch"), args.steps, args.warmup, settle=True)
        return
    agg_steps = max(3, args.steps // 2)
    agg_ms, agg_wall = event_ms(aggregate_pass, agg_steps, 2, settle=True)
    aggv_ms, _ = event_ms(aggregate_pass_norms_from_values, agg_steps, 1)
    agg2d_ms, _ = event_ms(aggregate_2d_pass, agg_steps, 1)
    aggk_ms, _ = event_ms(aggregate_kernel_only, agg_steps, 1)
    aggk_spread = launch_stats(aggregate_kernel_only, agg_steps)
    ceiling = None
    agg_bytes = n_chunks * (P * 11 * k // 2 + 16384)           # the fused kernel's launch
    if P <= 24 and k <= 64:
        mem_ms, _ = event_ms(lambda: calib(P), agg_steps, 2)
        fill_ms, _ = event_ms(lambda: calib(0), agg_steps, 2)
        ceiling = {"memory_only_ms": round(mem_ms, 4), "fill_only_ms": round(fill_ms, 4),
                   "frac_of_hbm_peak": round(agg_bytes / (mem_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                   "kernel_over_memory_only": round(aggk_ms / mem_ms, 4),
                   "what": "tplr_calib_aggregate: the kernel's own loads and stores (same grid, chunk ranges and "
                           "instructions) with no scatter and no transform - what this box's memory system needs "
                           "for the launch's traffic; fill_only: the stores alone"}
    # what a write of the launch's output costs this memory system under friendlier access patterns
    attainable = None
    if args.workload in ("cfg3_llama1b", "cfg5_72b_block", "cfg2_llama150m"):
        n_out = n_chunks * 16384
        names, fns = fill_references(dev, n_out)
        ref_ms = {nm: round(event_ms(fn, agg_steps, 2, settle=True)[0], 4) for nm, fn in zip(names, fns)}
        attainable = {
            "what": "reference points for this launch's 4-byte-per-lane row stores (64 rows of 256 B per chunk, rows a "
                    "tensor row apart): a write of the same number of bytes over a linear address range by the library's "
                    "fill (16 B per lane; grid-stride, or every wave on a span of its own), by torch's fill_ (one 16 B "
                    "store per thread, workgroups dispatched in address order) and torch's copy_ of that size (reads "
                    "and writes in equal parts); memory_only_ms is the launch's own loads and stores with nothing else",
            "output_bytes": n_out,
            "ms": ref_ms,
            "GBps": {nm: round((2 if nm == "torch_copy_" else 1) * n_out / (ms * 1e-3) / 1e9, 1) for nm, ms in ref_ms.items()},
            "chunk_pattern_fill_ms": ceiling["fill_only_ms"] if ceiling else None,
            "memory_only_ms": ceiling["memory_only_ms"] if ceiling else None,
        }
        del names, fns
        torch.cuda.empty_cache()
    # the aggregation as the benchmark's workload words it: sum over the peers, inverse transform, mean over
    # the peers, every tensor divided by its L2 norm (three launches; tplr.compress itself has no such mode)
    aggn_ms, _ = event_ms(lambda: tc.aggregate_mean_normalised_batch(out_batch, idxs, vals, k), agg_steps, 1)
    aggn2_ms, _ = event_ms(lambda: tc.aggregate_mean_normalised_batch(out_batch, idxs, vals, k, two_pass=True),
                           agg_steps, 1)
    # the aggregate together with what outer_step looks at next per parameter (L2 norm, mean, all-finite):
    # from two floats per chunk left by the same launch, against the three torch reductions per dense tensor
    aggs_ms, _ = event_ms(lambda: tc.batch_decompress_decode_batch(out_batch, idxs, vals, k, scale=scale, use_dct=DCT,
                                                                   stats=True), agg_steps, 1)

    def stats_by_torch():
        for o in outs:
            torch.linalg.vector_norm(o)
            o.mean()
            torch.isfinite(o).all()

    stats_torch_ms, _ = event_ms(stats_by_torch, 3, 1)
    agg_pt_ms, _ = event_ms(aggregate_per_tensor, 3, 1)
    agg_rc_ms, _ = event_ms(aggregate_reference_calls, 3, 1)
    # the same per-parameter loop recorded once into a HIP graph and replayed: what is left is device time
    side_stream = torch.cuda.Stream(device=dev)
    side_stream.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side_stream):
        aggregate_per_tensor()
    torch.cuda.current_stream(dev).wait_stream(side_stream)
    torch.cuda.synchronize()
    per_tensor_graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(per_tensor_graph):
        aggregate_per_tensor()
    agg_graph_ms, _ = event_ms(per_tensor_graph.replay, 5, 1)
    agg_pass_bytes = workloads.aggregate_bytes(shapes, k, P)  # the whole set, norm vectors included
    # validator-side checks on the same payloads: pairwise index overlap, repeats, bounds
    stats = None
    if P <= 32:
        st_ms, _ = event_ms(lambda: tc.index_stats_batch(out_batch, idxs, k), agg_steps, 1)
        st_bytes = n_chunks * P * (k + k // 2)
        stats = {"what": f"pairwise index overlap + repeats + bounds of {P} peers' packed indices, one launch",
                 "ms": round(st_ms, 4), "GBps": round(st_bytes / (st_ms * 1e-3) / 1e9, 2), "bytes": st_bytes}

    # the validator's per-peer evaluation update (neurons/validator.py:3595-3737): one peer's payload times its clip
    # factor, decompress, decode, p.data.sub_(decoded, alpha) - one launch that reads and writes every parameter once,
    # against decode into a dense gradient followed by the subtraction over the set
    evaluation = None
    if k <= 64:
        params = [torch.zeros_like(o) for o in outs]
        pb = tc.TensorBatch(params)
        clip0 = scale.reshape(len(out_batch), -1)[:, 0].contiguous()
        # (the per-parameter non-finite flags are left on the device: a caller reads them once per peer)
        ev_ms, _ = event_ms(lambda: tc.apply_decoded_batch(pb, idxs[0], vals[0], k, alpha=0.01, clip=clip0, use_dct=DCT,
                                                           on_nonfinite="flags"), agg_steps, 2)

        def decode_then_subtract():
            tc.batch_decompress_decode_batch(out_batch, idxs[:1], vals[:1], k, scale=clip0.reshape(-1, 1), use_dct=DCT)
            torch._foreach_sub_(params, outs, alpha=0.01)

        ev2_ms, _ = event_ms(decode_then_subtract, agg_steps, 1)
        ev_bytes = n_chunks * (11 * k // 2 + (2 * 16384 if DCT else 8 * k))
        evaluation = {"what": "one peer's payload applied to the parameters (values x clip factor, decompress, decode, "
                              "p -= alpha * decoded) in one launch over the set, against decode into a dense gradient and "
                              "a foreach subtraction; bytes: the payload + every chunk read and written (with the "
                              "transform) or k elements per chunk read and written (without)",
                      "ms": round(ev_ms, 4), "bytes": ev_bytes, "GBps": round(ev_bytes / (ev_ms * 1e-3) / 1e9, 2),
                      "decode_then_subtract_ms": round(ev2_ms, 4)}
        del params, pb

    # the outer step over the window (src/tplr/neurons.py:309-447 with the plain SGD of neurons/trainer.py:128-130):
    # p <- p - lr * decode(aggregate) in the launch that forms the aggregate, against the aggregate written as a
    # dense gradient, its statistics, the isfinite test and a foreach subtraction
    outer = None
    if DCT and 4 <= k <= 64 and P <= 15:
        params = [torch.zeros_like(o) for o in outs]
        pb = tc.TensorBatch(params)
        lr = 0.4
        factor = (scale * lr).contiguous()
        flags = torch.zeros(len(pb), dtype=torch.int32, device=dev)
        pc = torch.empty((n_chunks, 2), dtype=torch.float32, device=dev)
        pt = torch.empty((len(pb), 4), dtype=torch.float32, device=dev)

        def outer_kernel():
            _lib_mod.check(lib_c.tplr_outer_step_batch(ip_c, vp_c, factor.data_ptr(), P, k, pb.table.data_ptr(), len(pb),
                                                       n_chunks, pc.data_ptr(), pt.data_ptr(), flags.data_ptr(), cur_stream),
                           "tplr_outer_step_batch")

        ok_ms, _ = event_ms(outer_kernel, agg_steps, 2, settle=True)
        _, ow_wall = event_ms(lambda: tc.outer_step_batch(pb, idxs, vals, k, lr, scale=scale), agg_steps, 1)

        def aggregate_then_sgd():
            st = tc.batch_decompress_decode_batch(out_batch, idxs, vals, k, scale=scale, use_dct=DCT, stats=True)
            if bool((st[:, 2] == 1).all()):
                torch._foreach_sub_(params, outs, alpha=lr)

        ats_ms, ats_wall = event_ms(aggregate_then_sgd, agg_steps, 1)
        os_bytes = n_chunks * (P * 11 * k // 2 + 2 * 16384)
        outer = {"what": f"p <- p - lr * decode(aggregate of {P} peers) for every 2-D parameter, with the gradients' norm, "
                         "mean and all-finite flag: one launch that reads and writes every parameter once and never "
                         "writes the gradient (bytes: payload + every chunk read and written), against the aggregate "
                         "launch with statistics followed by torch's foreach subtraction of the dense gradients",
                 "kernel_ms": round(ok_ms, 4), "bytes": os_bytes, "GBps": round(os_bytes / (ok_ms * 1e-3) / 1e9, 2),
                 "frac_of_hbm_peak": round(os_bytes / (ok_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                 "call_wall_ms": round(ow_wall, 4), "aggregate_then_sgd_ms": round(ats_ms, 4),
                 "aggregate_then_sgd_wall_ms": round(ats_wall, 4)}
        del params, pb, pc

    # templar's own settings carry the values as the codes of a four-bin quantiser: the aggregate straight from
    # the codes against de-quantising every peer first (what outer_step does, src/tplr/neurons.py:325-364)
    def codes_figures(idxs_, vals_, kk):
        """idxs_/vals_: the peers' fp32 flat payloads of the 2-D set (views of a staged window) at top-k kk, chunks
        not transformed; they are quantised with four bins here."""
        PP, T = len(vals_), len(out_batch)
        cbuf = torch.empty((PP, n_chunks, kk), dtype=torch.uint8, device=dev)
        qps = [[None] * PP for _ in range(T)]
        peer_tables = []
        for p in range(PP):
            c, q_shift, q_scale, q_lookup = tc.quantize_batch(out_batch, vals_[p], kk, 4, 6.0)
            cbuf[p].copy_(c)
            peer_tables.append((q_lookup, q_shift))
            for i in range(T):
                qps[i][p] = (q_shift[i], 1.0, 2, q_lookup[i], torch.float32)
        codes = [cbuf[p] for p in range(PP)]
        fp32_buf = torch.empty((PP, n_chunks, kk), dtype=torch.float32, device=dev)
        q_tables = tc.dequantised_tables(qps, dev)   # once per window, like the stage's own tables

        def from_codes():
            tc.batch_decompress_decode_codes_batch(out_batch, idxs_, codes, qps, kk, validate=False, tables=q_tables)

        def dequantise_first():
            fp = [tc.dequantize_batch(out_batch, codes[p].reshape(-1), None, kk, out=fp32_buf[p], tables=peer_tables[p])
                  for p in range(PP)]
            tc.batch_decompress_decode_batch(out_batch, idxs_, fp, kk, clip_norm=True, use_dct=False)

        c_ms, c_wall = event_ms(from_codes, agg_steps, 2, settle=True)
        d_ms, d_wall = event_ms(dequantise_first, agg_steps, 2)
        # the outer step from the same codes: p <- p - lr * aggregate in the launch that forms it, against the
        # aggregate from codes with statistics followed by a foreach subtraction of the dense gradients
        prm = [torch.zeros_like(o) for o in outs]
        pbt = tc.TensorBatch(prm)
        o_ms, o_wall = event_ms(lambda: tc.outer_step_codes_batch(pbt, idxs_, codes, None, kk, 0.4, tables=q_tables,
                                                                  validate=False), agg_steps, 2)

        def codes_then_sgd():
            st = tc.batch_decompress_decode_codes_batch(out_batch, idxs_, codes, qps, kk, validate=False, tables=q_tables,
                                                        stats=True)
            if bool((st[:, 2] == 1).all()):
                torch._foreach_sub_(prm, outs, alpha=0.4)

        s_ms, s_wall = event_ms(codes_then_sgd, agg_steps, 1)
        del prm, pbt
        outer_bytes = n_chunks * (PP * (kk + kk // 2 + kk) + 2 * 16384)
        code_bytes = n_chunks * (PP * (kk + kk // 2 + kk) + 16384)
        return {"what": f"aggregate of the 2-D set from 4-bin codes, {PP} peers, k = {kk}, chunks not transformed (index "
                        "bytes + one byte per value read, dense written; norms from counts; no fp32 copy of the payload) "
                        "against de-quantise every peer, norms, fp32 aggregate",
                "from_codes_ms": round(c_ms, 4), "from_codes_wall_ms": round(c_wall, 4),
                "dequantise_first_ms": round(d_ms, 4), "dequantise_first_wall_ms": round(d_wall, 4),
                "from_codes_bytes": code_bytes,
                "from_codes_GBps": round(code_bytes / (c_ms * 1e-3) / 1e9, 2),
                "from_codes_frac_of_hbm_peak": round(code_bytes / (c_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                "outer_step_from_codes_ms": round(o_ms, 4), "outer_step_from_codes_wall_ms": round(o_wall, 4),
                "outer_step_from_codes_bytes": outer_bytes,
                "outer_step_from_codes_GBps": round(outer_bytes / (o_ms * 1e-3) / 1e9, 2),
                "outer_step_what": "p <- p - lr * aggregate for every 2-D parameter straight from the codes (norms from "
                                   "counts, clip factors, one fused launch, per-parameter statistics and non-finite "
                                   "flags read back: the whole call with its one synchronisation), against the "
                                   "aggregate from codes with statistics followed by a foreach subtraction",
                "aggregate_from_codes_then_sgd_ms": round(s_ms, 4), "aggregate_from_codes_then_sgd_wall_ms": round(s_wall, 4)}

    codes_path = None
    if not DCT and k <= 64 and P <= 24 and args.profile is None:
        codes_path = codes_figures(idxs, vals, k)

    # the same set at templar's own settings (hparams/hparams.json: topk_compression 64, use_dct false,
    # quantization_bins 4, 20 gathered peers), when this run is not already made with them: the encode launch
    # and the aggregate from codes, on payloads built here
    templar_settings = None
    if args.profile is None and args.workload == "cfg3_llama1b" and (DCT or k != 64 or P != 20):
        tk, tP = 64, 20
        g2 = [g for g in workloads.gradient_set(args.workload, device=dev) if g.dim() == 2]
        b2 = tc.TensorBatch(g2)
        t_idx = torch.empty(n_chunks * (tk // 2) * 3, dtype=torch.uint8, device=dev)
        t_val = torch.empty((n_chunks, tk), dtype=torch.float32, device=dev)
        te_ms, _ = event_ms(lambda: tc.encode_compress_batch(b2, tk, use_dct=False, idx12=t_idx, val=t_val),
                            args.steps, args.warmup, settle=True)
        te_bytes = n_chunks * (16384 + 11 * tk // 2)
        # the miner's whole step at these settings (src/tplr/neurons.py:147-171): momentum update + select, the 4-bin
        # quantiser over the payload, the sent values subtracted at their k positions per chunk
        t_efs = [torch.zeros_like(g) for g in g2]
        t_eb = tc.TensorBatch(t_efs)
        q4 = tc.TopKCompressor(use_quantization=True, quantization_bins=4, quantization_range=6)
        tm_ms, tm_wall = event_ms(lambda: tc.error_feedback_step_batch(t_eb, b2, 0.95, tk, use_dct=False, compressor=q4),
                                  max(3, args.steps // 4), 2)
        del t_efs, t_eb
        t_win = tc.PayloadStage(batch, tk, tP, quantized=False)
        t_idxs, t_vals = [], []
        for p in range(tP):
            own = [workloads.student_t3(tuple(g.shape), 3000 * (p + 1) + j, row_scale=True, device=dev).add_(g, alpha=0.5)
                   for j, g in enumerate(g2)]
            i12, v = t_win.regions(p)
            tc.encode_compress_batch(tc.TensorBatch(own), tk, use_dct=False, idx12=i12, val=v)
            torch.cuda.synchronize()
            t_idxs.append(i12)
            t_vals.append(v)
            del own
        del g2, b2
        templar_settings = {
            "what": "the same 1B set at templar's hparams.json settings: top-k 64 per chunk, chunks not transformed, "
                    "4-bin quantiser, 20 peers",
            "encode_ms": round(te_ms, 4), "encode_GBps": round(te_bytes / (te_ms * 1e-3) / 1e9, 2),
            "encode_frac_of_hbm_peak": round(te_bytes / (te_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "miner_step_ms": round(tm_ms, 4), "miner_step_wall_ms": round(tm_wall, 4),
            "aggregate": codes_figures(t_idxs, t_vals, tk),
        }
        del t_win, t_idxs, t_vals

    # a gathered window arriving as the reference's per-parameter host lists (torch.load output):
    # flat staging through one pinned buffer, against one transfer per tensor
    staging = None
    if P * n_chunks * 11 * k // 2 < 2 << 30:
        h_idx = [[pi[p].cpu() for p in range(P)] for pi, _, _ in per_param]
        h_val = [[pv[p].cpu() for p in range(P)] for _, pv, _ in per_param]
        stage = tc.PayloadStage(out_batch, k, P, quantized=False)
        _, st_wall = event_ms(lambda: stage.load(h_idx, h_val), 3, 1)
        _, pt_wall = event_ms(lambda: [[t.to(dev, non_blocking=True) for t in row] for row in h_idx + h_val], 3, 1)
        st_bytes = P * n_chunks * 11 * k // 2
        staging = {"what": f"{P} peers x {len(per_param)} parameters of host payload lists to the device: "
                           "flat pinned buffer packed by host threads, one transfer per peer, against one transfer per tensor "
                           "(wall time, PCIe included)",
                   "flat_ms": round(st_wall, 3), "per_tensor_ms": round(pt_wall, 3), "bytes": st_bytes,
                   "flat_GBps": round(st_bytes / (st_wall * 1e-3) / 1e9, 2)}
        del h_idx, h_val, stage

    result = {
        "metric": "encode+topk+pack GB/s and 15-peer decode-aggregate ms, 1B grads, 1 GPU",
        "value": round(enc_bytes / (enc_ms * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(enc_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: encode+top-k+pack of {len(shapes)} tensors "
                               f"({workloads.chunks_2d(shapes)} chunks 64x64, k={k}) and {P}-peer decode-aggregate",
                   "chunk": 64, "topk": k, "peers": P, "use_dct": DCT},
        "clock_settle_s": SETTLE_S,
        "encode_wall_ms": round(enc_wall, 4),
        "aggregate_ms": round(agg_ms, 4),
        "aggregate_GBps": round(agg_pass_bytes / (agg_ms * 1e-3) / 1e9, 2),
        "aggregate_wall_ms": round(agg_wall, 4),
        "aggregate_2d_ms": round(agg2d_ms, 4),
        "aggregate_norms_from_values_ms": round(aggv_ms, 4),
        "aggregate_note": "aggregate_ms: the whole pass over the window (clip factors of every parameter, the fused "
                          "launch over the 2-D set, the norm vectors) with the peers' per-row sums of squares noted when "
                          "their payloads arrived (PeerNorms: one launch per peer at arrival, 1/k of the value bytes "
                          "kept); aggregate_norms_from_values_ms: the same pass taking the norms from the values inside "
                          "it, as the reference does",
        "aggregate_sum_mean_normalised_ms": round(aggn_ms, 4),
        "aggregate_sum_mean_normalised_note": "the workload's own wording: scatter-sum over the peers, inverse DCT, "
                                              "divide by their number, divide each tensor by its L2 norm; the norms "
                                              "come from the payloads (orthonormal transform: one launch over the "
                                              "payload, no dense traffic) and are folded into the factors of the one "
                                              "aggregate launch; _two_pass_ms is the literal order (aggregate, norms "
                                              "of the dense result, one scaling pass); aggregate_ms is the "
                                              "reference's batch_decompress semantics",
        "aggregate_sum_mean_normalised_two_pass_ms": round(aggn2_ms, 4),
        "aggregate_from_quantised_codes": codes_path,
        "templar_settings": templar_settings,
        "aggregate_with_result_stats": {"kernel_with_stats_ms": round(aggs_ms, 4), "kernel_ms": round(aggk_ms, 4),
                                        "same_stats_by_torch_ms": round(stats_torch_ms, 4),
                                        "what": "per-parameter L2 norm, mean and all-finite flag of the decoded "
                                                "gradients from two floats per chunk left by the aggregate launch "
                                                "(+ one small launch), against norm, mean and isfinite().all() of "
                                                "every dense tensor by torch afterwards"},
        "ms_per_step_spread": {"median": enc_spread[0], "min": enc_spread[1], "max": enc_spread[2],
                               "what": "per-call durations of a further `steps` calls of the step, each between its own events"},
        "per_tensor_launches": {"encode_ms": round(enc_pt_ms, 4), "aggregate_ms": round(agg_pt_ms, 4),
                                "note": "same work as one fused launch per tensor through the reference-shaped API",
                                "aggregate_graph_replay_ms": round(agg_graph_ms, 4),
                                "reference_calls_encode_ms": round(enc_rc_ms, 4),
                                "reference_calls_aggregate_ms": round(agg_rc_ms, 4),
                                "reference_calls_note": "the reference's unchanged call sites: encode then compress, "
                                                        "batch_decompress then decode, per parameter"},
        "roofline": {
            "bound": "hbm", "kernel": "k_encode_topk_pack",
            "achieved": round(enc2d_bytes / (enc2d_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(enc2d_bytes / (enc2d_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic(args.workload, k, DCT, P, "encode"),
            "traffic_source": "profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this launch "
                              "(bench_profiles.py), not measured by this run; null for launches not profiled",
            "launches_per_step": 1, "bytes_per_launch": enc2d_bytes, "ms_per_launch": round(enc2d_ms, 4),
            "ms_per_launch_median": enc2d_spread[0], "ms_per_launch_min": enc2d_spread[1],
            "ceiling": {"read_only_ms": round(enc_read_ms, 4),
                        "frac_of_hbm_peak": round(n_chunks * 16384 / (enc_read_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                        "kernel_over_read_only": round(enc2d_ms / enc_read_ms, 4),
                        "what": "tplr_calib_encode: the kernel's own row loads (same grid, chunk ranges and "
                                "instructions) with no transform, no select and no payload stores - what this box's "
                                "memory system needs to deliver the launch's input"},
        },
        "roofline_aggregate": {
            "bound": "hbm", "kernel": "k_decode_aggregate",
            "achieved": round(agg_bytes / (aggk_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(agg_bytes / (aggk_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic(args.workload, k, DCT, P, "aggregate"),
            "traffic_source": "profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this launch "
                              "(bench_profiles.py), not measured by this run; null for launches not profiled",
            "launches_per_step": 1, "bytes_per_launch": agg_bytes, "ms_per_launch": round(aggk_ms, 4),
            "ms_per_launch_median": aggk_spread[0], "ms_per_launch_min": aggk_spread[1],
            "ceiling": ceiling,
            "attainable": attainable,
        },
    }
    # the codec runs once per window, minutes apart: one call after the device has sat idle
    def after_idle(fn):
        torch.cuda.synchronize()
        time.sleep(2.0)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        return round(a.elapsed_time(b), 4)

    result["first_call_after_idle_ms"] = {
        "encode": after_idle(encode_pass), "aggregate": after_idle(aggregate_pass),
        "what": "one call of the step / of the aggregate pass after 2 s without work on the device (events around the "
                "single call): what a miner or validator that runs the codec once per window sees, clocks not settled"}
    if miner is not None:
        result["error_feedback_step"] = miner
    if stats is not None:
        result["index_stats"] = stats
    if evaluation is not None:
        result["evaluation_update"] = evaluation
    if outer is not None:
        result["outer_step"] = outer
    if staging is not None:
        result["payload_staging"] = staging
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload, k, P, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
