"""tplr_quantize_batch_static, the entry point that allocates nothing, against tplr_quantize_batch.

Both run the same four kernels; the static form keeps the partial sums in the library's own
device array instead of a caller-provided workspace.  Two calls in a row, the second on a
smaller input, must each equal the workspace form bit for bit: the array keeps the first
call's contents, and nothing in it may leak into the second.
"""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import templar_amd.compress as tc  # noqa: E402
from templar_amd import _lib  # noqa: E402


def _payload(shapes, k, seed, dev):
    rng = np.random.default_rng(seed)
    batch = tc.TensorBatch([torch.zeros(s, device=dev) for s in shapes])
    parts = [rng.standard_t(3, size=((s[0] // 64) * (s[1] // 64), k)).astype(np.float32) * np.float32(10.0 ** (i % 4 - 3))
             + np.float32(0.01 * i) for i, s in enumerate(shapes)]
    return batch, torch.from_numpy(np.concatenate(parts)).to(dev)


def _run(lib, batch, val, k, bins, slices, static):
    dev, n, T = batch.device, batch.total_chunks, len(batch)
    codes = torch.full((n, k), 255, dtype=torch.uint8, device=dev)
    shift = torch.full((T,), -7.0, device=dev)
    scale = torch.full((T,), -7.0, device=dev)
    lookup = torch.full((T, bins), -7.0, device=dev)
    stream = tc._stream(dev)
    with tc._on(dev):
        if static:
            st = lib.tplr_quantize_batch_static(tc._ptr(val), k, tc._ptr(batch.table), T, bins, C.c_float(6.0), slices,
                                                tc._ptr(codes), tc._ptr(shift), tc._ptr(scale), tc._ptr(lookup), stream)
        else:
            work = torch.empty(T * slices * (2 + 2 * bins), dtype=torch.float64, device=dev)
            st = lib.tplr_quantize_batch(tc._ptr(val), k, tc._ptr(batch.table), T, bins, C.c_float(6.0), slices,
                                         tc._ptr(work), tc._ptr(codes), tc._ptr(shift), tc._ptr(scale), tc._ptr(lookup),
                                         stream)
    assert st == 0, lib.tplr_status_string(st)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (codes, shift, scale, lookup)]


@pytest.mark.parametrize("bins", [4, 256])
def test_static_scratch_quantiser_equals_workspace_form_twice(dev, bins):
    lib = _lib.load()
    k = 32
    big = [(256, 512), (64, 192), (1024, 512), (64, 64), (192, 128), (512, 64)]
    small = [(64, 128), (128, 64)]
    for shapes, slices, seed in ((big, 16, 11 + bins), (small, 3, 12 + bins)):  # second call: smaller input
        batch, val = _payload(shapes, k, seed, dev)
        want = _run(lib, batch, val, k, bins, slices, static=False)
        got = _run(lib, batch, val, k, bins, slices, static=True)
        for name, g, w in zip(("codes", "shift", "scale", "lookup"), got, want):
            assert g.dtype == w.dtype and g.shape == w.shape
            assert np.array_equal(g.view(np.uint8), w.view(np.uint8)), name  # bit for bit


def test_static_scratch_rejects_what_does_not_fit(dev):
    lib = _lib.load()
    cap = lib.tplr_static_work_bytes() // 8
    assert cap == 2048 * (2 + 2 * 256)
    k, bins, slices = 32, 256, 1024
    T = cap // (slices * (2 + 2 * bins)) + 1  # one tensor too many for the array
    p = tc._ptr(torch.zeros(64, device=dev))  # valid, aligned; never dereferenced: the call must refuse first
    st = lib.tplr_quantize_batch_static(p, k, p, T, bins, C.c_float(6.0), slices, p, p, p, p, None)
    assert st == _lib.TPLR_E_WORKSPACE
    assert b"static scratch" in lib.tplr_status_string(st)
    torch.cuda.synchronize()
