"""The reference's own unit tests for the codec classes (tests/unit/test_compress.py:18-275),
case by case, against this module on the GPU: same inputs, same calls, same assertions, plus
the oracle's result where the reference only checks shapes."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import codec as orc  # noqa: E402  (the checker)
from templar_amd.compress import (ChunkingTransformer, TopKCompressor, pack_12bit_indices,  # noqa: E402
                                  unpack_12bit_indices)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")


@pytest.fixture
def comp():
    return TopKCompressor(use_quantization=False)


# ---------------------------------------------------------------- TestTopKCompressor (:18-221)
def test_compress_produces_packed_indices(dev, comp):  # :33-50
    x = torch.randn(10, 10, device=dev)
    idx, val, xshape, totalk = comp.compress(x, 10)
    assert idx.dtype == torch.uint8 and val.shape[-1] == 10 and xshape == x.shape and totalk == x.shape[-1]
    want_i, want_v = orc.topk_rows(x.cpu().numpy(), 10)
    assert np.array_equal(unpack_12bit_indices(idx, val.shape).cpu().numpy(), want_i)
    assert np.array_equal(val.cpu().numpy(), want_v)


def test_compress_with_quantization(dev):  # :52-70
    q = TopKCompressor(use_quantization=True, quantization_bins=256, quantization_range=6)
    x = torch.randn(10, 10, device=dev)
    result = q.compress(x, 20)
    assert len(result) == 5
    idx, val, _, _, qparams = result
    assert idx.dtype == torch.uint8 and val.dtype == torch.uint8 and qparams is not None and len(qparams) == 5
    assert val.shape[-1] == 10  # top-k clamps to the row length


def test_decompress_with_12bit_format(dev, comp):  # :72-95
    p = torch.zeros(10, 10, device=dev)
    original = torch.tensor([[0, 1, 2, 3], [4, 5, 6, 7]], dtype=torch.int64)
    idx = pack_12bit_indices(original.to(dev))
    val = torch.tensor([[0.1, 0.2, 0.3, 0.4], [0.5, 0.6, 0.7, 0.8]], device=dev)
    # the reference's call: xshape (10, 10), totalk 100, two rows of indices (the scatter fills
    # the first two rows and leaves the rest zero)
    result = comp.decompress(p, idx, val, (10, 10), 100)
    assert result.shape == (10, 10) and result.dtype == p.dtype
    want = orc.decompress(orc.pack12(original.numpy()), val.cpu().numpy(), (2, 10), 10)
    assert np.array_equal(result[:2].cpu().numpy(), want) and float(result[2:].abs().max()) == 0.0


def test_batch_decompress_multiple_12bit_formats(dev, comp):  # :97-125
    idx1 = torch.tensor([[0, 1], [2, 3]], dtype=torch.int64)
    idx2 = torch.tensor([[4, 5], [6, 7]], dtype=torch.int64)
    val1 = torch.tensor([[0.1, 0.2], [0.3, 0.4]])
    val2 = torch.tensor([[0.5, 0.6], [0.7, 0.8]])
    p = torch.zeros(10, 10, device=dev)
    result = comp.batch_decompress(p, [pack_12bit_indices(idx1.to(dev)), pack_12bit_indices(idx2.to(dev))],
                                   [val1.to(dev), val2.to(dev)], (10, 10), 100)
    assert result.shape == (10, 10) and result.dtype == p.dtype
    want = orc.batch_decompress([orc.pack12(idx1.numpy()), orc.pack12(idx2.numpy())], [val1.numpy(), val2.numpy()],
                                (2, 10), 10)
    assert np.allclose(result[:2].cpu().numpy(), want, rtol=1e-6, atol=0) and float(result[2:].abs().max()) == 0.0


def test_compress_decompress_round_trip(dev, comp):  # :127-158
    x = torch.zeros(10, 10, device=dev)
    x[0, 0], x[1, 1], x[2, 2], x[3, 3] = 1.0, 2.0, 3.0, 4.0
    idx, val, xshape, totalk = comp.compress(x, 4)
    assert idx.dtype == torch.uint8 and val.shape[-1] == 4
    result = comp.decompress(torch.zeros_like(x), idx, val, xshape, totalk)
    assert result.shape == x.shape and result.abs().max() > 0
    top_vals = torch.topk(result.abs().flatten(), k=4).values
    assert torch.allclose(top_vals.cpu(), torch.tensor([4.0, 3.0, 2.0, 1.0]), atol=1e-5)
    assert torch.equal(result, x)  # the four spikes and nothing else


def test_12bit_index_value_range(dev, comp):  # :160-187
    x = torch.randn(100, 100, device=dev)
    idx, val, _, totalk = comp.compress(x, 100)
    assert idx.dtype == torch.uint8
    unpacked = unpack_12bit_indices(idx, val.shape)
    assert unpacked.max().item() < 10000
    if totalk > 256:
        assert unpacked.max() > 255
    # every row keeps all of its 100 elements: a permutation of the row, largest first
    assert torch.equal(unpacked.sort(dim=-1).values, torch.arange(100, device=dev).expand(100, 100))
    want_i, want_v = orc.topk_rows(x.cpu().numpy(), 100)
    assert np.array_equal(unpacked.cpu().numpy(), want_i) and np.array_equal(val.cpu().numpy(), want_v)


def test_batch_decompress_with_norm_options(dev, comp):  # :189-221
    p = torch.zeros(10, 10, device=dev)
    xshape, totalk = (10, 10), 100
    idx_orig = torch.tensor([[0, 1, 2, 3]], dtype=torch.int64)
    idx = [pack_12bit_indices(idx_orig.to(dev))]
    val = [torch.tensor([[10.0, 20.0, 30.0, 40.0]], device=dev)]
    packed = [orc.pack12(idx_orig.numpy())]
    host_val = [v.cpu().numpy() for v in val]
    r_norm = comp.batch_decompress(p, idx, val, xshape, totalk, normalise=True)
    assert r_norm.shape == xshape
    assert np.allclose(r_norm[:1].cpu().numpy(), orc.batch_decompress(packed, host_val, (1, 10), 10, normalise=True),
                       rtol=1e-6)
    r_clip = comp.batch_decompress(p, idx, val, xshape, totalk, clip_norm=True)
    assert r_clip.shape == xshape
    assert np.allclose(r_clip[:1].cpu().numpy(), orc.batch_decompress(packed, host_val, (1, 10), 10, clip_norm=True),
                       rtol=1e-6)
    norms = torch.tensor([15.0], device=dev)
    r_bn = comp.batch_decompress(p, idx, val, xshape, totalk, block_norms=norms, clip_norm=True)
    assert r_bn.shape == xshape
    want = orc.batch_decompress(packed, host_val, (1, 10), 10, block_norms=np.array([15.0], np.float32))
    assert np.allclose(r_bn[:1].cpu().numpy(), want, rtol=1e-6) and float(r_bn[1:].abs().max()) == 0.0


# ---------------------------------------------------------------- TestChunkingTransformer (:223-275)
class _SimpleModel(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.layer1 = torch.nn.Linear(32, 64)
        self.layer2 = torch.nn.Linear(64, 128)


def test_transform_init(dev):  # :238-253
    model = _SimpleModel().to(dev)
    tr = ChunkingTransformer(model, 16)
    assert len(tr.shape_dict) > 0 and len(tr.f_dict) > 0 and len(tr.b_dict) > 0
    for param in model.parameters():
        if param.requires_grad:
            for d in param.shape:
                assert d in tr.shape_dict


def test_encode_decode_real_tensors(dev):  # :255-275
    model = _SimpleModel().to(dev)
    tr = ChunkingTransformer(model, 8)
    param = next(model.parameters()).detach()
    encoded = tr.encode(param, use_dct=False)
    assert encoded.numel() == param.numel()
    decoded = tr.decode(encoded, use_dct=False)
    assert decoded.shape == param.shape and torch.allclose(decoded, param.reshape(decoded.shape))
    encoded_dct = tr.encode(param, use_dct=True)
    decoded_dct = tr.decode(encoded_dct, use_dct=True)
    assert decoded_dct.shape == param.shape
    # 8x8 chunks: the dense-contraction kernel; against the oracle and as a round trip
    want = orc.encode2d(param.cpu().numpy(), 8, 8)
    assert np.abs(encoded_dct.cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max()
    assert torch.allclose(decoded_dct, param, atol=1e-6)


# ---------------------------------------------------------------- callers' init-time shape probe
@pytest.mark.parametrize("use_dct", [False, True])
def test_init_time_shape_probe(dev, use_dct):
    # neurons/miner.py:245-254, neurons/validator.py:394-404: encode + compress of an uninitialised
    # fp16 tensor per parameter, only to record xshape and totalk
    shapes = [(128, 192), (64,), (2048,), (100, 48), (192, 64)]
    tr = ChunkingTransformer(_Shapes(shapes, dev), 64)
    q = TopKCompressor(use_quantization=True, quantization_bins=4, quantization_range=6)
    want = {(128, 192): ((2, 3, 64, 64), 4096), (64,): ((1, 64), 64), (2048,): ((32, 64), 64),
            (100, 48): ((2, 1, 50, 48), 2400), (192, 64): ((3, 1, 64, 64), 4096)}
    for s in shapes:
        probe = torch.full(s, float("nan"), dtype=torch.float16, device=dev)
        enc = tr.encode(probe, use_dct=use_dct)
        idx, val, xshape, totalk, qp = q.compress(enc, 32)
        assert (tuple(xshape), totalk) == want[s]
        assert idx.dtype == torch.uint8 and val.dtype == torch.uint8 and len(qp) == 5
        k = min(32, totalk)
        assert val.shape == tuple(xshape[:-2 if len(xshape) == 4 else -1]) + (k,)
        assert idx.numel() * 2 == val.numel() * 3


class _Shapes:
    def __init__(self, shapes, dev):
        self._p = [torch.nn.Parameter(torch.empty(s, device=dev)) for s in shapes]

    def named_parameters(self):
        for i, p in enumerate(self._p):
            yield f"p{i}", p


def test_transformer_honours_an_unnormalised_basis(dev):
    # ChunkingTransformer(model, 64, norm=None): the bases are the unnormalised DCT-II (2 sum x cos) and its
    # inverse, as _dct / _idct build them (src/tplr/compress.py:710-788); 64-element chunks then go through the
    # dense contraction with those bases, not through the orthonormal kernels
    import scipy.fft
    from types import SimpleNamespace

    class M:
        def named_parameters(self):
            yield "w", SimpleNamespace(requires_grad=True, shape=(128, 192), dtype=torch.float32, device=dev)
            yield "b", SimpleNamespace(requires_grad=True, shape=(128,), dtype=torch.float32, device=dev)

    tr = ChunkingTransformer(M(), 64, norm=None)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((128, 192)).astype(np.float32)
    coef = tr.encode(torch.from_numpy(x).to(dev), use_dct=True)
    chunks = x.reshape(2, 64, 3, 64).transpose(0, 2, 1, 3)
    want = scipy.fft.dctn(chunks.astype(np.float64), type=2, norm=None, axes=(2, 3))
    assert coef.shape == (2, 3, 64, 64)
    assert np.abs(coef.cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max()
    back = tr.decode(coef, use_dct=True)
    assert np.abs(back.cpu().numpy() - x).max() <= 1e-5 * np.abs(x).max()
    v = rng.standard_normal(128).astype(np.float32)
    c1 = tr.encode(torch.from_numpy(v).to(dev), use_dct=True)
    want1 = scipy.fft.dct(v.reshape(2, 64).astype(np.float64), type=2, norm=None, axis=1)
    assert np.abs(c1.cpu().numpy() - want1).max() <= 1e-5 * np.abs(want1).max()
    assert np.abs(tr.decode(c1, use_dct=True).cpu().numpy() - v).max() <= 1e-5 * np.abs(v).max()

