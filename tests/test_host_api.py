"""Host-side logic of templar_amd that needs no GPU: the C ABI's symbol table, the helper
functions the reference's tests import, argument validation and error text, the host-memory
pack/unpack entry points, and the zero-copy chunk view."""
import ctypes
import json
import os
import re

import ctypes as C

import numpy as np
import pytest
import torch

import templar_amd
import templar_amd.compress as tc
from templar_amd import _lib
from oracle import codec as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KATS = json.load(open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")))


def header_functions():
    text = open(os.path.join(ROOT, "include", "tplr_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(tplr_[a-z0-9_]+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    names = header_functions()
    assert len(names) >= 15 and len(set(names)) == len(names)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert getattr(lib, n) is not None
    assert set(names) == set(_lib.SIGNATURES), "ctypes table and header disagree"
    assert _lib.load().tplr_version() >= 100
    assert _lib.load().tplr_status_string(0) == b"ok"


def test_api_surface_matches_reference_module():
    for name in ["pack_12bit_indices", "unpack_12bit_indices", "ChunkingTransformer", "TopKCompressor", "_dct", "_idct",
                 "_get_smaller_split", "_get_divisors", "_get_prime_divisors", "TransformDCT", "CompressDCT",
                 "ShapeT", "Shape4D", "TotK", "IdxT", "ValT", "QuantParamsT"]:
        assert hasattr(tc, name), name
    assert tc.TransformDCT is tc.ChunkingTransformer and tc.CompressDCT is tc.TopKCompressor
    c = tc.TopKCompressor(use_quantization=True, quantization_bins=4, quantization_range=6)
    assert c.use_quantization and c.n_bins == 4 and c.range_in_sigmas == 6
    for m in ["compress", "decompress", "batch_decompress", "_quantize_values", "_dequantize_values",
              "maybe_dequantize_values", "_clamp_topk"]:
        assert callable(getattr(c, m))
    assert templar_amd.compress is tc


@pytest.mark.parametrize("n,c,want", [tuple(x) for x in KATS["smaller_split"]])
def test_smaller_split_reference_vectors(n, c, want):
    assert tc._get_smaller_split(n, c) == want


def test_divisor_helpers_against_oracle():
    for n in list(range(1, 300)) + [768, 2048, 3072, 8192, 29568, 32000]:
        assert tc._get_divisors(n) == orc.divisors(n)
        prod = 1
        for p in tc._get_prime_divisors(n):
            prod *= p
            assert all(p % q for q in range(2, int(p ** 0.5) + 1))
        assert prod == n
        for c in (1, 7, 16, 64, 100):
            assert tc._get_smaller_split(n, c) == orc.smaller_split(n, c)
    assert tc._get_divisors(0) == []


def test_dct_helpers():
    x = torch.randn(4, 8)
    X = tc._dct(x, norm="ortho")
    assert torch.allclose(tc._idct(X, norm="ortho"), x, atol=1e-6)  # tests/unit/test_compress.py:281-290
    assert np.allclose(tc._dct(torch.eye(64), norm="ortho").numpy(), orc.dct_basis(64), atol=1e-7)
    assert np.allclose(tc._idct(torch.eye(64), norm="ortho").numpy(), orc.dct_basis(64).T, atol=1e-7)
    # un-normalised convention of torch-dct: X_k = 2 sum x_n cos(pi (2n+1) k / 2N)
    e = torch.zeros(1, 8)
    e[0, 0] = 1.0
    assert torch.allclose(tc._dct(e)[0], 2 * torch.cos(torch.arange(8) * torch.pi / 16), atol=1e-6)
    assert torch.allclose(tc._idct(tc._dct(x)), x, atol=1e-5)


class _Model:
    def __init__(self, shapes, dtype=torch.float32):
        self.params = [torch.nn.Parameter(torch.zeros(s, dtype=dtype)) for s in shapes]
        self.params.append(torch.nn.Parameter(torch.zeros(7, 7), requires_grad=False))

    def named_parameters(self):
        return [(f"w{i}", p) for i, p in enumerate(self.params)]


def test_chunking_transformer_tables():
    tr = tc.ChunkingTransformer(_Model([(64, 32), (128, 64), (128,), (100, 30)]), 16)
    assert tr.target_chunk == 16
    assert tr.shape_dict == {64: 16, 32: 16, 128: 16, 100: 10, 30: 15}
    assert 7 not in tr.shape_dict  # frozen parameters are skipped
    assert set(tr.f_dict) == {16, 10, 15} == set(tr.b_dict)
    for n in tr.f_dict:
        assert np.allclose(tr.f_dict[n].numpy(), orc.dct_basis(n), atol=1e-6)
        assert np.allclose(tr.b_dict[n].numpy(), orc.dct_basis(n).T, atol=1e-6)
    tr16 = tc.ChunkingTransformer(_Model([(64, 64)], dtype=torch.bfloat16), 64)
    assert tr16.f_dict[64].dtype == torch.bfloat16


def test_encode_decode_without_dct_is_a_view():
    tr = tc.ChunkingTransformer(_Model([(32, 64), (64,)]), 8)
    x = torch.arange(32 * 64, dtype=torch.float32).reshape(32, 64)
    e = tr.encode(x, use_dct=False)
    assert e.shape == (4, 8, 8, 8) and e.data_ptr() == x.data_ptr()
    assert np.array_equal(e.numpy(), orc.encode2d(x.numpy(), 8, 8, use_dct=False))
    assert torch.equal(tr.decode(e, use_dct=False), x)
    v = torch.arange(64, dtype=torch.float32)
    ev = tr.encode(v, use_dct=False)
    assert ev.shape == (8, 8) and torch.equal(tr.decode(ev, use_dct=False), v)
    with pytest.raises(KeyError):
        tr.encode(torch.zeros(48, 64), use_dct=False)
    with pytest.raises(RuntimeError, match="HIP device"):
        tr.encode(x, use_dct=True)


def test_clamp_topk():
    c = tc.TopKCompressor()
    for last in (1, 2, 3, 10, 64, 100, 4096):
        for k in (0, 1, 2, 3, 31, 32, 33, 64, 5000):
            assert c._clamp_topk(torch.empty(3, last), k) == orc.clamp_topk(last, k)


def test_host_pack_unpack_vectors():
    for case in KATS["pack_roundtrip"]:
        idx = torch.tensor(case["indices"], dtype=torch.int64)
        packed = tc.pack_12bit_indices(idx)
        assert packed.dtype == torch.uint8 and packed.numel() == case["packed_len"]
        assert np.array_equal(packed.numpy(), orc.pack12(case["indices"]))
        back = tc.unpack_12bit_indices(packed, idx.shape)
        assert back.dtype == torch.int64 and torch.equal(back, idx)
    torch.manual_seed(42)
    idx = torch.randint(0, 4096, (100,), dtype=torch.int64)
    packed = tc.pack_12bit_indices(idx)
    assert packed.numel() == 150 and torch.equal(tc.unpack_12bit_indices(packed, idx.shape), idx)
    two_d = torch.tensor([[10, 20, 30, 40], [50, 60, 70, 80]])
    assert torch.equal(tc.unpack_12bit_indices(tc.pack_12bit_indices(two_d), two_d.shape), two_d)
    assert tc.pack_12bit_indices(torch.arange(1000)).numel() == 1500  # 75 % of int16


def test_host_gather_concatenates_parts_with_any_thread_count():
    import ctypes as C

    from templar_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(5)
    sizes = [0, 1, 7, 4096, 3, 1 << 20, 123457, 0, 999, 2 << 20]
    parts = [rng.integers(0, 256, n, dtype=np.uint8) for n in sizes]
    want = np.concatenate(parts)
    ptrs = (C.c_void_p * len(parts))(*[p.ctypes.data if p.size else None for p in parts])
    nbytes = (C.c_int64 * len(parts))(*sizes)
    for threads in (1, 2, 3, 8, 64):
        dst = np.full(want.size + 16, 0xEE, np.uint8)
        assert lib.tplr_gather_host(ptrs, nbytes, len(parts), dst.ctypes.data + 8, threads) == 0
        assert np.array_equal(dst[8:-8], want) and (dst[:8] == 0xEE).all() and (dst[-8:] == 0xEE).all()
    assert lib.tplr_gather_host(ptrs, nbytes, len(parts), None, 4) == _lib.TPLR_E_BADARG
    assert lib.tplr_gather_host(ptrs, nbytes, len(parts), 1, 0) == _lib.TPLR_E_BADARG
    assert lib.tplr_gather_host(None, None, 0, None, 1) == 0


def test_entry_points_reject_bad_arguments_before_any_launch():
    # argument checks run on the host and return before a kernel is launched: no device needed.
    # (1 stands for "some non-null pointer": a rejected call never dereferences it.)
    from templar_amd import _lib
    lib = _lib.load()
    E = _lib
    p = 1 << 12
    assert lib.tplr_version() > 0
    assert lib.tplr_pack12(None, 2, p, None, None) == E.TPLR_E_BADARG
    assert lib.tplr_pack12(p, 3, p, None, None) == E.TPLR_E_ODD
    assert lib.tplr_pack12(p, -2, p, None, None) == E.TPLR_E_BADARG
    assert lib.tplr_pack12(None, 0, None, None, None) == 0
    assert lib.tplr_unpack12(None, 2, p, None) == E.TPLR_E_BADARG
    assert lib.tplr_unpack12(p, 5, p, None) == E.TPLR_E_ODD
    assert lib.tplr_dct2d_fwd(None, 64, 64, 64, p, None) == E.TPLR_E_BADARG
    assert lib.tplr_dct2d_fwd(p, 64, 96 + 1, 128, p, None) == E.TPLR_E_SHAPE
    assert lib.tplr_dct2d_inv(p, 63, 64, p, 64, None) == E.TPLR_E_SHAPE
    assert lib.tplr_topk_pack(p, 1, 4096, 33, p, p, None) == E.TPLR_E_BADARG      # odd k
    assert lib.tplr_topk_pack(p, 1, 5000, 32, p, p, None) == E.TPLR_E_TOOMANY     # row too long
    assert lib.tplr_encode_topk_pack(p, 64, 64, 32, 32, 1, p, p, None) == E.TPLR_E_BADARG  # stride below the width
    assert lib.tplr_encode_topk_pack(p, 64, 64, 64, 130, 1, p, p, None) == E.TPLR_E_BADARG  # k above 128
    assert lib.tplr_encode_topk_pack_batch(None, 1, 1, 32, 1, p, p, None) == E.TPLR_E_BADARG
    ptrs = (C.c_void_p * 2)(p, p)
    assert lib.tplr_decode_aggregate(ptrs, ptrs, None, 2, 31, 64, 64, 0, 0, 1, p, 64, None, None) == E.TPLR_E_BADARG
    assert lib.tplr_decode_aggregate(ptrs, ptrs, None, 2, 32, 64, 65, 0, 0, 1, p, 65, None, None) == E.TPLR_E_SHAPE
    many = (C.c_void_p * 129)(*([p] * 129))
    assert lib.tplr_decode_aggregate(many, many, None, 129, 32, 64, 64, 0, 0, 1, p, 64, None, None) == E.TPLR_E_TOOMANY
    assert lib.tplr_index_stats_batch(many, 33, 32, p, 1, 1, p, p, p, None) == E.TPLR_E_TOOMANY
    assert lib.tplr_index_stats_batch(ptrs, 2, 33, p, 1, 1, p, p, p, None) == E.TPLR_E_BADARG
    assert lib.tplr_dequantize_batch(p, p, p, 300, 32, p, 1, 1, p, None) == E.TPLR_E_BADARG   # more than 256 bins
    assert lib.tplr_dequantize_peers(ptrs, 2, 6, p, p, 4, ptrs, None) == E.TPLR_E_BADARG       # n not a multiple of 4
    assert lib.tplr_quantize_batch(p, 32, p, 1, 4, C.c_float(6.0), 0, p, p, p, p, p, None) == E.TPLR_E_BADARG  # no slices
    assert lib.tplr_quantize_batch(p + 4, 32, p, 1, 4, C.c_float(6.0), 1, p, p, p, p, p, None) == E.TPLR_E_BADARG
    assert lib.tplr_aggregate_rows(ptrs, ptrs, None, 2, 31, None, 0, 4, 64, 0, p, None, None) == E.TPLR_E_BADARG
    assert lib.tplr_aggregate_rows(ptrs, ptrs, p, 2, 32, None, 0, 4, 64, 0, p, None, None) == E.TPLR_E_BADARG  # factors without a table
    assert lib.tplr_aggregate_rows(many, many, None, 129, 32, None, 0, 4, 64, 0, p, None, None) == E.TPLR_E_TOOMANY
    assert lib.tplr_aggregate_rows(ptrs, ptrs, None, 2, 32, None, 0, 4, 5000, 0, p, None, None) == E.TPLR_E_TOOMANY
    assert lib.tplr_segment_sumsq(ptrs, 2, 32, p, 1, 0, p, None) == E.TPLR_E_BADARG
    assert lib.tplr_clip_scales(None, 2, 0, p, None, None) == E.TPLR_E_BADARG
    for code in (0, E.TPLR_E_BADARG, E.TPLR_E_ODD, E.TPLR_E_SHAPE, E.TPLR_E_TOOMANY, 1):
        assert len(lib.tplr_status_string(code)) > 0


def test_pack_unpack_errors():
    with pytest.raises(ValueError, match="Number of indices must be even, got 3"):
        tc.pack_12bit_indices(torch.tensor([1, 2, 3]))
    with pytest.raises(ValueError, match=r"Index 4096 exceeds 12-bit limit \(4095\)"):
        tc.pack_12bit_indices(torch.tensor([0, 4096]))
    with pytest.raises(ValueError, match="exceeds 12-bit limit"):
        tc.pack_12bit_indices(torch.tensor([1, 2, 5000]))  # the range check comes first
    with pytest.raises(ValueError, match="Number of indices must be even, got 3"):
        tc.unpack_12bit_indices(torch.zeros(6, dtype=torch.uint8), (3,))
    with pytest.raises(RuntimeError, match="shape mismatch"):
        tc.unpack_12bit_indices(torch.zeros(5, dtype=torch.uint8), (4,))
    empty = tc.pack_12bit_indices(torch.tensor([], dtype=torch.int64))
    assert empty.numel() == 0
    assert tc.unpack_12bit_indices(empty, (0,)).shape == (0,)


def test_decompress_validation_happens_before_any_kernel():
    c = tc.TopKCompressor()
    p = torch.zeros(10, 10)
    with pytest.raises(ValueError, match=r"Expected uint8 \(packed\) or int64 \(unpacked\) indices, got torch.int32"):
        c.decompress(p, torch.zeros(4, dtype=torch.int32), torch.zeros(2, 2), (10, 10), 10)
    with pytest.raises(ValueError, match="Expected uint8 for 12-bit packed indices, got torch.int64"):
        c.batch_decompress(p, [torch.zeros(4, dtype=torch.int64)], [torch.zeros(2, 2)], (10, 10), 10)
    with pytest.raises(RuntimeError, match="HIP device"):
        c.compress(torch.randn(10, 10), 4)
    with pytest.raises(RuntimeError, match="HIP device"):
        c.decompress(p, torch.zeros(6, dtype=torch.uint8), torch.zeros(2, 2), (10, 10), 10)


def test_quantiser_matches_oracle_and_reference_contract():
    c = tc.TopKCompressor(use_quantization=True, quantization_bins=256, quantization_range=6)
    g = torch.Generator().manual_seed(3)
    v = torch.randn(4, 3, 32, generator=g)
    q, qp = c._quantize_values(v)
    assert q.dtype == torch.uint8 and len(qp) == 5 and qp[2] == 128 and qp[4] == torch.float32
    oq, (oshift, oscale, ooff, olook) = orc.quantize(v.numpy(), 256, 6)
    assert abs(qp[1] - oscale) <= 1e-6 * oscale and abs(float(qp[0]) - oshift) < 1e-7
    assert (q.numpy() != oq).mean() < 0.01  # rounding of the scale may move a value on a bin edge
    assert np.allclose(qp[3].numpy(), olook, atol=1e-5)
    deq = c._dequantize_values(q, qp)
    assert deq.dtype == torch.float32 and (deq - v).abs().max() <= qp[1]
    assert c._dequantize_values(v, qp) is v  # not uint8: returned untouched
    # constant tensor -> scale 1.0
    _, qp2 = tc.TopKCompressor(use_quantization=True, quantization_bins=4)._quantize_values(torch.full((8,), 0.25))
    assert qp2[1] == 1.0
    # list handling of maybe_dequantize_values (reference :646-696)
    out = c.maybe_dequantize_values([q, q], [qp, qp], torch.device("cpu"))
    assert len(out) == 2 and torch.equal(out[0], deq)
    assert c.maybe_dequantize_values([v], [qp], torch.device("cpu"))[0] is v
    assert torch.equal(c.maybe_dequantize_values([q], qp, torch.device("cpu"))[0], deq)  # a bare 5-tuple
    with pytest.raises(IndexError, match="Mismatch in val lengths"):
        c.maybe_dequantize_values([q, q], [qp, None], torch.device("cpu"))


# ---------------------------------------------------------------- check_compressed_indices
def test_check_compressed_indices_reference_cases():
    """The cases of the reference's tests/test_comms.py:1828-2004 (hparams.topk_compression = 4),
    on host tensors: same acceptances, same error messages."""
    chk = lambda name, idxs, totalk, **kw: tc.check_compressed_indices(name, idxs, totalk, topk_compression=4, **kw)  # noqa: E731
    pk = tc.pack_12bit_indices
    v = lambda *shape: torch.randn(*shape)  # noqa: E731
    # valid: flat and multi-dimensional
    chk("test_param", pk(torch.tensor([1, 5, 9, 3])), 10, vals=v(4))
    chk("param", pk(torch.tensor([[0, 1, 2, 3], [4, 5, 6, 7]])), 20, vals=v(2, 4))
    # not packed / wrong dtype
    for bad in (torch.tensor([0, 1, 2, 3], dtype=torch.long), torch.tensor([0, 1, 2, 3], dtype=torch.int32)):
        with pytest.raises(ValueError, match="Expected uint8 for 12-bit packed indices"):
            chk("param", bad, 20, vals=v(4))
    # wrong top-k dimension, flat and multi-dimensional
    with pytest.raises(ValueError, match="Invalid topk dimension"):
        chk("param", pk(torch.tensor([0, 1])), 10, vals=v(2))
    with pytest.raises(ValueError, match="Invalid topk dimension"):
        chk("param", pk(torch.tensor([[0, 1, 2, 3, 4, 5], [6, 7, 8, 9, 10, 11]])), 20, vals=v(2, 6))
    # out of bounds
    with pytest.raises(ValueError, match="Index 10 out of bounds"):
        chk("param", pk(torch.tensor([0, 1, 10, 3])), 10, vals=v(4))
    # allowed_topk override
    chk("param", pk(torch.tensor([0, 9])), 10, allowed_topk=2, vals=v(2))
    with pytest.raises(ValueError, match="Invalid topk dimension"):
        chk("param", pk(torch.tensor([0, 1, 2, 3])), 10, allowed_topk=2, vals=v(4))
    # totalk below the configured top-k
    chk("param", pk(torch.tensor([0, 1])), 2, vals=v(2))
    with pytest.raises(ValueError, match="Invalid topk dimension"):
        chk("param", pk(torch.tensor([0, 1, 0, 1])), 2, vals=v(4))
    # the reference's other refusals
    with pytest.raises(ValueError, match="Values tensor required"):
        chk("param", pk(torch.tensor([0, 1])), 10)
    with pytest.raises(ValueError, match="Empty packed indices tensor"):
        chk("param", torch.empty(0, dtype=torch.uint8), 10, vals=v(0))
    with pytest.raises(ValueError, match="Expected tensor but got"):
        chk("param", [0, 1, 2, 3], 10, vals=v(4))



def test_quantiser_tables_round_through_the_senders_dtype():
    # src/tplr/compress.py:641-643: (lookup[code] + shift).to(orig_dtype); the flat tables carry that rounding as
    # lookup' = round(lookup + shift), shift' = 0, so that the kernels' fp32 sum reproduces it
    import torch

    import templar_amd.compress as tc
    from oracle import torch_cpu_path as tcp

    torch.manual_seed(5)
    lookup = torch.randn(4) * 1e-2
    shift = torch.tensor(3.3e-3)
    qp32 = (shift, 1.0, 2, lookup, torch.float32)
    qp16 = (shift, 1.0, 2, lookup, torch.bfloat16)
    lk, sh, n_bins = tc._qparam_tables([qp32, qp16], torch.device("cpu"))
    assert n_bins == 4
    codes = torch.arange(4, dtype=torch.uint8)
    assert torch.equal(lk[0][codes.long()] + sh[0], tcp.dequantize(codes, qp32))
    want16 = tcp.dequantize(codes, qp16)
    assert want16.dtype == torch.bfloat16
    assert torch.equal(lk[1][codes.long()] + sh[1], want16.float())
    deq, _ = tc.dequantised_tables([[qp32, qp16]], torch.device("cpu"))
    assert torch.equal(deq[0, 0], tcp.dequantize(codes, qp32)) and torch.equal(deq[0, 1], want16.float())
    with pytest.raises(ValueError, match="different sizes"):
        tc._qparam_tables([qp32, (shift, 1.0, 4, torch.randn(8), torch.float32)], torch.device("cpu"))
