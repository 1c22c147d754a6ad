"""Shapes at the two ends of the feature width: rows of a single float4 (the flat decoders and
encoders index by a 32-bit reciprocal that does not exist for one item per row) and fused SQ
rows wider than the row-block kernels stage (2 KB of codes per edge)."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from f2cgt_amd import capi

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def graph(rng, rows, n_src, max_deg):
    deg = rng.integers(0, max_deg + 1, size=rows)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    return indptr, rng.integers(0, n_src, size=int(indptr[-1])).astype(np.int64)


@pytest.mark.parametrize("bits,d", [(1, 8), (1, 4), (2, 4), (4, 4), (8, 4), (16, 4), (1, 16), (4, 8)])
def test_log_sq_rows_of_one_lane(bits, d):
    print("case log_sq narrow bits=%d d=%d" % (bits, d), flush=True)
    rng = np.random.default_rng(bits * 10 + d)
    x = rng.uniform(-2, 2, size=(3001, d)).astype(np.float32)
    cb = np.stack([oc.sq_codebook(x)])
    codes = oc.sq_compress(x, cb, bits, d)
    assert np.array_equal(host(capi.sq_compress(dev(x), dev(cb), bits, d)), codes)
    store = oc.sq_codes_to_storage(codes, bits)
    assert np.array_equal(host(capi.sq_encode(dev(x), dev(cb), bits, d)).view(store.dtype), store)
    want = oc.sq_decompress(store, cb, bits, d, d)
    assert np.array_equal(host(capi.sq_decompress(dev(store), dev(cb), bits, d, d)), want)
    per = max(1, 8 // bits)
    if d % per == 0:
        indptr, indices = graph(rng, 500, 3001, 9)
        got = host(capi.sq_decompress_spmm_csr(dev(store), dev(cb), dev(indptr), dev(indices), bits, d, d))
        assert np.array_equal(got, oc.sq_decompress_spmm_csr(store, cb, indptr, indices, bits, d, d))


@pytest.mark.parametrize("bits,d", [(1, 8), (2, 4), (4, 4), (8, 4), (8, 8)])
def test_affine_sq_rows_of_one_lane(bits, d):
    print("case affine narrow bits=%d d=%d" % (bits, d), flush=True)
    rng = np.random.default_rng(100 + bits * 10 + d)
    raw = rng.integers(0, 1 << bits, size=(2999, d), dtype=np.uint8)
    store = oc.packbits(raw, bits) if bits < 8 else raw
    params = np.stack([rng.standard_normal(d), 0.01 + rng.random(d)]).astype(np.float32)
    want = oc.sq_affine_decompress(store, params, bits, d)
    assert np.array_equal(host(capi.sq_affine_decompress(dev(store), dev(params), bits, d)), want)
    indptr, indices = graph(rng, 400, 2999, 9)
    got = host(capi.sq_affine_decompress_spmm_csr(dev(store), dev(params), dev(indptr), dev(indices), bits, d))
    ref = oc.sq_affine_decompress_spmm_csr(store, params, indptr, indices, bits, d)
    assert np.allclose(got, ref, rtol=RTOL, atol=RTOL * np.abs(want).max())


def test_hybrid_rows_of_four_columns():
    print("case hybrid d=4", flush=True)
    rng = np.random.default_rng(5)
    n, n_sq, d = 3000, 400, 4
    row_map = np.concatenate([np.arange(n_sq), -np.arange(1, n - n_sq + 1)]).astype(np.int32)
    sq_codes = rng.integers(0, 256, size=(n_sq, d), dtype=np.uint8)
    params = np.stack([rng.standard_normal(d), 0.01 + 0.02 * rng.random(d)]).astype(np.float32)
    vq_codes = rng.integers(0, 256, size=(n - n_sq, 1), dtype=np.uint8)
    vcb = rng.standard_normal((1, 256, 4)).astype(np.float32)
    indptr, indices = graph(rng, 700, n, 14)
    want = oc.hybrid_decompress_spmm_csr(row_map, sq_codes, params, vq_codes, vcb, indptr, indices, d)
    got = host(capi.hybrid_decompress_spmm_csr(dev(row_map), dev(sq_codes), dev(params), dev(vq_codes), dev(vcb),
                                               dev(indptr), dev(indices), d))
    assert np.allclose(got, want, rtol=RTOL, atol=RTOL * 8)


@pytest.mark.parametrize("bits,d", [(8, 2040), (8, 2044), (8, 2048), (8, 4096), (4, 4080), (4, 4096)])
def test_fused_sq_with_wide_rows(bits, d):
    print("case fused sq wide bits=%d d=%d" % (bits, d), flush=True)
    rng = np.random.default_rng(bits + d)
    n, rows = 600, 150
    x = rng.uniform(-2, 2, size=(n, d)).astype(np.float32)
    cs = d // 2 if (d // 2) % (8 // bits) == 0 else d
    cbs = np.stack([oc.sq_codebook(x[:, s:s + cs]) for s in range(0, d, cs)])
    store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, cs), bits)
    indptr, indices = graph(rng, rows, n, 12)
    got = host(capi.sq_decompress_spmm_csr(dev(store), dev(cbs), dev(indptr), dev(indices), bits, cs, d))
    assert np.array_equal(got, oc.sq_decompress_spmm_csr(store, cbs, indptr, indices, bits, cs, d))
    raw = rng.integers(0, 1 << bits, size=(n, d), dtype=np.uint8)
    packed = oc.packbits(raw, bits) if bits < 8 else raw
    params = np.stack([rng.standard_normal(d), 0.01 + rng.random(d)]).astype(np.float32)
    got = host(capi.sq_affine_decompress_spmm_csr(dev(packed), dev(params), dev(indptr), dev(indices), bits, d))
    ref = oc.sq_affine_decompress_spmm_csr(packed, params, indptr, indices, bits, d)
    assert np.allclose(got, ref, rtol=RTOL, atol=RTOL * np.abs(ref).max())


def test_module_refuses_unsigned_eight_bit_log_codes():
    import f2cgt_amd
    lib = f2cgt_amd.load()
    cb = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
    codes = torch.zeros((4, 16), dtype=torch.uint8, device="cuda")
    ip = torch.tensor([0, 2, 4], device="cuda")
    ix = torch.tensor([0, 1, 2, 3], device="cuda")
    with pytest.raises(RuntimeError, match="int8"):
        lib.sq_decompress(codes, cb, 8, 16, 16)
    with pytest.raises(RuntimeError, match="int8"):
        lib.sq_decompress_spmm_csr(codes, cb, ip, ix, 8, 16, 16)
    a = lib.sq_decompress(codes.view(torch.int8), cb, 8, 16, 16)
    assert a.shape == (4, 16)
