"""The aggregation followed by the dense layer that consumes it (first GraphSAGE layer with the mean
aggregator, examples/conv.py:68-69): `*_decompress_spmm_csr_linear` of the F2CGTLib module.
The destination rows can be processed in blocks, one after the other or with the aggregation of
the next block on a second stream; with the identity as weight every form must give the unblocked
aggregate bit for bit (x*1 plus zeros is exact), which checks every block boundary and the stream
hand-over; with a random weight the result is compared with the oracle's aggregate times the
weight in float64."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from parity_bars import assert_mean_aggregate

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def graph(rng, rows, n_src, max_deg, idx):
    deg = rng.integers(0, max_deg + 1, size=rows)
    deg[rng.integers(0, rows, size=max(1, rows // 50))] = 0
    indptr = np.zeros(rows + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    return indptr, rng.integers(0, n_src, size=int(indptr[-1])).astype(idx)


@pytest.fixture(scope="module")
def lib():
    import f2cgt_amd

    return f2cgt_amd.load()


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("n_cb,width,feat_dim", [(16, 8, 128), (24, 32, 768), (3, 4, 10)])
def test_vq_linear_blocks_match_unblocked_aggregate(lib, idx, n_cb, width, feat_dim):
    rng = np.random.default_rng(n_cb * 100 + width)
    n_src, rows = 5000, 3001
    codes = rng.integers(0, 256, size=(n_src, n_cb), dtype=np.uint8)
    cbs = rng.standard_normal((n_cb, 256, width)).astype(np.float32)
    indptr, indices = graph(rng, rows, n_src, 20, idx)
    c, cb, ip, ix = dev(codes), dev(cbs), dev(indptr), dev(indices)
    whole = lib.vq_decompress_spmm_csr(c, cb, ip, ix, feat_dim)
    dec = oc.vq_decompress(codes, cbs, feat_dim)
    i64 = (indptr.astype(np.int64), indices.astype(np.int64))
    want_agg, exact_agg, unit = oc.spmm_csr(dec, *i64), oc.spmm_csr(dec.astype(np.float64), *i64), np.abs(dec).max()
    assert_mean_aggregate(whole.cpu().numpy(), want_agg, exact_agg, unit, np.diff(i64[0]))
    eye = torch.eye(feat_dim, device="cuda")
    for block_rows in (0, 1, 7, 256, 1000, 3001, 10000):
        if block_rows == 1 and feat_dim > 10:
            continue  # 3001 single-row launches add nothing over the narrow case
        for overlap in (False, True):
            got = lib.vq_decompress_spmm_csr_linear(c, cb, ip, ix, feat_dim, eye, None, block_rows, overlap)
            assert got.shape == (rows, feat_dim)
            # a row block is a launch of its own and may take another kernel than the whole graph does
            # (few rows: the per-row skeleton, which divides; many: the pipelined kernel, which
            # multiplies by a refined reciprocal): equal to 2 ulp, and bit for bit in edge-order sums
            assert_mean_aggregate(got.cpu().numpy(), want_agg, exact_agg, unit, np.diff(indptr.astype(np.int64)))
    # a real layer: weight [hidden, feat_dim] and bias, against float64 on the oracle's aggregate
    hidden = 48
    w = (rng.standard_normal((hidden, feat_dim)) / np.sqrt(feat_dim)).astype(np.float32)
    b = rng.standard_normal(hidden).astype(np.float32)
    want = exact_agg @ w.T.astype(np.float64)
    # the same layer evaluated in fp32 from the reference's fp32 aggregate: how far fp32 itself is from float64
    fp32_err = np.abs((want_agg @ w.T).astype(np.float64) - want).max()
    for bias, ref in ((dev(b), want + b), (None, want)):
        for block_rows, overlap in ((0, False), (512, False), (512, True)):
            got = host(lib.vq_decompress_spmm_csr_linear(c, cb, ip, ix, feat_dim, dev(w), bias, block_rows, overlap))
            assert np.allclose(got, ref, rtol=RTOL, atol=RTOL * np.abs(ref).max())
            # and no further from the float64 layer than twice an fp32 evaluation of it in another order
            assert np.abs(got - ref).max() <= 2 * fp32_err + 8 * np.spacing(np.float32(np.abs(ref).max()))


@pytest.mark.parametrize("bits", [4, 8])
def test_sq_linear_blocks_match_unblocked_aggregate(lib, bits):
    rng = np.random.default_rng(bits)
    n_src, rows, feat_dim = 4000, 2500, 100
    x = rng.uniform(-1, 1, size=(n_src, feat_dim)).astype(np.float32)
    cbs = np.stack([oc.sq_codebook(x)])
    codes = oc.sq_compress(x, cbs, bits, feat_dim)
    store = oc.sq_codes_to_storage(codes, bits).view(np.int8)
    indptr, indices = graph(rng, rows, n_src, 12, np.int64)
    c, cb, ip, ix = dev(store), dev(cbs), dev(indptr), dev(indices)
    whole = lib.sq_decompress_spmm_csr(c, cb, ip, ix, bits, feat_dim, feat_dim)
    eye = torch.eye(feat_dim, device="cuda")
    for block_rows in (0, 333, 2500):
        for overlap in (False, True):
            got = lib.sq_decompress_spmm_csr_linear(c, cb, ip, ix, bits, feat_dim, feat_dim, eye, None, block_rows,
                                                    overlap)
            assert torch.equal(got, whole), (block_rows, overlap)
    w = (rng.standard_normal((32, feat_dim)) / 10).astype(np.float32)
    b = rng.standard_normal(32).astype(np.float32)
    agg = oc.spmm_csr(oc.sq_decompress(store, cbs, bits, feat_dim, feat_dim), indptr, indices)
    want = agg.astype(np.float64) @ w.T.astype(np.float64) + b
    got = host(lib.sq_decompress_spmm_csr_linear(c, cb, ip, ix, bits, feat_dim, feat_dim, dev(w), dev(b), 700))
    assert np.allclose(got, want, rtol=RTOL, atol=RTOL * np.abs(want).max())
    fp32_err = np.abs((agg @ w.T + b).astype(np.float64) - want).max()
    assert np.abs(got - want).max() <= 2 * fp32_err + 8 * np.spacing(np.float32(np.abs(want).max()))


def test_linear_argument_errors(lib):
    rng = np.random.default_rng(3)
    codes = dev(rng.integers(0, 256, size=(50, 2), dtype=np.uint8))
    cb = dev(rng.standard_normal((2, 256, 4)).astype(np.float32))
    ip = dev(np.array([0, 2, 2, 5], dtype=np.int64))
    ix = dev(np.array([1, 2, 3, 4, 49], dtype=np.int64))
    good = torch.zeros((3, 8), device="cuda")
    assert lib.vq_decompress_spmm_csr_linear(codes, cb, ip, ix, 8, good).shape == (3, 3)
    with pytest.raises(RuntimeError, match="weight"):
        lib.vq_decompress_spmm_csr_linear(codes, cb, ip, ix, 8, torch.zeros((3, 7), device="cuda"))
    with pytest.raises(RuntimeError, match="bias"):
        lib.vq_decompress_spmm_csr_linear(codes, cb, ip, ix, 8, good, torch.zeros((4,), device="cuda"))
    with pytest.raises(RuntimeError, match="block_rows"):
        lib.vq_decompress_spmm_csr_linear(codes, cb, ip, ix, 8, good, None, -1)
    empty = lib.vq_decompress_spmm_csr_linear(codes, cb, ip[:1], ix[:0], 8, good)
    assert empty.shape == (0, 3)
