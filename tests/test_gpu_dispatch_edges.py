"""Shapes on either side of the thresholds that pick a workgroup size: the two-table kernel runs
one wave per workgroup at 8-32 edges per row and up to 128 columns and 256 threads otherwise, the
staged-rows kernel of the log-domain SQ runs 128 threads for 1/2-bit rows and 256 for 4/8-bit
ones.  Every side of every threshold must give the oracle's result."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from f2cgt_amd import capi

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def fixed_fanout(rng, rows, n_src, fanout, ragged):
    deg = np.full(rows, fanout, dtype=np.int64)
    if ragged:                                   # same mean, rows from empty to twice the fanout
        deg = rng.integers(0, 2 * fanout + 1, size=rows)
        deg[-1] += fanout * rows - deg.sum() if deg.sum() < fanout * rows else 0
    indptr = np.zeros(rows + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    return indptr, rng.integers(0, n_src, size=int(indptr[-1]))


@pytest.mark.parametrize("feat_dim", [128, 112, 144])
@pytest.mark.parametrize("fanout", [7, 8, 32, 33])
@pytest.mark.parametrize("ragged", [False, True])
def test_hybrid_on_both_sides_of_the_workgroup_thresholds(feat_dim, fanout, ragged):
    rng = np.random.default_rng(1000 * feat_dim + 10 * fanout + ragged)
    n, n_sq, w = 5000, 1200, 16
    n_cb = feat_dim // w
    row_map = np.empty(n, dtype=np.int32)
    row_map[:n_sq] = rng.permutation(n_sq)
    row_map[n_sq:] = -rng.permutation(n - n_sq) - 1
    sq_codes = rng.integers(0, 256, size=(n_sq, feat_dim), dtype=np.uint8)
    params = np.stack([rng.standard_normal(feat_dim) - 3, 0.01 + 0.02 * rng.random(feat_dim)]).astype(np.float32)
    vq_codes = rng.integers(0, 256, size=(n - n_sq, n_cb), dtype=np.uint8)
    vcb = rng.standard_normal((n_cb, 256, w)).astype(np.float32)
    indptr, indices = fixed_fanout(rng, 333, n, fanout, ragged)
    # most edges name SQ rows, as in the two-level scheme
    indices = np.where(rng.random(indices.shape[0]) < 0.9, indices % n_sq, indices)
    want = oc.hybrid_decompress_spmm_csr(row_map, sq_codes, params, vq_codes, vcb, indptr, indices, feat_dim)
    for idx in (np.int64, np.int32):
        got = capi.hybrid_decompress_spmm_csr(dev(row_map), dev(sq_codes), dev(params), dev(vq_codes), dev(vcb),
                                              dev(indptr.astype(idx)), dev(indices.astype(idx)), feat_dim)
        torch.cuda.synchronize()
        assert np.allclose(got.cpu().numpy(), want, rtol=RTOL, atol=RTOL * 8)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("feat_dim", [100, 128, 36])
def test_fused_log_sq_with_either_workgroup_size(bits, feat_dim):
    rng = np.random.default_rng(77 * bits + feat_dim)
    n = 4000
    src_dim = (feat_dim * bits + 7) // 8
    codes = rng.integers(0, 256, size=(n, src_dim), dtype=np.uint8)
    cb = np.array([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], dtype=np.float32)
    per = 8 // bits
    column_slice = (feat_dim + per - 1) // per * per        # one codebook, a multiple of the codes per byte
    for fanout, ragged in ((2, True), (12, False), (40, True)):
        indptr, indices = fixed_fanout(rng, 500, n, fanout, ragged)
        stored = codes.view(np.int8) if bits == 8 else codes
        want = oc.sq_decompress_spmm_csr(stored, cb, indptr, indices, bits, column_slice, feat_dim)
        got = capi.sq_decompress_spmm_csr(dev(stored), dev(cb), dev(indptr), dev(indices), bits, column_slice, feat_dim)
        torch.cuda.synchronize()
        assert np.allclose(got.cpu().numpy(), want, rtol=RTOL, atol=RTOL * 3.0)


@pytest.mark.parametrize("rows", [16383, 16384, 32767, 32768, 65535, 65536, 114687, 114688])
def test_fused_sq_on_both_sides_of_the_rows_per_block_steps(rows):
    # launches below ~2000 workgroups shrink their row blocks in steps of 8 rows: the integer-accumulating
    # kernel (affine, 128 threads) and the staged-rows kernel (log domain, 256 threads) at every step
    print("case rows-per-block steps rows=%d" % rows, flush=True)
    rng = np.random.default_rng(rows)
    n, d = 3000, 100
    deg = rng.integers(0, 5, size=rows)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n, size=int(indptr[-1]))
    raw = rng.integers(0, 16, size=(n, d), dtype=np.uint8)
    packed = oc.packbits(raw, 4)
    params = np.stack([rng.standard_normal(d), 0.01 + rng.random(d)]).astype(np.float32)
    got = capi.sq_affine_decompress_spmm_csr(dev(packed), dev(params), dev(indptr), dev(indices), 4, d)
    torch.cuda.synchronize()
    # the decode is affine in the code: the mean of the codes, then one scale and shift per output
    dec = oc.sq_affine_decompress(packed, params, 4, d)
    sums = np.zeros((rows, d), dtype=np.float64)
    np.add.at(sums, np.repeat(np.arange(rows), deg), dec[indices].astype(np.float64))
    want = (sums / np.maximum(deg, 1)[:, None]).astype(np.float32)
    assert np.allclose(got.cpu().numpy(), want, rtol=RTOL, atol=RTOL * np.abs(dec).max())
    cb = np.array([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], dtype=np.float32)
    got = capi.sq_decompress_spmm_csr(dev(packed), dev(cb), dev(indptr), dev(indices), 4, d, d)
    torch.cuda.synchronize()
    dec = oc.sq_decompress(packed, cb, 4, d, d)
    sums[:] = 0
    np.add.at(sums, np.repeat(np.arange(rows), deg), dec[indices].astype(np.float64))
    want = (sums / np.maximum(deg, 1)[:, None]).astype(np.float32)
    assert np.allclose(got.cpu().numpy(), want, rtol=RTOL, atol=RTOL * np.abs(dec).max())
