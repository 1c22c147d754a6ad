"""Shapes on either side of the thresholds that pick a workgroup size or a row partition: the two-table kernel runs
one wave per workgroup up to 32 edges per row and up to 128 columns, and beyond that the smallest workgroup (128 or
256 threads, 4 to 16 edges per thread) whose edge batch holds eight rows of the average length, the
staged-rows kernel of the log-domain SQ runs 128 threads for 1/2-bit rows and 256 for 4/8-bit
ones.  Every side of every threshold must give the oracle's result."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from parity_bars import assert_mean_aggregate
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


@pytest.mark.parametrize("feat_dim", [128, 112, 144, 48])
@pytest.mark.parametrize("fanout", [1, 2, 7, 8, 24, 25, 32, 33, 64, 65, 128, 129, 260])
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
    for fanout, ragged in ((2, True), (12, False), (20, False), (40, True), (60, False)):
        indptr, indices = fixed_fanout(rng, 500, n, fanout, ragged)
        stored = codes.view(np.int8) if bits == 8 else codes
        want = oc.sq_decompress_spmm_csr(stored, cb, indptr, indices, bits, column_slice, feat_dim)
        got = capi.sq_decompress_spmm_csr(dev(stored), dev(cb), dev(indptr), dev(indices), bits, column_slice, feat_dim)
        torch.cuda.synchronize()
        assert np.allclose(got.cpu().numpy(), want, rtol=RTOL, atol=RTOL * 3.0)


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("feat_dim", [602, 102, 66, 18, 14, 10])
def test_fused_sq_rows_of_an_even_number_of_columns_that_is_no_multiple_of_four(feat_dim, bits, idx):
    """602, 102 ... columns: output rows start at multiples of 8 bytes only and end with a group of two columns, code
    rows may end inside a byte group.  Affine and log-domain forms, staged and unstaged blocks (rows of 2, 12, 40 and
    300 edges on average), plain and streamed stores; many edges name the table's last row."""
    rng = np.random.default_rng(13 * feat_dim + bits + (idx == np.int32))
    n = 3000
    per = 8 // bits
    src_dim = (feat_dim + per - 1) // per
    codes = rng.integers(0, 256, size=(n, src_dim), dtype=np.uint8)
    if feat_dim % per:                                   # bits of a row's last byte beyond its columns stay 0
        codes[:, -1] &= (1 << (bits * (feat_dim % per))) - 1
    params = np.stack([rng.standard_normal(feat_dim) - 3, 0.01 + 0.02 * rng.random(feat_dim)]).astype(np.float32)
    cb = np.array([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], dtype=np.float32)
    column_slice = src_dim * per
    stored = codes.view(np.int8) if bits == 8 else codes
    for fanout, ragged in ((2, True), (12, False), (40, True), (300, True)):
        indptr, indices = fixed_fanout(rng, 400, n, fanout, ragged)
        indices[::5] = n - 1
        ip, ix = dev(indptr.astype(idx)), dev(indices.astype(idx))
        dec_a = oc.sq_affine_decompress(codes, params, bits, feat_dim).astype(np.float64)
        exact_a = oc.spmm_csr(dec_a, indptr, indices)
        want_a = oc.sq_affine_decompress_spmm_csr(codes, params, indptr, indices, bits, feat_dim)
        want_l = oc.sq_decompress_spmm_csr(stored, cb, indptr, indices, bits, column_slice, feat_dim)
        for mode in (capi.STORE_CACHED, capi.STORE_STREAM):
            was = capi.set_store_mode(mode)
            try:
                got_a = capi.sq_affine_decompress_spmm_csr(dev(codes), dev(params), ip, ix, bits, feat_dim)
                got_l = capi.sq_decompress_spmm_csr(dev(stored), dev(cb), ip, ix, bits, column_slice, feat_dim)
                torch.cuda.synchronize()
            finally:
                capi.set_store_mode(was)
            assert_mean_aggregate(got_a.cpu().numpy(), want_a, exact_a, float(np.abs(dec_a).max()))
            err = np.abs(got_l.cpu().numpy() - want_l).max()
            assert err <= RTOL * 3.0, (fanout, mode, float(err))


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


@pytest.mark.parametrize("mean_deg", [22, 45])
def test_fused_vq_chunk_dealing_with_shared_rows(mean_deg):
    """Above 16 edges per row on average the lane groups of a pass share a row (two or one row per
    mini-block); the same chunk dealing, sums no longer in edge order: rtol 1e-5."""
    rng = np.random.default_rng(mean_deg)
    rows, n_src, n_cb, width, feat_dim = 256 * 200 + 9, 20000, 16, 8, 128
    codes = rng.integers(0, 256, size=(n_src, n_cb), dtype=np.uint8)
    cbs = rng.standard_normal((n_cb, 256, width)).astype(np.float32)
    deg = rng.integers(0, 2 * mean_deg + 1, size=rows)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1]))
    got = capi.vq_decompress_spmm_csr(dev(codes), dev(cbs), dev(indptr), dev(indices), feat_dim)
    full = capi.spmm_csr(capi.vq_decompress(dev(codes), dev(cbs), feat_dim), dev(indptr), dev(indices))
    torch.cuda.synchronize()
    scale = float(full.abs().max())
    assert torch.allclose(got, full, rtol=RTOL, atol=RTOL * scale)
    sample = np.unique(np.concatenate([np.arange(30), np.arange(rows - 30, rows), rng.integers(0, rows, size=200)]))
    sub_ptr = np.zeros(len(sample) + 1, dtype=np.int64)
    sub_ptr[1:] = np.cumsum(deg[sample])
    sub_idx = np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in sample]).astype(np.int64)
    want = oc.vq_decompress_spmm_csr(codes, cbs, sub_ptr, sub_idx, feat_dim)
    assert np.allclose(got.cpu().numpy()[sample], want, rtol=RTOL, atol=RTOL * np.abs(want).max())


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("feat_dim,n_cb,width", [(100, 13, 8), (64, 8, 8), (96, 12, 8), (192, 24, 8), (160, 5, 32),
                                                 (96, 3, 32), (48, 3, 16), (200, 13, 16), (100, 4, 32), (600, 19, 32),
                                                 (120, 16, 8), (602, 19, 32), (102, 13, 8), (50, 7, 8), (90, 3, 32),
                                                 (30, 4, 8), (130, 17, 8), (258, 17, 16)])
@pytest.mark.parametrize("mean_deg", [3, 12, 40])
def test_fused_vq_code_rows_that_are_no_multiple_of_a_tile(feat_dim, n_cb, width, mean_deg, idx):
    """Code rows of 13, 8, 12, 24 ... bytes where a 128-column tile takes 16 (8, 4) of them: the pipelined kernel
    fetches its code words at any alignment and reads the table's last rows byte by byte.  Many edges name the last two
    source rows; feat_dim may be less than n_cb * width (the reference's truncation).  Output rows of an even number
    of columns that is no multiple of four (602, 102, 50 ...) are only 8-byte aligned: they are written in 8-byte
    pairs, the last pair of a row possibly alone in its group of four."""
    rng = np.random.default_rng(feat_dim * 100 + mean_deg + (idx == np.int32))
    n_src, rows = 777, 3000
    codes = rng.integers(0, 256, size=(n_src, n_cb), dtype=np.uint8)
    cbs = rng.standard_normal((n_cb, 256, width)).astype(np.float32)
    deg = rng.integers(0, 2 * mean_deg + 1, size=rows)
    indptr = np.zeros(rows + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1])).astype(idx)
    indices[::7] = n_src - 1
    indices[1::11] = n_src - 2
    got = capi.vq_decompress_spmm_csr(dev(codes), dev(cbs), dev(indptr), dev(indices), feat_dim)
    torch.cuda.synchronize()
    want = oc.vq_decompress_spmm_csr(codes, cbs, indptr.astype(np.int64), indices.astype(np.int64), feat_dim)
    dec = oc.vq_decompress(codes, cbs, feat_dim).astype(np.float64)
    exact = oc.spmm_csr(dec, indptr.astype(np.int64), indices.astype(np.int64))
    assert_mean_aggregate(got.cpu().numpy(), want, exact, float(np.abs(dec).max()))


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("feat_dim,n_cb,width", [(128, 16, 8), (136, 17, 8), (200, 25, 8), (200, 13, 16), (264, 33, 8),
                                                 (512, 16, 32), (160, 5, 32), (328, 41, 8), (256, 16, 16), (96, 6, 16),
                                                 (96, 3, 32), (224, 7, 32)])
@pytest.mark.parametrize("fanout,ragged", [(9, False), (10, True), (11, False), (14, True), (20, False), (40, True)])
def test_fused_vq_halves_exchanged_inside_lane_quads(feat_dim, n_cb, width, fanout, ragged, idx):
    """Nine to eleven edges per row from a small code table: the two 16-byte halves of a lane's eight columns are
    exchanged inside lane quads so that a store instruction writes whole 64-byte pieces.  Last tiles of 8, 72 and 32
    columns leave quads with one, two or three lanes beyond the columns, whose pieces must not be stored; 13 x 16 and
    5 x 32 are code rows that are no multiple of a tile; the last tile of 328 columns is 72 columns wide.  With
    codebooks of 32 (16) columns and rows of whole such groups the four (two) lanes that share a code own its columns
    together instead, at every row length (four-, two- and one-row mini-blocks)."""
    rng = np.random.default_rng(feat_dim * 31 + fanout + (idx == np.int32))
    n_src, rows = 5000, 2500
    codes = rng.integers(0, 256, size=(n_src, n_cb), dtype=np.uint8)
    cbs = rng.standard_normal((n_cb, 256, width)).astype(np.float32)
    indptr, indices = fixed_fanout(rng, rows, n_src, fanout, ragged)
    indices[::9] = n_src - 1
    got = capi.vq_decompress_spmm_csr(dev(codes), dev(cbs), dev(indptr.astype(idx)), dev(indices.astype(idx)), feat_dim)
    torch.cuda.synchronize()
    want = oc.vq_decompress_spmm_csr(codes, cbs, indptr, indices, feat_dim)
    dec = oc.vq_decompress(codes, cbs, feat_dim).astype(np.float64)
    exact = oc.spmm_csr(dec, indptr, indices)
    assert_mean_aggregate(got.cpu().numpy(), want, exact, float(np.abs(dec).max()))
    # the streaming store mode turns the results round in LDS at these row lengths too: same sums, bit for bit
    was = capi.set_store_mode(capi.STORE_STREAM)
    try:
        streamed = capi.vq_decompress_spmm_csr(dev(codes), dev(cbs), dev(indptr.astype(idx)), dev(indices.astype(idx)),
                                               feat_dim)
        torch.cuda.synchronize()
    finally:
        capi.set_store_mode(was)
    assert torch.equal(got, streamed)


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("n_cb,width", [(16, 8), (6, 32)])
@pytest.mark.parametrize("mean_deg", [10, 16, 25, 32, 50, 100, 300])
def test_fused_vq_rows_and_mini_blocks_longer_than_the_staging(mean_deg, n_cb, width, idx):
    """Four-, two- and one-row mini-blocks (up to 16 / 32 / beyond edges per row on average) whose edges exceed the 64
    a wave stages go through the staging in slices: ragged rows around the average, rows of 65, 128, 129 and 700 edges,
    empty rows, and uniform rows at the limits (16, 32) where every mini-block is exactly full."""
    rng = np.random.default_rng(1000 * mean_deg + n_cb + (idx == np.int32))
    feat_dim = n_cb * width
    rows, n_src = 16 * 12 * 9 + 7, 30000
    codes = rng.integers(0, 256, size=(n_src, n_cb), dtype=np.uint8)
    cbs = rng.standard_normal((n_cb, 256, width)).astype(np.float32)
    if mean_deg in (16, 32):
        deg = np.full(rows, mean_deg)
    else:
        deg = rng.integers(0, 2 * mean_deg + 1, size=rows)
        deg[[3, 50, 51, 400]] = [65, 128, 129, 700]
        deg[rng.integers(0, rows, size=rows // 20)] = 0
    indptr = np.zeros(rows + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1])).astype(idx)
    got = capi.vq_decompress_spmm_csr(dev(codes), dev(cbs), dev(indptr), dev(indices), feat_dim)
    torch.cuda.synchronize()
    want = oc.vq_decompress_spmm_csr(codes, cbs, indptr.astype(np.int64), indices.astype(np.int64), feat_dim)
    dec = oc.vq_decompress(codes, cbs, feat_dim).astype(np.float64)
    exact = oc.spmm_csr(dec, indptr.astype(np.int64), indices.astype(np.int64))
    assert_mean_aggregate(got.cpu().numpy(), want, exact, float(np.abs(dec).max()))
    assert not got.cpu().numpy()[deg == 0].any()


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("rows", [256 * 191 + 3, 256 * 192, 256 * 192 + 1, 256 * 205 + 7, 256 * 12 * 17 + 5])
def test_fused_vq_on_both_sides_of_the_chunk_dealing_threshold(rows, idx):
    """The fused VQ kernel gives every wave one piece of its workgroup's rows while a workgroup has
    fewer than 16 x 12 rows and deals 12-row chunks among the waves from there on: row counts on
    either side of that step, last chunks of one to twelve rows, empty rows, and rows with more
    edges than a wave stages (summed straight from memory).  Edge order is kept; the mean is the sum
    times a refined reciprocal, so the result is the oracle's to 2 ulp."""
    rng = np.random.default_rng(rows % 100003)
    n_src, n_cb, width, feat_dim = 20000, 16, 8, 128
    codes = rng.integers(0, 256, size=(n_src, n_cb), dtype=np.uint8)
    cbs = rng.standard_normal((n_cb, 256, width)).astype(np.float32)
    deg = rng.integers(0, 11, size=rows)
    heavy = rng.integers(0, rows, size=40)
    deg[heavy] = rng.integers(65, 120, size=40)          # more than the 64 staged edges of a mini-block
    deg[rng.integers(0, rows, size=rows // 20)] = 0
    indptr = np.zeros(rows + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1])).astype(idx)
    got = capi.vq_decompress_spmm_csr(dev(codes), dev(cbs), dev(indptr), dev(indices), feat_dim)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    tag = capi.DT_I64 if idx == np.int64 else capi.DT_I32
    rc, plan = capi.dry_run("f2cgt_vq_decompress_spmm_csr", 16, capi.DT_U8, 16, 16, 16, tag, 16, rows, int(indptr[-1]),
                            n_src, feat_dim, n_cb, 256, width, None)
    assert rc == 0 and plan.kernel == b"vq_wave_kernel"
    # the oracle on a sample of rows (first, last, around every workgroup boundary, the heavy ones)
    per_wg = -(-rows // 256)
    sample = np.unique(np.clip(np.concatenate([
        np.arange(0, 40), np.arange(rows - 40, rows), heavy,
        (np.arange(1, 256)[:, None] * (-(-per_wg // 12) * 12) + np.arange(-2, 3)[None, :]).ravel(),
        rng.integers(0, rows, size=400)]), 0, rows - 1))
    sub_ptr = np.zeros(len(sample) + 1, dtype=np.int64)
    sub_ptr[1:] = np.cumsum(deg[sample])
    sub_idx = np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in sample]).astype(np.int64)
    want = oc.vq_decompress_spmm_csr(codes, cbs, sub_ptr, sub_idx, feat_dim)
    dec = oc.vq_decompress(codes, cbs, feat_dim)
    exact = oc.spmm_csr(dec.astype(np.float64), sub_ptr, sub_idx)
    assert_mean_aggregate(got[sample], want, exact, np.abs(dec).max(), deg[sample])
    # every row against the unfused composition on the device (the reference's order and division)
    full = capi.spmm_csr(capi.vq_decompress(dev(codes), dev(cbs), feat_dim), dev(indptr), dev(indices)).cpu().numpy()
    scale = np.maximum(np.abs(full).max(axis=1, keepdims=True), 1e-30)
    assert np.all(np.abs(got - full) <= 1e-5 * scale)
    assert np.array_equal(got[deg <= 1], full[deg <= 1])
