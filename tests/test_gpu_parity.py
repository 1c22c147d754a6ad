"""Parity of the HIP library (through the C ABI, and through the F2CGTLib module) with
the CPU oracle on seeded inputs.  Integer/byte results and decodes are bit-exact;
aggregations use rtol 1e-5 (they are bit-exact too wherever the kernel keeps the
sequential edge order, which is asserted where it holds)."""
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


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def random_graph(rng, rows, n_src, max_deg, idx=np.int64, empty_rows=True):
    deg = rng.integers(0 if empty_rows else 1, max_deg + 1, size=rows)
    indptr = np.zeros(rows + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1])).astype(idx)
    return indptr, indices


def close(got, want, atol_scale=1.0):
    scale = float(np.abs(want).max()) if want.size else 1.0
    return np.allclose(got, want, rtol=RTOL, atol=RTOL * scale * atol_scale)


# ---- golden fixtures ----------------------------------------------------------------------
def test_golden_fixtures(golden):
    g = golden
    for bits in (1, 2, 4):
        assert np.array_equal(host(capi.packbits(dev(g["pack%d_in" % bits]), bits)), g["pack%d_out" % bits])
        assert np.array_equal(host(capi.unpackbits(dev(g["pack%d_out" % bits]), bits, 13)),
                              g["unpack%d_out" % bits])
    cbs = dev(g["sq_codebooks"])
    ip, ix = dev(g["g_indptr"]), dev(g["g_indices"])
    for bits in (1, 2, 4, 8, 16):
        assert np.array_equal(host(capi.sq_compress(dev(g["sq_x"]), cbs, bits, 12)), g["sq%d_codes" % bits])
        store = dev(g["sq%d_store" % bits])
        assert np.array_equal(host(capi.sq_decompress(store, cbs, bits, 12, 24)), g["sq%d_decoded" % bits])
        fused = host(capi.sq_decompress_spmm_csr(store[:3].contiguous(), cbs, ip, ix, bits, 12, 24))
        assert np.array_equal(fused, g["g_sq%d_fused" % bits])
    assert np.array_equal(host(capi.vq_decompress(dev(g["vq_idx"]), dev(g["vq_codebooks"]), 10)), g["vq_decoded"])
    assert np.array_equal(host(capi.vq_decompress_spmm_csr(dev(g["vq_idx"]), dev(g["vq_codebooks"]), ip, ix, 10)),
                          g["g_vq_fused"])
    assert np.array_equal(host(capi.spmm_csr(dev(g["g_feat"]), ip, ix)), g["g_spmm"])
    for bits in (4, 8):
        store, params = dev(g["aff%d_store" % bits]), dev(g["aff%d_params" % bits])
        assert np.array_equal(host(capi.sq_affine_decompress(store, params, bits, 10)), g["aff%d_decoded" % bits])
        # 4/8-bit affine aggregation sums integer codes (exact) instead of decoded floats:
        # equal up to fp32 rounding of the summands
        assert close(host(capi.sq_affine_decompress_spmm_csr(store, params, ip, ix, bits, 10)),
                     g["g_aff%d_fused" % bits])
    hy = host(capi.hybrid_decompress_spmm_csr(dev(g["hy_map"]), dev(g["hy_sq"]), dev(g["hy_params"]),
                                              dev(g["hy_vq"]), dev(g["hy_cb"]), dev(g["hy_indptr"]),
                                              dev(g["hy_indices"]), 8))
    assert close(hy, g["hy_fused"])  # SQ part summed as integers: equal up to fp32 rounding
    for metric in ("l2", "cosine"):
        d = host(capi.pairwise_distance(dev(g["enc_x"]), dev(g["enc_c"]), metric))
        assert np.allclose(d, g["enc_dist_" + metric], rtol=1e-5, atol=1e-5)
        assert np.array_equal(host(capi.kmeans_predict(dev(g["enc_x"]), dev(g["enc_c"]), metric)),
                              g["enc_labels_" + metric])
        d = host(capi.pairwise_distance(dev(g["enc24_x"]), dev(g["enc24_c"]), metric))
        assert np.allclose(d, g["enc24_dist_" + metric], rtol=1e-5, atol=1e-6)
    ft, fi = dev(g["fetch_table"]), dev(g["fetch_index"])
    assert np.array_equal(host(capi.fetch_rows(ft, fi)), g["fetch_plain"])
    assert np.array_equal(host(capi.fetch_rows(ft, fi, dev(g["fetch_hot"]), dev(g["fetch_slot"]))), g["fetch_cached"])


# ---- packbits / unpackbits -------------------------------------------------------------------
@pytest.mark.parametrize("bits", [1, 2, 4])
@pytest.mark.parametrize("shape", [(0, 8), (1, 1), (3, 13), (257, 100), (1000, 128), (5, 1031), (4099, 50)])
def test_pack_unpack_bit_exact(bits, shape):
    rng = np.random.default_rng(bits * 1000 + shape[0] + shape[1])
    u = rng.integers(0, 256, size=shape, dtype=np.uint8)
    want = oc.packbits(u, bits)
    got = host(capi.packbits(dev(u), bits))
    assert got.shape == want.shape and np.array_equal(got, want)
    back = host(capi.unpackbits(dev(want), bits, shape[1]))
    assert np.array_equal(back, oc.unpackbits(want, bits, shape[1]))
    assert np.array_equal(back, u & ((1 << bits) - 1))


def test_pack_large_roundtrip_property():
    # C2 table shape: [2.4e6, 100] 4-bit codes -> [2.4e6, 50]
    g = torch.Generator(device="cuda").manual_seed(0)
    u = torch.randint(0, 16, (2_400_000, 100), generator=g, device="cuda", dtype=torch.uint8)
    p = capi.packbits(u, 4)
    assert p.shape == (2_400_000, 50)
    assert torch.equal(capi.unpackbits(p, 4, 100), u)
    assert torch.equal(p, (u[:, 0::2] | (u[:, 1::2] << 4)))


# ---- SQ encode / decode ------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [1, 2, 4, 8, 16])
def test_sq_compress_decompress_bit_exact(bits):
    # shapes of tests/test_sq.py: 10000 x 200 single codebook; (60+50) two codebooks
    rng = np.random.default_rng(bits)
    x = rng.uniform(-1, 1, size=(10000, 200)).astype(np.float32)
    x[0, :4] = [0.0, -0.0, 1e-9, 5.0]
    cb = np.stack([oc.sq_codebook(x)])
    codes = oc.sq_compress(x, cb, bits, 200)
    got = host(capi.sq_compress(dev(x), dev(cb), bits, 200))
    assert np.array_equal(got, codes)
    store = oc.sq_codes_to_storage(codes, bits)
    dec = host(capi.sq_decompress(dev(store), dev(cb), bits, 200, 200))
    assert np.array_equal(dec, oc.sq_decompress(store, cb, bits, 200, 200))

    a = rng.uniform(-1, 1, size=(3000, 60)).astype(np.float32)
    b = (rng.uniform(-1, 1, size=(3000, 50)) + 10).astype(np.float32)
    x2 = np.concatenate([a, b], axis=1)
    cbs = np.stack([oc.sq_codebook(a), oc.sq_codebook(b)])
    codes2 = oc.sq_compress(x2, cbs, bits, 60)
    assert np.array_equal(host(capi.sq_compress(dev(x2), dev(cbs), bits, 60)), codes2)
    store2 = oc.sq_codes_to_storage(codes2, bits)
    dec2 = host(capi.sq_decompress(dev(store2), dev(cbs), bits, 60, 110))
    assert np.array_equal(dec2, oc.sq_decompress(store2, cbs, bits, 60, 110))


@pytest.mark.parametrize("bits", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("d,cs", [(200, 200), (110, 60), (13, 5)])
def test_sq_encode_is_compress_cast_pack(bits, d, cs):
    rng = np.random.default_rng(bits * 100 + d)
    x = rng.uniform(-2, 2, size=(3001, d)).astype(np.float32)
    x[0, :4] = [0.0, -0.0, 1e-9, 5.0]
    cbs = np.stack([oc.sq_codebook(x[:, s:s + cs]) for s in range(0, d, cs)])
    want = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, cs), bits)
    got = host(capi.sq_encode(dev(x), dev(cbs), bits, cs))
    assert got.shape == want.shape
    assert np.array_equal(got.view(want.dtype) if got.dtype != want.dtype else got, want)
    # and equals the three-call sequence on the GPU
    codes = capi.sq_compress(dev(x), dev(cbs), bits, cs)
    if bits < 8:
        three = host(capi.packbits(codes.to(torch.uint8), bits))
    else:
        three = host(codes.to(torch.int8 if bits == 8 else torch.int16))
    assert np.array_equal(got.view(three.dtype), three)


@pytest.mark.parametrize("bits", [2, 4, 8, 16])
def test_sq_encode_values_on_bucket_edges(bits):
    # the encoder decides most buckets from a hardware logarithm with an error bound; magnitudes
    # placed on and next to every bucket edge, and around 1.0 where log2 changes sign, are the
    # ones that bound has to hand to the exact path
    rng = np.random.default_rng(bits)
    base = rng.uniform(-3, 3, size=(4096, 64)).astype(np.float32)
    cb = np.stack([oc.sq_codebook(base)])
    emin, emax = float(cb[0, 2]), float(cb[0, 3])
    n_edges = min(1 << (bits - 1), 4096)
    j = np.linspace(0, 1 << (bits - 1), n_edges + 1)
    edge = np.exp2(emin + j * (emax - emin) / (1 << (bits - 1))).astype(np.float32)
    near = [edge]
    for _ in range(4):
        near.append(np.nextafter(near[-1], np.float32(np.inf)))
    lo = edge
    for _ in range(4):
        lo = np.nextafter(lo, np.float32(0))
        near.append(lo)
    one = np.float32(1.0) + np.arange(-32, 33, dtype=np.float32) * np.float32(2.0 ** -24)
    vals = np.concatenate(near + [one])
    vals = np.concatenate([vals, -vals])
    pad = (-len(vals)) % 64
    x = np.concatenate([vals, np.zeros(pad, np.float32)]).reshape(-1, 64)
    want = oc.sq_compress(x, cb, bits, 64)
    assert np.array_equal(host(capi.sq_compress(dev(x), dev(cb), bits, 64)), want)
    got = host(capi.sq_encode(dev(x), dev(cb), bits, 64))
    store = oc.sq_codes_to_storage(want, bits)
    assert np.array_equal(got.view(store.dtype), store)


@pytest.mark.parametrize("bits", [2, 4, 8, 16])
def test_sq_decompress_every_code(bits):
    n = 1 << bits
    raw = np.arange(n, dtype=np.int64)
    cbs = np.array([[0.01, 3.0, np.log2(0.01), np.log2(3.0) + 1e-5, 0.4],
                    [1e-5, 900.0, np.log2(1e-5), np.log2(900.0), 0.2]], dtype=np.float32)
    if bits < 8:
        store = oc.packbits(np.concatenate([raw, raw]).astype(np.uint8)[None, :], bits)
    elif bits == 8:
        store = np.concatenate([raw, raw]).astype(np.uint8).view(np.int8)[None, :]
    else:
        store = np.concatenate([raw, raw]).astype(np.uint16).view(np.int16)[None, :]
    want = oc.sq_decompress(store, cbs, bits, n, 2 * n)
    got = host(capi.sq_decompress(dev(store), dev(cbs), bits, n, 2 * n))
    assert np.array_equal(got, want)
    assert np.array_equal(want[0, :n], oc.sq_lut(cbs, bits)[0])


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("d,cs", [(602, 304), (102, 102), (66, 40)])
def test_sq_decompress_rows_of_4k_plus_2_columns(bits, d, cs):
    """Even widths that are no multiple of four: output rows start at multiples of 8 bytes only and end with a group of
    two columns; the last source row's code bytes end with the table."""
    rng = np.random.default_rng(bits * 1000 + d)
    x = (rng.standard_normal((3001, d)) * rng.uniform(0.5, 2, size=d)).astype(np.float32)
    n_cb = (d + cs - 1) // cs
    cbs = np.stack([oc.sq_codebook(x[:, i * cs:(i + 1) * cs]) for i in range(n_cb)])
    store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, cs), bits)
    got = host(capi.sq_decompress(dev(store), dev(cbs), bits, cs, d))
    assert np.array_equal(got, oc.sq_decompress(store, cbs, bits, cs, d))


def test_sq_decompress_accepts_int8_storage():
    rng = np.random.default_rng(9)
    x = rng.uniform(-1, 1, size=(100, 64)).astype(np.float32)
    cb = np.stack([oc.sq_codebook(x)])
    store = oc.sq_codes_to_storage(oc.sq_compress(x, cb, 4, 64), 4)
    a = host(capi.sq_decompress(dev(store), dev(cb), 4, 64, 64))
    b = host(capi.sq_decompress(dev(store.view(np.int8)), dev(cb), 4, 64, 64))
    assert np.array_equal(a, b)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("d", [10, 100, 128, 102, 602, 66])
def test_sq_affine_decompress_bit_exact(bits, d):
    rng = np.random.default_rng(bits * 10 + d)
    x = (rng.standard_normal((2000, d)) * rng.uniform(0.5, 2, size=d)).astype(np.float32)
    params = oc.sq_affine_params(x, bits)
    codes = oc.sq_affine_compress(x, params, bits)
    store = oc.packbits(codes, bits) if bits < 8 else codes
    got = host(capi.sq_affine_decompress(dev(store), dev(params), bits, d))
    assert np.array_equal(got, oc.sq_affine_decompress(store, params, bits, d))


# ---- VQ decode ----------------------------------------------------------------------------------
@pytest.mark.parametrize("cdt", [np.uint8, np.int8, np.int16])
@pytest.mark.parametrize("cbdt", [np.float32, np.float16])
def test_vq_decompress_dtypes(cdt, cbdt):
    rng = np.random.default_rng(0)
    K = 100 if cdt == np.int8 else (700 if cdt == np.int16 else 256)
    cb = rng.standard_normal((4, K, 8)).astype(cbdt)
    idx = rng.integers(0, K, size=(3000, 4)).astype(cdt)
    for feat_dim in (32, 27):
        got = host(capi.vq_decompress(dev(idx), dev(cb), feat_dim))
        assert np.array_equal(got, oc.vq_decompress(idx, cb, feat_dim))


def test_vq_decompress_reference_shapes():
    # tests/test_vq.py: 1 codebook x 128 wide; (60 | 50 zero padded to 60) two codebooks
    rng = np.random.default_rng(1)
    cb = rng.uniform(-5, 5, size=(1, 256, 128)).astype(np.float32)
    idx = rng.integers(0, 256, size=(100000, 1), dtype=np.uint8)
    got = capi.vq_decompress(dev(idx), dev(cb), 128)
    want = torch.index_select(dev(cb[0]), 0, dev(idx[:, 0]).long())
    assert torch.equal(got, want)
    cb2 = np.zeros((2, 256, 60), dtype=np.float32)
    cb2[0] = rng.uniform(-5, 5, size=(256, 60))
    cb2[1, :, :50] = rng.uniform(-10, 10, size=(256, 50))
    idx2 = rng.integers(0, 256, size=(50000, 2), dtype=np.uint8)
    got2 = host(capi.vq_decompress(dev(idx2), dev(cb2), 110))
    assert np.array_equal(got2, oc.vq_decompress(idx2, cb2, 110))


def test_vq_decompress_codebook_larger_than_lds():
    rng = np.random.default_rng(2)
    cb = rng.standard_normal((24, 256, 32)).astype(np.float32)  # 768 KB
    idx = rng.integers(0, 256, size=(2000, 24), dtype=np.uint8)
    got = host(capi.vq_decompress(dev(idx), dev(cb), 768))
    assert np.array_equal(got, oc.vq_decompress(idx, cb, 768))


@pytest.mark.parametrize("shape", [(16, 256, 8, 128, 5077), (8, 64, 16, 100, 3001), (25, 256, 4, 100, 1024),
                                   (24, 200, 32, 768, 2049), (2, 256, 64, 128, 4096), (16, 256, 8, 64, 1500),
                                   (19, 256, 32, 602, 2049), (13, 256, 8, 102, 3001), (17, 64, 8, 130, 1100),
                                   (9, 256, 8, 66, 1500)])
def test_vq_decompress_tile_path(shape):
    # uint8 codes + fp32 codebooks of a width dividing 128: the persistent LDS-tile kernel, with
    # row counts that leave a remainder after the last full 256-row step
    n_cb, K, w, feat_dim, rows = shape
    rng = np.random.default_rng(rows)
    cb = rng.standard_normal((n_cb, K, w)).astype(np.float32)
    idx = rng.integers(0, K, size=(rows, n_cb), dtype=np.uint8)
    idx[::97, 0] = 255   # codes >= K read entry K - 1, as in the generic kernel
    got = host(capi.vq_decompress(dev(idx), dev(cb), feat_dim))
    want = oc.vq_decompress(np.minimum(idx, K - 1), cb, feat_dim)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_sq_affine_decompress_padded_storage(bits):
    # storage rows wider than the decoded columns need (odd byte pitch: rows are not word aligned)
    rng = np.random.default_rng(bits)
    d = 72
    x = rng.standard_normal((3000, d)).astype(np.float32)
    params = oc.sq_affine_params(x, bits)
    codes = oc.sq_affine_compress(x, params, bits)
    store = oc.packbits(codes, bits) if bits < 8 else codes
    wide = np.concatenate([store, rng.integers(0, 256, size=(3000, 5), dtype=np.uint8)], axis=1)
    got = host(capi.sq_affine_decompress(dev(wide), dev(params), bits, d))
    assert np.array_equal(got, oc.sq_affine_decompress(store, params, bits, d))


# ---- plain CSC mean ---------------------------------------------------------------------------
@pytest.mark.parametrize("idx", [np.int32, np.int64])
@pytest.mark.parametrize("d", [1, 7, 100, 128, 300, 2, 6, 102, 602])
def test_spmm_csr_f32(idx, d):
    rng = np.random.default_rng(d)
    feat = rng.standard_normal((1000, d)).astype(np.float32)
    indptr, indices = random_graph(rng, 700, 1000, 17, idx)
    got = host(capi.spmm_csr(dev(feat), dev(indptr), dev(indices)))
    want = oc.spmm_csr(feat, indptr, indices)
    assert np.array_equal(got, want)  # sequential edge order is kept
    # a feature matrix that starts 4 bytes off an 8-byte boundary takes the one-column-per-lane form
    flat = torch.zeros(feat.size + 1, dtype=torch.float32, device="cuda")
    flat[1:] = dev(feat).reshape(-1)
    got = host(capi.spmm_csr(flat[1:].view(1000, d), dev(indptr), dev(indices)))
    assert np.array_equal(got, want)


def test_spmm_csr_f16_f64_and_empty():
    rng = np.random.default_rng(3)
    indptr, indices = random_graph(rng, 300, 500, 9)
    f64 = rng.standard_normal((500, 33))
    got = host(capi.spmm_csr(dev(f64), dev(indptr), dev(indices)))
    assert np.array_equal(got, oc.spmm_csr(f64, indptr, indices))
    f16 = rng.standard_normal((500, 33)).astype(np.float16)
    # half features: the sum is rounded to half after every edge, as the reference's DType accumulator is
    got16 = host(capi.spmm_csr(dev(f16), dev(indptr), dev(indices)))
    assert got16.dtype == np.float16 and np.array_equal(got16, oc.spmm_csr(f16, indptr, indices))
    # no rows, no edges
    e = capi.spmm_csr(dev(f64.astype(np.float32)), dev(np.zeros(1, np.int64)), dev(np.zeros(0, np.int64)))
    assert e.shape == (0, 33)
    z = host(capi.spmm_csr(dev(f64.astype(np.float32)), dev(np.zeros(6, np.int64)), dev(np.zeros(0, np.int64))))
    assert z.shape == (5, 33) and not z.any()


# ---- fused VQ ---------------------------------------------------------------------------------
def test_fused_vq_reference_literal_case():
    # tests/test_fusion_decompress_spmm.py:19-33: fused == spmm_csr(vq_decompress(.)), bit for bit
    rng = np.random.default_rng(4)
    indptr = dev(np.array([0, 1, 3, 6], dtype=np.int64))
    indices = dev(np.array([0, 1, 1, 2, 2, 0], dtype=np.int64))
    cb = dev(rng.standard_normal((1, 256, 100)).astype(np.float32))
    codes = dev(rng.integers(0, 256, size=(6, 1), dtype=np.uint8))
    out1 = capi.spmm_csr(capi.vq_decompress(codes, cb, 100), indptr, indices)
    out2 = capi.vq_decompress_spmm_csr(codes, cb, indptr, indices, 100)
    assert torch.equal(out1, out2)


@pytest.mark.parametrize("idx", [np.int32, np.int64])
@pytest.mark.parametrize("shape", [(16, 256, 8, 128), (16, 256, 8, 100), (8, 256, 16, 128), (24, 256, 32, 768),
                                   (3, 16, 4, 10), (1, 256, 100, 100), (5, 64, 6, 29)])
def test_fused_vq_vs_oracle(idx, shape):
    n_cb, K, w, feat_dim = shape
    rng = np.random.default_rng(n_cb * 7 + w)
    N, R = 5000, 1500
    cb = rng.standard_normal((n_cb, K, w)).astype(np.float32)
    codes = rng.integers(0, K, size=(N, n_cb), dtype=np.uint8)
    indptr, indices = random_graph(rng, R, N, 20, idx)
    got = host(capi.vq_decompress_spmm_csr(dev(codes), dev(cb), dev(indptr), dev(indices), feat_dim))
    want = oc.vq_decompress_spmm_csr(codes, cb, indptr, indices, feat_dim)
    dec = oc.vq_decompress(codes, cb, feat_dim)
    exact = oc.spmm_csr(dec.astype(np.float64), indptr.astype(np.int64), indices.astype(np.int64))
    assert_mean_aggregate(got, want, exact, np.abs(dec).max(), np.diff(indptr.astype(np.int64)))
    unfused = host(capi.spmm_csr(capi.vq_decompress(dev(codes), dev(cb), feat_dim), dev(indptr), dev(indices)))
    assert np.array_equal(unfused, want)       # the unfused composition is the reference's order and division


@pytest.mark.parametrize("max_deg,rows", [(50, 1500), (200, 700), (3, 4099)])
def test_fused_vq_degree_regimes(max_deg, rows):
    # average degree up to 15: wave-granular pipeline with 4-row mini-blocks, with a row count that
    # leaves partial chunks and mini-blocks; above 60: block-synchronous pipeline (blocks above 1024
    # edges summed from HBM).  Both keep the sequential edge order and take the mean as sum * (1 / n)
    # with a refined reciprocal (within 2 ulp of the reference's division).  In between (max_deg 50:
    # about 25 per row) two or four lane groups share a row and their partial sums are added, so the
    # order differs as well.  The bar for all of them: 1e-5 of the row's magnitude, no further from
    # the float64 mean than the reference's own fp32 evaluation, single-neighbour rows bit-exact.
    rng = np.random.default_rng(max_deg)
    N = 3000
    cb = rng.standard_normal((16, 256, 8)).astype(np.float32)
    codes = rng.integers(0, 256, size=(N, 16), dtype=np.uint8)
    indptr, indices = random_graph(rng, rows, N, max_deg)
    got = host(capi.vq_decompress_spmm_csr(dev(codes), dev(cb), dev(indptr), dev(indices), 128))
    want = oc.vq_decompress_spmm_csr(codes, cb, indptr, indices, 128)
    dec = oc.vq_decompress(codes, cb, 128)
    exact = oc.spmm_csr(dec.astype(np.float64), indptr, indices)
    assert_mean_aggregate(got, want, exact, np.abs(dec).max(), np.diff(indptr))


@pytest.mark.parametrize("fanout,rows", [(20, 1003), (27, 515), (45, 300), (60, 130)])
def test_fused_vq_shared_rows(fanout, rows):
    # fixed fanouts of the 2-row and 1-row mini-block modes, wide features (two column tiles),
    # int32 indices, rows that do not fill the last mini-block
    rng = np.random.default_rng(fanout)
    N = 5000
    cb = rng.standard_normal((32, 256, 8)).astype(np.float32)
    codes = rng.integers(0, 256, size=(N, 32), dtype=np.uint8)
    indptr = (np.arange(rows + 1) * fanout).astype(np.int32)
    indices = rng.integers(0, N, size=rows * fanout).astype(np.int32)
    got = host(capi.vq_decompress_spmm_csr(dev(codes), dev(cb), dev(indptr), dev(indices), 256))
    want = oc.vq_decompress_spmm_csr(codes, cb, indptr.astype(np.int64), indices.astype(np.int64), 256)
    dec = oc.vq_decompress(codes, cb, 256)
    exact = oc.spmm_csr(dec.astype(np.float64), indptr.astype(np.int64), indices.astype(np.int64))
    assert_mean_aggregate(got, want, exact, np.abs(dec).max())


@pytest.mark.parametrize("w,n_cb,feat_dim", [(8, 32, 200), (16, 16, 248), (32, 8, 160)])
def test_fused_vq_sparse_rows_partial_tiles(w, n_cb, feat_dim):
    # few edges per row: results are turned around in LDS before they are stored; the last column
    # tile is partial, rows do not fill the last mini-block, some rows are empty
    rng = np.random.default_rng(w + feat_dim)
    N, rows = 4000, 2051
    cb = rng.standard_normal((n_cb, 256, w)).astype(np.float32)
    codes = rng.integers(0, 256, size=(N, n_cb), dtype=np.uint8)
    indptr, indices = random_graph(rng, rows, N, 5)
    got = host(capi.vq_decompress_spmm_csr(dev(codes), dev(cb), dev(indptr), dev(indices), feat_dim))
    want = oc.vq_decompress_spmm_csr(codes, cb, indptr, indices, feat_dim)
    assert got.shape == (rows, feat_dim)
    dec = oc.vq_decompress(codes, cb, feat_dim)
    exact = oc.spmm_csr(dec.astype(np.float64), indptr, indices)
    assert_mean_aggregate(got, want, exact, np.abs(dec).max(), np.diff(indptr))


def test_fused_vq_int16_codes_big_codebook():
    rng = np.random.default_rng(5)
    cb = rng.standard_normal((2, 5000, 8)).astype(np.float32)   # 160 KB per slice: global path
    codes = rng.integers(0, 5000, size=(800, 2)).astype(np.int16)
    indptr, indices = random_graph(rng, 300, 800, 6)
    got = host(capi.vq_decompress_spmm_csr(dev(codes), dev(cb), dev(indptr), dev(indices), 16))
    assert close(got, oc.vq_decompress_spmm_csr(codes, cb, indptr, indices, 16))


# ---- fused SQ (log domain) --------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [1, 2, 4, 8, 16])
def test_fused_sq_reference_literal_case(bits):
    # tests/test_fusion_decompress_spmm.py:93-120
    rng = np.random.default_rng(bits)
    indptr = dev(np.array([0, 1, 3, 6], dtype=np.int64))
    indices = dev(np.array([0, 1, 1, 2, 2, 0], dtype=np.int64))
    x = rng.standard_normal((6, 100)).astype(np.float32)
    cb = np.stack([oc.sq_codebook(x)])
    codes = capi.sq_compress(dev(x), dev(cb), bits, 100)
    if bits < 8:
        exp = capi.packbits(codes.to(torch.uint8), bits)
    elif bits == 8:
        exp = codes.to(torch.int8)
    else:
        exp = codes.to(torch.int16)
    out1 = capi.spmm_csr(capi.sq_decompress(exp, dev(cb), bits, 100, 100), indptr, indices)
    out2 = capi.sq_decompress_spmm_csr(exp, dev(cb), indptr, indices, bits, 100, 100)
    assert torch.equal(out1, out2)
    want = oc.sq_decompress_spmm_csr(host(exp), cb, host(indptr), host(indices), bits, 100, 100)
    assert np.array_equal(host(out2), want)


@pytest.mark.parametrize("bits", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("d,cs", [(128, 128), (100, 100), (128, 32), (110, 56), (24, 8)])
def test_fused_sq_vs_oracle(bits, d, cs):
    rng = np.random.default_rng(bits * 100 + d)
    N, R = 3000, 900
    x = rng.uniform(-1, 1, size=(N, d)).astype(np.float32) * (1 + np.arange(d) // cs)
    n_cb = (d + cs - 1) // cs
    cbs = np.stack([oc.sq_codebook(x[:, i * cs:(i + 1) * cs]) for i in range(n_cb)])
    store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, cs), bits)
    indptr, indices = random_graph(rng, R, N, 14, np.int64)
    got = host(capi.sq_decompress_spmm_csr(dev(store), dev(cbs), dev(indptr), dev(indices), bits, cs, d))
    want = oc.sq_decompress_spmm_csr(store, cbs, indptr, indices, bits, cs, d)
    assert np.array_equal(got, want)


# ---- fused affine SQ and hybrid ------------------------------------------------------------------------
@pytest.mark.parametrize("bits,d", [(8, 128), (4, 100), (4, 128), (2, 64), (1, 40), (4, 7), (8, 30)])
@pytest.mark.parametrize("idx", [np.int32, np.int64])
def test_fused_affine_vs_oracle(bits, d, idx):
    rng = np.random.default_rng(bits * 10 + d)
    N, R = 4000, 1200
    x = (rng.standard_normal((N, d)) * rng.uniform(0.5, 2, size=d)).astype(np.float32)
    params = oc.sq_affine_params(x, bits)
    codes = oc.sq_affine_compress(x, params, bits)
    store = oc.packbits(codes, bits) if bits < 8 else codes
    indptr, indices = random_graph(rng, R, N, 12, idx)
    got = host(capi.sq_affine_decompress_spmm_csr(dev(store), dev(params), dev(indptr), dev(indices), bits, d))
    want = oc.sq_affine_decompress_spmm_csr(store, params, indptr, indices, bits, d)
    if bits in (4, 8):
        # integer code sums, one float conversion per output: within fp32 rounding of the
        # sequential float sum, and exact for rows with a single neighbour
        assert close(got, want)
        deg = np.diff(indptr.astype(np.int64))
        assert np.array_equal(got[deg <= 1], want[deg <= 1])
        # tighter: against the exact mean in float64
        dec = oc.sq_affine_decompress(store, params, bits, d).astype(np.float64)
        exact = oc.spmm_csr(dec, indptr, indices)
        assert np.abs(got - exact).max() <= np.abs(want - exact).max() + 4 * np.spacing(np.float32(np.abs(dec).max()))
    else:
        assert np.array_equal(got, want)


@pytest.mark.parametrize("bits", [4, 8])
def test_store_mode_changes_no_result(bits):
    """Plain, non-temporal and size-chosen output stores of the row-block SQ kernels write the same bits."""
    rng = np.random.default_rng(bits)
    N, R, d = 5000, 3000, 100
    x = rng.standard_normal((N, d)).astype(np.float32)
    params = oc.sq_affine_params(x, bits)
    store = oc.sq_affine_compress(x, params, bits)
    store = oc.packbits(store, bits) if bits < 8 else store
    cbs = np.stack([oc.sq_codebook(x)])
    log_store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, d), bits)
    indptr, indices = random_graph(rng, R, N, 12, np.int64)
    s, p, ls, cb, ip, ix = dev(store), dev(params), dev(log_store), dev(cbs), dev(indptr), dev(indices)
    was = capi.set_store_mode(capi.STORE_AUTO)
    try:
        results = []
        for mode in (capi.STORE_AUTO, capi.STORE_STREAM, capi.STORE_CACHED):
            capi.set_store_mode(mode)
            results.append((host(capi.sq_affine_decompress_spmm_csr(s, p, ip, ix, bits, d)),
                            host(capi.sq_decompress_spmm_csr(ls, cb, ip, ix, bits, d, d))))
    finally:
        capi.set_store_mode(was)
    for affine, log_domain in results[1:]:
        assert np.array_equal(affine, results[0][0]) and np.array_equal(log_domain, results[0][1])
    assert np.array_equal(results[0][1], oc.sq_decompress_spmm_csr(log_store, cbs, indptr, indices, bits, d, d))


@pytest.mark.parametrize("bits,d,max_deg", [(4, 100, 150), (8, 128, 120), (8, 64, 700), (4, 40, 5000)])
def test_fused_affine_high_degree_rows(bits, d, max_deg):
    # many edge batches per row block, and rows beyond the 16-bit accumulator field capacity
    rng = np.random.default_rng(bits + max_deg)
    N, R = 3000, 40
    x = (rng.standard_normal((N, d)) * 2).astype(np.float32)
    params = oc.sq_affine_params(x, bits)
    codes = oc.sq_affine_compress(x, params, bits)
    store = oc.packbits(codes, bits) if bits < 8 else codes
    deg = rng.integers(0, max_deg + 1, size=R)
    deg[3] = max_deg
    deg[7] = 0
    indptr = np.zeros(R + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, N, size=int(indptr[-1])).astype(np.int64)
    indices[-1] = N - 1  # the last row of the table (its tail dword is partial when src_dim % 4 != 0)
    got = host(capi.sq_affine_decompress_spmm_csr(dev(store), dev(params), dev(indptr), dev(indices), bits, d))
    dec = oc.sq_affine_decompress(store, params, bits, d).astype(np.float64)
    exact = oc.spmm_csr(dec, indptr, indices)
    assert np.allclose(got, exact, rtol=1e-5, atol=1e-5 * np.abs(dec).max())


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("bits,d", [(4, 100), (4, 128), (8, 128), (8, 36)])
@pytest.mark.parametrize("mean_deg", [7, 12, 24])
def test_fused_affine_six_and_more_edges_per_row(bits, d, mean_deg, idx):
    """From six edges per row on the lane groups of the affine kernel take contiguous shares of a block's edges, from
    nine on the accumulators of 4-bit codes are sized for 16-bit fields (rows above 17 edges), and 11-20 edges per row
    run sixteen rows per block.  Ragged rows around those limits, empty rows, a last block of five rows."""
    rng = np.random.default_rng(1000 * bits + 10 * d + mean_deg + (idx == np.int32))
    N, R = 5000, 16 * 40 + 5
    x = (rng.standard_normal((N, d)) * 2).astype(np.float32)
    params = oc.sq_affine_params(x, bits)
    codes = oc.sq_affine_compress(x, params, bits)
    store = oc.packbits(codes, bits) if bits < 8 else codes
    deg = rng.integers(0, 2 * mean_deg + 1, size=R)
    deg[:8] = [0, 17, 18, 1, 0, 0, 40, 16]
    deg[R - 1] = 19
    indptr = np.zeros(R + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    E = int(indptr[-1])
    assert E >= 6 * R
    indices = rng.integers(0, N, size=E).astype(idx)
    got = host(capi.sq_affine_decompress_spmm_csr(dev(store), dev(params), dev(indptr), dev(indices), bits, d))
    dec = oc.sq_affine_decompress(store, params, bits, d)
    exact = oc.spmm_csr(dec.astype(np.float64), indptr.astype(np.int64), indices.astype(np.int64))
    assert np.allclose(got, exact, rtol=1e-5, atol=1e-5 * np.abs(dec).max())
    assert not got[deg == 0].any()
    one = np.nonzero(deg == 1)[0]
    assert np.array_equal(got[one], dec[indices[indptr[one]]])


@pytest.mark.parametrize("shape", [(8, 256, 16), (16, 256, 8), (4, 64, 5), (3, 64, 100)])
def test_hybrid_vs_oracle(shape):
    n_cb, K, w = shape
    D = n_cb * w
    rng = np.random.default_rng(n_cb)
    N, n_hot, R = 6000, 300, 1500
    row_map = np.empty(N, dtype=np.int32)
    perm = rng.permutation(N)
    row_map[perm[:n_hot]] = np.arange(n_hot)
    row_map[perm[n_hot:]] = -np.arange(N - n_hot) - 1
    sq = rng.integers(0, 256, size=(n_hot, D), dtype=np.uint8)
    params = np.stack([rng.standard_normal(D), rng.uniform(0.01, 0.05, D)]).astype(np.float32)
    vq = rng.integers(0, K, size=(N - n_hot, n_cb), dtype=np.uint8)
    cb = rng.standard_normal((n_cb, K, w)).astype(np.float32)
    indptr, indices = random_graph(rng, R, N, 12)
    hot_ids = perm[:n_hot]
    # make ~60 % of the edges hit the hot table
    mask = rng.random(indices.shape[0]) < 0.6
    indices[mask] = rng.choice(hot_ids, size=int(mask.sum()))
    got = host(capi.hybrid_decompress_spmm_csr(dev(row_map), dev(sq), dev(params), dev(vq), dev(cb), dev(indptr),
                                               dev(indices), D))
    want = oc.hybrid_decompress_spmm_csr(row_map, sq, params, vq, cb, indptr, indices, D)
    if w % 4 == 0:   # row-block kernel: integer sums for the SQ rows, then the VQ rows in edge order
        assert close(got, want)
    else:            # per-row skeleton: sequential fp32 sum, bit-exact
        assert np.array_equal(got, want)


def test_hybrid_high_degree_and_vq_heavy():
    rng = np.random.default_rng(21)
    n_cb, K, w = 8, 256, 16
    D = n_cb * w
    N, n_hot, R = 5000, 2500, 60
    row_map = np.empty(N, dtype=np.int32)
    perm = rng.permutation(N)
    row_map[perm[:n_hot]] = np.arange(n_hot)
    row_map[perm[n_hot:]] = -np.arange(N - n_hot) - 1
    sq = rng.integers(0, 256, size=(n_hot, D), dtype=np.uint8)
    params = np.stack([rng.standard_normal(D), rng.uniform(0.01, 0.05, D)]).astype(np.float32)
    vq = rng.integers(0, K, size=(N - n_hot, n_cb), dtype=np.uint8)
    cb = rng.standard_normal((n_cb, K, w)).astype(np.float32)
    deg = rng.integers(0, 60, size=R)
    deg[5] = 700   # beyond the 16-bit field capacity of the SQ accumulators
    deg[9] = 0
    indptr = np.zeros(R + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, N, size=int(indptr[-1])).astype(np.int64)
    got = host(capi.hybrid_decompress_spmm_csr(dev(row_map), dev(sq), dev(params), dev(vq), dev(cb), dev(indptr),
                                               dev(indices), D))
    dec = oc.hybrid_decompress(row_map, sq, params, vq, cb, D, np.arange(N)).astype(np.float64)
    exact = oc.spmm_csr(dec, indptr, indices)
    assert np.allclose(got, exact, rtol=1e-5, atol=1e-5 * np.abs(dec).max())


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("vq_share", [0.05, 0.6])
def test_hybrid_eight_row_blocks(idx, vq_share):
    """Up to 32 edges per row on average and at most 128 columns: single-wave workgroups, of eight rows here, which find an
    edge's row by compares with the block's inner row starts.  Ragged rows, runs of empty rows (equal starts), rows with
    more than 64 edges (outside the per-row mask) and one beyond the 16-bit field capacity, a last block of three rows."""
    rng = np.random.default_rng(int(vq_share * 100) + (idx == np.int32))
    n_cb, K, w = 8, 256, 16
    D = n_cb * w
    N, n_hot, R = 20000, 4000, 8 * 150 + 3
    row_map = np.empty(N, dtype=np.int32)
    perm = rng.permutation(N)
    row_map[perm[:n_hot]] = np.arange(n_hot)
    row_map[perm[n_hot:]] = -np.arange(N - n_hot) - 1
    sq = rng.integers(0, 256, size=(n_hot, D), dtype=np.uint8)
    params = np.stack([rng.standard_normal(D), rng.uniform(0.01, 0.05, D)]).astype(np.float32)
    vq = rng.integers(0, K, size=(N - n_hot, n_cb), dtype=np.uint8)
    cb = rng.standard_normal((n_cb, K, w)).astype(np.float32)
    deg = rng.integers(0, 33, size=R)
    deg[rng.random(R) < 0.2] = 0          # runs of empty rows inside blocks
    deg[16:24] = 0                        # a block without edges
    deg[40] = 90                          # more edges than the per-row mask holds
    deg[41] = 1
    deg[100] = 300                        # beyond the field capacity: summed in the epilogue
    deg[R - 1] = 17
    indptr = np.zeros(R + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    E = int(indptr[-1])
    assert 8.0 <= E / R <= 32.0
    indices = rng.integers(0, N, size=E)
    hot = rng.random(E) >= vq_share
    indices[hot] = rng.choice(perm[:n_hot], size=int(hot.sum()))
    indices = indices.astype(idx)
    rc, plan = capi.dry_run("f2cgt_hybrid_decompress_spmm_csr", 0x1000, 0x1000, 0x1000, D, 0x1000, 0x1000, 0x1000, 0x1000,
                            capi.DT_I64 if idx == np.int64 else capi.DT_I32, 0x1000, R, E, N, n_hot, N - n_hot, D, n_cb, K, w,
                            None)
    assert rc == 0 and plan.block == 64 and plan.rows_per_block == 8
    got = host(capi.hybrid_decompress_spmm_csr(dev(row_map), dev(sq), dev(params), dev(vq), dev(cb), dev(indptr),
                                               dev(indices), D))
    dec = oc.hybrid_decompress(row_map, sq, params, vq, cb, D, np.arange(N)).astype(np.float64)
    exact = oc.spmm_csr(dec, indptr.astype(np.int64), indices.astype(np.int64))
    assert np.allclose(got, exact, rtol=1e-5, atol=1e-5 * np.abs(dec).max())
    assert not got[deg == 0].any()
    one = np.nonzero(deg == 1)[0]
    assert np.array_equal(got[one], dec[indices[indptr[one]]].astype(np.float32))


# ---- encode -------------------------------------------------------------------------------------
@pytest.mark.parametrize("metric", ["l2", "cosine"])
@pytest.mark.parametrize("m,n,k", [(1000, 256, 32), (333, 17, 5), (64, 64, 64), (129, 300, 100)])
def test_pairwise_distance(metric, m, n, k):
    rng = np.random.default_rng(m + n + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    y = rng.standard_normal((n, k)).astype(np.float32)
    got = host(capi.pairwise_distance(dev(x), dev(y), metric))
    want = oc.pairwise_distance(x, y, metric, dtype=np.float64)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("metric", ["l2", "cosine"])
@pytest.mark.parametrize("m,n,k", [(5000, 256, 32), (4097, 255, 9), (700, 37, 16), (1000, 1000, 17), (321, 600, 33),
                                   (2000, 256, 48), (999, 230, 64), (500, 100, 65), (70, 3, 24), (1, 1, 32)])
def test_pairwise_distance_matrix_core_shapes(metric, m, n, k):
    """9 to 64 dimensions go through the matrix cores (y in chunks that fit LDS, vector or scalar
    stores by the row pitch); the neighbours of that range take the vector-ALU kernel."""
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    y = rng.standard_normal((n, k)).astype(np.float32)
    got = host(capi.pairwise_distance(dev(x), dev(y), metric))
    want = oc.pairwise_distance(x, y, metric, dtype=np.float64)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("k", [16, 32, 40, 64])
def test_pairwise_l2_between_almost_equal_points(k):
    """|x|^2 + |y|^2 - 2 x.y cancels when x is close to y; those entries must still be the sum of
    squared differences, to its own relative accuracy (and exactly zero for x == y)."""
    rng = np.random.default_rng(k)
    y = (rng.standard_normal((300, k)) * 10).astype(np.float32)
    x = y[rng.integers(0, 300, size=2000)].copy()
    x[:500] += (rng.standard_normal((500, k)) * 1e-3).astype(np.float32)     # close
    x[500:1000] += (rng.standard_normal((500, k)) * 1e-6).astype(np.float32)  # mostly identical after rounding
    x[1500:] = (rng.standard_normal((500, k)) * 10).astype(np.float32)       # far
    got = host(capi.pairwise_distance(dev(x), dev(y), "l2"))
    want = oc.pairwise_distance(x, y, "l2", dtype=np.float64)
    assert np.allclose(got, want, rtol=1e-5, atol=0.0)
    same = (x[:, None, :] == y[None, :, :]).all(axis=2)
    assert same.any() and not got[same].any()


def test_pairwise_cosine_with_vectors_without_a_direction():
    rng = np.random.default_rng(8)
    k = 32
    x = rng.standard_normal((400, k)).astype(np.float32)
    y = rng.standard_normal((96, k)).astype(np.float32)
    x[3] = 0
    x[77] *= 1e-7            # |x||y| falls below the clamp of the denominator
    x[200] *= 1e-4
    y[5] = 0
    y[40] *= 1e-6
    got = host(capi.pairwise_distance(dev(x), dev(y), "cosine"))
    want = oc.pairwise_distance(x, y, "cosine", dtype=np.float64)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # without degenerate centres only the rows near the clamp take the exact path
    y2 = rng.standard_normal((96, k)).astype(np.float32)
    got = host(capi.pairwise_distance(dev(x), dev(y2), "cosine"))
    assert np.allclose(got, oc.pairwise_distance(x, y2, "cosine", dtype=np.float64), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("metric", ["l2", "cosine"])
@pytest.mark.parametrize("m,n,k", [(20000, 256, 32), (5000, 256, 8), (3001, 100, 16), (777, 37, 5),
                                   (4000, 256, 64), (500, 1000, 24), (300, 50, 200),
                                   # beyond the matrix-core kernels (more than 64 dimensions, many centres): tiles on the
                                   # vector ALUs with a running arg-min; 63 rows and fewer: one wave per row
                                   (5000, 256, 65), (3000, 300, 128), (700, 4096, 8), (129, 17, 200), (64, 3, 70),
                                   (63, 5, 100), (4000, 256, 96), (1000, 512, 64)])
def test_kmeans_predict_vs_oracle(metric, m, n, k):
    rng = np.random.default_rng(m + n + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    c = rng.standard_normal((n, k)).astype(np.float32)
    want, near = oc.kmeans_predict(x, c, metric)
    got = host(capi.kmeans_predict(dev(x), dev(c), metric))
    assert np.array_equal(got[~near], want[~near])
    assert near.mean() < 0.01
    if n <= 256:
        got8 = host(capi.kmeans_predict(dev(x), dev(c), metric, u8=True))
        assert np.array_equal(got8.astype(np.int64), got)


@pytest.mark.parametrize("metric", ["l2", "cosine"])
@pytest.mark.parametrize("m,n,k", [(2000, 8, 8), (3000, 256, 32), (500, 1000, 24), (300, 50, 200), (3000, 256, 96)])
def test_kmeans_predict_rows_that_are_not_numbers(metric, m, n, k):
    """Rows with NaN or infinite entries have no nearest centre.  Their labels must still be valid
    indices (centre 0: the callers' trainer turns NaN distances into 1 before its arg-min,
    examples/my_kmeans.py:92-94, which sends such a row to the first centre) and the other rows must
    not notice: an arg-min stage that found no comparable distance used to keep its "none yet" index."""
    rng = np.random.default_rng(m + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    c = rng.standard_normal((n, k)).astype(np.float32)
    clean, near = oc.kmeans_predict(x, c, metric)
    bad = rng.choice(m, size=25, replace=False)
    x[bad[:10], rng.integers(0, k, size=10)] = np.nan
    x[bad[10:18]] = np.nan
    x[bad[18:], rng.integers(0, k, size=7)] = np.inf
    got = host(capi.kmeans_predict(dev(x), dev(c), metric))
    assert got.min() >= 0 and got.max() < n
    assert np.all(got[bad[:18]] == 0)
    keep = np.ones(m, dtype=bool)
    keep[bad] = False
    assert np.array_equal(got[keep & ~near], clean[keep & ~near])
    if n <= 256:
        got8 = host(capi.kmeans_predict(dev(x), dev(c), metric, u8=True))
        assert np.array_equal(got8.astype(np.int64), got)


@pytest.mark.parametrize("k", [32, 96])
def test_kmeans_predict_exact_ties_pick_first(k):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((4000, k)).astype(np.float32)
    c = rng.standard_normal((256, k)).astype(np.float32)
    c[200] = c[7]
    c[255] = c[100]
    got = host(capi.kmeans_predict(dev(x), dev(c), "l2"))
    want, _ = oc.kmeans_predict(x, c, "l2")
    assert np.array_equal(got, want)  # fp64 refinement resolves the duplicates to the first index
    assert not np.isin(got, [200, 255]).any()
    # data points that ARE centres
    got_c = host(capi.kmeans_predict(dev(c), dev(c), "l2"))
    assert np.array_equal(got_c, oc.kmeans_predict(c, c, "l2")[0])


@pytest.mark.parametrize("metric", ["l2", "cosine"])
def test_kmeans_predict_when_the_expanded_form_cancels(metric):
    # a common offset makes |x|^2 and |c|^2 about 1e4 times the distances between them, so most rows
    # fall inside the rounding bound of the matrix-core scores and take the exact re-evaluation
    rng = np.random.default_rng(21)
    x = (rng.standard_normal((6000, 32)) * 0.3 + 17.0).astype(np.float32)
    c = (rng.standard_normal((256, 32)) * 0.3 + 17.0).astype(np.float32)
    want, near = oc.kmeans_predict(x, c, metric)
    got = host(capi.kmeans_predict(dev(x), dev(c), metric))
    assert np.array_equal(got[~near], want[~near])
    assert near.mean() < 0.05


@pytest.mark.parametrize("scale", [1e-19, 3e-17, 1e15])
def test_kmeans_predict_extreme_magnitudes(scale):
    # tiny values: the second-order piece products (and at 1e-19 the products themselves) fall below
    # the smallest normal fp32 number inside the matrix core; huge ones: squares near 1e32
    rng = np.random.default_rng(23)
    x = (rng.standard_normal((3000, 32)) * scale).astype(np.float32)
    c = (rng.standard_normal((256, 32)) * scale).astype(np.float32)
    want, near = oc.kmeans_predict(x, c, "l2")
    got = host(capi.kmeans_predict(dev(x), dev(c), "l2"))
    assert np.array_equal(got[~near], want[~near])


@pytest.mark.parametrize("k,n", [(1, 256), (1, 700), (2, 300), (3, 256)])
def test_kmeans_predict_few_dimensions_many_close_centres(k, n):
    # points and centres packed on a short segment away from the origin: distances of 1e-5 next to
    # norms of 4, so every row takes the exact path and its candidate filter (leading bf16 pieces of
    # the centres, off by up to 2^-8 of their size) has to keep the true minimum among many
    rng = np.random.default_rng(24 + k + n)
    x = (rng.standard_normal((4000, k)) + 2.0).astype(np.float32)
    c = (rng.standard_normal((n, k)) + 2.0).astype(np.float32)
    want, near = oc.kmeans_predict(x, c, "l2")
    got = host(capi.kmeans_predict(dev(x), dev(c), "l2"))
    assert np.array_equal(got[~near], want[~near])
    wantc, nearc = oc.kmeans_predict(x, c, "cosine")
    gotc = host(capi.kmeans_predict(dev(x), dev(c), "cosine"))
    assert np.array_equal(gotc[~nearc], wantc[~nearc])


@pytest.mark.parametrize("offset", [0.0, 1000.0])
def test_kmeans_predict_l2_exact_ties_far_from_the_origin(offset):
    """The L2 kernel works on x - mu and c - mu; ties and near-ties of the original rows must still
    be decided as the original rows say: an exact tie goes to the first centre, a centre that is
    closer by a few units in the last place wins."""
    rng = np.random.default_rng(17)
    k, m = 32, 32
    p = (offset + rng.integers(-10, 11, size=(m, k))).astype(np.float32)
    e = (rng.integers(0, 2, size=(m, k)) * 0.5 - 0.25).astype(np.float32)      # +-0.25, exact at this magnitude
    c = np.empty((2 * m, k), dtype=np.float32)
    c[0::2], c[1::2] = p + e, p - e
    assert np.array_equal((c[0::2] - p), e) and np.array_equal((p - c[1::2]), e)
    got = host(capi.kmeans_predict(dev(p), dev(c), "l2"))
    assert np.array_equal(got, 2 * np.arange(m))                             # exact ties: the first
    c2 = c.copy()
    c2[1::2, 0] += np.sign(e[:, 0]) * np.float32(2.0 ** -13)                 # the second moves a hair closer
    d = oc.pairwise_distance(p, c2, "l2", dtype=np.float64)
    assert np.all(d[np.arange(m), 2 * np.arange(m) + 1] < d[np.arange(m), 2 * np.arange(m)])
    got = host(capi.kmeans_predict(dev(p), dev(c2), "l2"))
    assert np.array_equal(got, 2 * np.arange(m) + 1)
    # three equidistant centres: the row is decided over every centre
    c3 = np.concatenate([c, c[0:1]])
    got = host(capi.kmeans_predict(dev(p), dev(c3), "l2"))
    assert got[0] == 0 and np.array_equal(got[1:], 2 * np.arange(1, m))


def test_kmeans_predict_l2_does_not_slow_down_far_from_the_origin():
    """With the mean of the centres subtracted, a common offset no longer sends rows to the exact
    re-evaluation; labels stay those of the fp64 distances."""
    rng = np.random.default_rng(23)
    x = (rng.standard_normal((20000, 32)) + 300.0).astype(np.float32)
    c = (rng.standard_normal((256, 32)) + 300.0).astype(np.float32)
    want, near = oc.kmeans_predict(x, c, "l2")
    got = host(capi.kmeans_predict(dev(x), dev(c), "l2"))
    assert np.array_equal(got[~near], want[~near])


@pytest.mark.parametrize("offset", [3.0, 100.0])
def test_kmeans_predict_cosine_far_from_the_origin(offset):
    """Centres that share most of their direction: the kernel takes their mean direction out of
    the scores; labels stay those of the fp64 cosines, duplicates go to the first copy."""
    rng = np.random.default_rng(29)
    x = (rng.standard_normal((20000, 32)) + offset).astype(np.float32)
    c = (rng.standard_normal((256, 32)) + offset).astype(np.float32)
    c[200] = c[5]
    want, near = oc.kmeans_predict(x, c, "cosine")
    got = host(capi.kmeans_predict(dev(x), dev(c), "cosine"))
    assert np.array_equal(got[~near], want[~near])
    assert not np.any(got == 200) and np.any(got == 5)


def test_kmeans_predict_cosine_with_a_centre_without_direction():
    rng = np.random.default_rng(22)
    x = rng.standard_normal((3000, 32)).astype(np.float32)
    c = rng.standard_normal((256, 32)).astype(np.float32)
    c[17] = 0.0
    want, near = oc.kmeans_predict(x, c, "cosine")
    got = host(capi.kmeans_predict(dev(x), dev(c), "cosine"))
    assert np.array_equal(got[~near], want[~near])


# ---- the F2CGTLib module (same kernels through the pybind shim) ------------------------------------
def test_module_surface_end_to_end():
    import f2cgt_amd

    lib = f2cgt_amd.load()
    rng = np.random.default_rng(12)
    x = rng.uniform(-1, 1, size=(500, 100)).astype(np.float32)
    cb = np.stack([oc.sq_codebook(x)])
    indptr, indices = random_graph(rng, 200, 500, 10)
    ip, ix = dev(indptr), dev(indices)
    for bits in (1, 2, 4, 8, 16):
        codes = lib.sq_compress(dev(x), dev(cb), bits, 100)
        if bits < 8:
            exp = lib.packbits(codes.to(torch.uint8), bits)
            assert torch.equal(lib.unpackbits(exp, bits, 100), codes.to(torch.uint8))
            exp = exp.to(torch.int8)  # packed tables are stored as int8 (examples/process_compress.py:109-141)
        elif bits == 8:
            exp = codes.to(torch.int8)
        else:
            exp = codes.to(torch.int16)
        out1 = lib.spmm_csr(lib.sq_decompress(exp, dev(cb), bits, 100, 100), ip, ix)
        out2 = lib.sq_decompress_spmm_csr(exp, dev(cb), ip, ix, bits, 100, 100)
        assert torch.equal(out1, out2)
    # int16 index tensors are accepted like the reference's dispatch
    out3 = lib.spmm_csr(dev(x), ip.to(torch.int16), ix.to(torch.int16))
    assert torch.equal(out3, lib.spmm_csr(dev(x), ip, ix))
    # VQ through KMeans: fit, predict, decode, fused aggregate
    data = dev(rng.standard_normal((3000, 16)).astype(np.float32))
    km = lib.KMeans(64, 16, "l2")
    km.fit(data)
    centers = km.get_centers()
    assert centers.shape == (64, 16) and centers.data_ptr() == km.get_centers().data_ptr()
    labels = km.predict(data)
    assert labels.dtype == torch.int64 and labels.shape == (3000,)
    want, near = oc.kmeans_predict(host(data), host(centers), "l2")
    assert np.array_equal(host(labels)[~near], want[~near])
    km2 = lib.KMeans(centers, "cosine")
    lc = km2.predict(data, normalize_weights=False)
    wc, nearc = oc.kmeans_predict(host(data), host(centers), "cosine")
    assert np.array_equal(host(lc)[~nearc], wc[~nearc])
    dist = lib.pairwise_distance(data[:100], centers, "euclidean")
    assert torch.equal(dist.argmin(dim=1), labels[:100]) or near[:100].any()
    codes8 = labels.to(torch.uint8).reshape(-1, 1)
    cbk = centers.reshape(1, 64, 16)
    ipv, ixv = random_graph(rng, 400, 3000, 15)
    o1 = lib.spmm_csr(lib.vq_decompress(codes8, cbk, 16), dev(ipv), dev(ixv))
    o2 = lib.vq_decompress_spmm_csr(codes8, cbk, dev(ipv), dev(ixv), 16)
    # 400 rows take the pipelined kernel, whose mean is the sum times a refined reciprocal: within 2 ulp of the
    # division that spmm_csr performs (the reference's own 3-row case stays on the bit-exact per-row form)
    dec64 = host(lib.vq_decompress(codes8, cbk, 16)).astype(np.float64)
    assert_mean_aggregate(host(o2), host(o1), oc.spmm_csr(dec64, ipv, ixv), float(np.abs(dec64).max()))
    with pytest.raises(RuntimeError, match="column_slice"):
        lib.sq_decompress_spmm_csr(exp, dev(cb), ip, ix, 4, 0, 100)
    with pytest.raises(RuntimeError):
        lib.packbits(dev(np.zeros((2, 4), np.uint8)), 3)


def test_ops_run_on_the_current_stream():
    rng = np.random.default_rng(13)
    cb = dev(rng.standard_normal((16, 256, 8)).astype(np.float32))
    codes = dev(rng.integers(0, 256, size=(20000, 16), dtype=np.uint8))
    indptr, indices = random_graph(rng, 5000, 20000, 15)
    ip, ix = dev(indptr), dev(indices)
    ref = capi.vq_decompress_spmm_csr(codes, cb, ip, ix, 128)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        out = capi.vq_decompress_spmm_csr(codes, cb, ip, ix, 128)
    side.synchronize()
    assert torch.equal(out, ref)
