"""Seeded random shapes through every fused operator and the streaming ones: the fast kernels are
chosen by shape (column count, bits, degree, index type, alignment), so many small, odd shapes are
what finds a path that a hand-picked list misses.  Same bars as the parity tests.

F2CGT_FUZZ_SEED0 (first seed, default 0) and F2CGT_FUZZ_MULT (multiplier of the number of seeds per
test, default 1) widen the sweep for a one-off run; the defaults are what the suite runs."""
import os

import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from f2cgt_amd import capi

pytestmark = pytest.mark.gpu
RTOL = 1e-5
SEED0 = int(os.environ.get("F2CGT_FUZZ_SEED0", "0"))
MULT = int(os.environ.get("F2CGT_FUZZ_MULT", "1"))


def seeds(n):
    return range(SEED0, SEED0 + n * MULT)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def graph(rng, rows, n_src, idx):
    kind = rng.integers(0, 6)
    if kind == 4:
        deg = np.zeros(rows, dtype=np.int64)                         # no edges at all
    elif kind == 5:
        deg = rng.integers(0, 3, size=rows)                          # a few very long rows among short ones
        deg[rng.integers(0, rows, size=min(3, rows))] = int(rng.integers(300, 2500))
    elif kind == 0:
        deg = rng.integers(0, 4, size=rows)                          # sparse, with empty rows
    elif kind == 1:
        deg = np.full(rows, int(rng.integers(1, 40)))                # fixed fanout
    elif kind == 2:
        deg = np.minimum(rng.zipf(1.8, size=rows), 300)              # heavy tail
    else:
        deg = rng.integers(0, int(rng.integers(2, 90)), size=rows)
    indptr = np.zeros(rows + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1])).astype(idx)
    return indptr, indices


def close(got, want):
    scale = float(np.abs(want).max()) if want.size else 1.0
    return np.allclose(got, want, rtol=RTOL, atol=RTOL * scale)


def agg_ok(got, want32, decoded, indptr, indices):
    """Aggregation bar: within 1e-5 of the reference's sequential fp32 sum, or, where that sum
    itself has drifted further from the exact mean (rows of thousands of edges), at least as close
    to the fp64 mean of the same decoded fp32 values as the sequential fp32 sum is."""
    if close(got, want32):
        return True
    exact = oc.spmm_csr(decoded.astype(np.float64), indptr.astype(np.int64), indices.astype(np.int64))
    scale = float(np.abs(exact).max()) if exact.size else 1.0
    bound = np.maximum(np.abs(want32 - exact), RTOL * np.abs(exact) + 1e-6 * scale)
    return bool(np.all(np.abs(got - exact) <= bound))


@pytest.mark.parametrize("seed", seeds(24))
def test_fused_affine_sq_random_shape(seed):
    rng = np.random.default_rng(1000 + seed)
    bits = int(rng.choice([1, 2, 4, 8]))
    D = int(rng.choice([4, 8, 12, 20, 36, 64, 100, 128, 132, 256, 300]))
    N, rows = int(rng.integers(50, 3000)), int(rng.integers(1, 1500))
    idx = rng.choice([np.int32, np.int64])
    x = rng.standard_normal((N, D)).astype(np.float32) * rng.uniform(0.1, 10)
    params = oc.sq_affine_params(x, bits)
    codes = oc.sq_affine_compress(x, params, bits)
    indptr, indices = graph(rng, rows, N, idx)
    got = host(capi.sq_affine_decompress_spmm_csr(dev(codes), dev(params), dev(indptr), dev(indices), bits, D))
    want = oc.sq_affine_decompress_spmm_csr(codes, params, indptr.astype(np.int64), indices.astype(np.int64), bits, D)
    assert got.shape == want.shape
    assert agg_ok(got, want, oc.sq_affine_decompress(codes, params, bits, D), indptr, indices)


@pytest.mark.parametrize("seed", seeds(24))
def test_fused_log_sq_random_shape(seed):
    rng = np.random.default_rng(2000 + seed)
    bits = int(rng.choice([1, 2, 4, 8, 16]))
    per = max(1, 8 // bits)
    D = int(rng.choice([8, 16, 24, 40, 64, 100, 128, 200]))
    slices = [s for s in (8, 16, 40, 64, D) if s % per == 0 and s <= D]
    cs = int(rng.choice(slices))
    N, rows = int(rng.integers(50, 2500)), int(rng.integers(1, 1200))
    idx = rng.choice([np.int32, np.int64])
    x = rng.uniform(-3, 3, size=(N, D)).astype(np.float32)
    cbs = np.stack([oc.sq_codebook(x[:, s:s + cs]) for s in range(0, D, cs)])
    store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, cs), bits)
    indptr, indices = graph(rng, rows, N, idx)
    got = host(capi.sq_decompress_spmm_csr(dev(store), dev(cbs), dev(indptr), dev(indices), bits, cs, D))
    raw = store.view(np.uint8) if store.dtype == np.int8 and bits < 8 else store
    want = oc.sq_decompress_spmm_csr(raw, cbs, indptr.astype(np.int64), indices.astype(np.int64), bits, cs, D)
    assert agg_ok(got, want, oc.sq_decompress_per_byte_codebook(raw, cbs, bits, cs, D), indptr, indices)
    # and the standalone decode of the same table, bit for bit
    dec = host(capi.sq_decompress(dev(store), dev(cbs), bits, cs, D))
    assert np.array_equal(dec, oc.sq_decompress(raw, cbs, bits, cs, D))


@pytest.mark.parametrize("seed", seeds(24))
def test_fused_vq_random_shape(seed):
    rng = np.random.default_rng(3000 + seed)
    w = int(rng.choice([4, 8, 16, 32]))
    n_cb = int(rng.choice([1, 2, 4, 8, 16, 24]))
    K = int(rng.choice([16, 100, 256]))
    full = n_cb * w
    D = int(rng.choice([full, max(4, full - 4), max(4, full - w // 2)]))
    D = max(4, D - D % 4)
    N, rows = int(rng.integers(50, 3000)), int(rng.integers(1, 1500))
    idx = rng.choice([np.int32, np.int64])
    cb = rng.standard_normal((n_cb, K, w)).astype(np.float32)
    codes = rng.integers(0, K, size=(N, n_cb), dtype=np.uint8)
    indptr, indices = graph(rng, rows, N, idx)
    got = host(capi.vq_decompress_spmm_csr(dev(codes), dev(cb), dev(indptr), dev(indices), D))
    want = oc.vq_decompress_spmm_csr(codes, cb, indptr.astype(np.int64), indices.astype(np.int64), D)
    assert agg_ok(got, want, oc.vq_decompress(codes, cb, D), indptr, indices)
    dec = host(capi.vq_decompress(dev(codes), dev(cb), D))
    assert np.array_equal(dec, oc.vq_decompress(codes, cb, D))


@pytest.mark.parametrize("seed", seeds(16))
def test_hybrid_random_shape(seed):
    rng = np.random.default_rng(4000 + seed)
    w = int(rng.choice([8, 16, 32]))
    D = int(rng.choice([32, 64, 128, 256]))
    n_cb = D // w
    N, rows = int(rng.integers(100, 3000)), int(rng.integers(1, 1200))
    idx = rng.choice([np.int32, np.int64])
    n_sq = int(rng.integers(1, N))
    n_vq = N - n_sq
    x = rng.standard_normal((n_sq, D)).astype(np.float32)
    params = oc.sq_affine_params(x, 8)
    sq = oc.sq_affine_compress(x, params, 8)
    cb = rng.standard_normal((n_cb, 256, w)).astype(np.float32)
    vq = rng.integers(0, 256, size=(max(n_vq, 1), n_cb), dtype=np.uint8)
    perm = rng.permutation(N)
    row_map = np.empty(N, dtype=np.int32)
    row_map[perm[:n_sq]] = np.arange(n_sq, dtype=np.int32)
    row_map[perm[n_sq:]] = -np.arange(n_vq, dtype=np.int32) - 1
    indptr, indices = graph(rng, rows, N, idx)
    got = host(capi.hybrid_decompress_spmm_csr(dev(row_map), dev(sq), dev(params), dev(vq), dev(cb), dev(indptr),
                                               dev(indices), D))
    want = oc.hybrid_decompress_spmm_csr(row_map, sq, params, vq, cb, indptr.astype(np.int64),
                                         indices.astype(np.int64), D)
    assert agg_ok(got, want, oc.hybrid_decompress(row_map, sq, params, vq, cb, D, np.arange(N)), indptr, indices)


@pytest.mark.parametrize("seed", seeds(16))
def test_pack_and_sq_encode_random_shape(seed):
    rng = np.random.default_rng(5000 + seed)
    bits = int(rng.choice([1, 2, 4]))
    rows, U = int(rng.integers(1, 700)), int(rng.integers(1, 300))
    codes = rng.integers(0, 1 << bits, size=(rows, U), dtype=np.uint8)
    packed = host(capi.packbits(dev(codes), bits))
    assert np.array_equal(packed, oc.packbits(codes, bits))
    assert np.array_equal(host(capi.unpackbits(dev(packed), bits, U)), codes)
    ebits = int(rng.choice([1, 2, 4, 8, 16]))
    per = max(1, 8 // ebits)
    D = int(rng.choice([4, 13, 32, 100, 130]))
    cs = int(rng.choice([c for c in (8, 16, 64, 256) if c % per == 0]))
    x = rng.uniform(-2, 2, size=(rows, D)).astype(np.float32)
    cbs = np.stack([oc.sq_codebook(x[:, s:s + cs]) for s in range(0, D, cs)])
    want = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, ebits, cs), ebits)
    got = host(capi.sq_encode(dev(x), dev(cbs), ebits, cs))
    assert np.array_equal(got.view(want.dtype) if got.dtype != want.dtype else got, want)


@pytest.mark.parametrize("seed", seeds(40))
def test_encode_random_shape(seed):
    rng = np.random.default_rng(6000 + seed)
    metric = str(rng.choice(["l2", "cosine"]))
    m = int(rng.integers(1, 5000))
    n = int(rng.choice([1, 2, 7, 33, 64, 100, 256, 300, 700]))
    k = int(rng.choice([1, 3, 8, 16, 24, 32, 40, 64, 72, 130]))
    shift = float(rng.choice([0.0, 0.0, 2.0, 30.0]))          # an offset makes the expanded form cancel
    x = (rng.standard_normal((m, k)) + shift).astype(np.float32)
    c = (rng.standard_normal((n, k)) + shift).astype(np.float32)
    want, near = oc.kmeans_predict(x, c, metric)
    got = host(capi.kmeans_predict(dev(x), dev(c), metric))
    assert got.shape == (m,)
    assert np.array_equal(got[~near], want[~near])
    if n <= 256:
        got8 = host(capi.kmeans_predict(dev(x), dev(c), metric, u8=True))
        assert np.array_equal(got8.astype(np.int64), got)
    d = host(capi.pairwise_distance(dev(x), dev(c), metric))
    ref = oc.pairwise_distance(x, c, metric, dtype=np.float64)
    assert np.allclose(d, ref, rtol=1e-5, atol=1e-5 * max(1.0, float(np.abs(ref).max())))


@pytest.mark.parametrize("seed", seeds(24))
def test_fetch_rows_random_shape(seed):
    rng = np.random.default_rng(7000 + seed)
    dtype = [np.uint8, np.int8, np.int16, np.float32, np.float64, np.float16][int(rng.integers(0, 6))]
    cols = int(rng.integers(1, 200))
    n = int(rng.integers(1, 3000))
    m = int(rng.integers(0, 4000))
    table = (rng.standard_normal((n, cols)) * 50).astype(dtype)
    idx = [np.int32, np.int64][int(rng.integers(0, 2))]
    index = rng.integers(0, n, size=m).astype(idx)
    t_dev = dev(table)
    assert np.array_equal(host(capi.fetch_rows(t_dev, dev(index))).view(np.uint8), table[index].view(np.uint8))
    n_hot = int(rng.integers(0, n + 1))
    if n_hot:
        hot_ids = rng.permutation(n)[:n_hot]
        hot = (rng.standard_normal((n_hot, cols)) * 50).astype(dtype)
        slot = np.full(n, -1, dtype=np.int32)
        slot[hot_ids] = np.arange(n_hot, dtype=np.int32)
        got = host(capi.fetch_rows(t_dev, dev(index), dev(hot), dev(slot)))
        assert np.array_equal(got.view(np.uint8), oc.fetch_rows(table, index, hot, slot).view(np.uint8))


@pytest.mark.parametrize("seed", seeds(12))
def test_module_dtype_surface_random(seed):
    """The F2CGTLib module with the reference's accepted dtypes (src/common.h:17-104): index tensors of
    any integer width, fp16 / fp64 features for spmm_csr, fp16 codebooks and int16 codes for vq_decompress."""
    import f2cgt_amd
    lib = f2cgt_amd.load()
    rng = np.random.default_rng(7000 + seed)
    idt = [torch.int8, torch.uint8, torch.int16, torch.int32, torch.int64][seed % 5]
    cap = {torch.int8: 127, torch.uint8: 255, torch.int16: 32767}.get(idt, 1 << 20)
    n_src = int(min(cap, rng.integers(20, 2000)))
    D = int(rng.choice([4, 16, 60, 128]))
    # rows and edges limited so that every offset fits the index type
    rows = int(rng.integers(1, 40))
    deg = rng.integers(0, 4, size=rows)
    while deg.sum() > cap:
        deg = deg // 2
    indptr = np.zeros(rows + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1]))
    ip, ix = torch.from_numpy(indptr).to(idt).cuda(), torch.from_numpy(indices).to(idt).cuda()
    for ft in (torch.float32, torch.float16, torch.float64):
        feat = torch.from_numpy(rng.standard_normal((n_src, D)).astype(np.float32)).to(ft).cuda()
        out = lib.spmm_csr(feat, ip, ix)
        assert out.dtype == ft and tuple(out.shape) == (rows, D)
        want = oc.spmm_csr(feat.cpu().double().numpy(), indptr, indices)
        tol = 2e-3 if ft == torch.float16 else 1e-5
        assert np.allclose(out.cpu().double().numpy(), want, rtol=tol, atol=tol * max(1.0, float(np.abs(want).max())))
    w, n_cb, K = 8, (D + 7) // 8, int(rng.choice([50, 256, 1000]))
    if D >= 8:
        cb = rng.standard_normal((n_cb, K, w)).astype(np.float32)
        cdt = torch.uint8 if K <= 256 else torch.int16
        codes = torch.from_numpy(rng.integers(0, K, size=(n_src, n_cb))).to(cdt).cuda()
        for cbt in (torch.float32, torch.float16):
            cbd = torch.from_numpy(cb).to(cbt).cuda()
            dec = lib.vq_decompress(codes, cbd, D)
            want = oc.vq_decompress(codes.cpu().numpy().astype(np.int64), cbd.float().cpu().numpy(), D)
            assert np.array_equal(dec.float().cpu().numpy(), want)
        fused = lib.vq_decompress_spmm_csr(codes, torch.from_numpy(cb).cuda(), ip, ix, D)
        wantf = oc.vq_decompress_spmm_csr(codes.cpu().numpy().astype(np.int64), cb, indptr, indices, D)
        assert close(fused.cpu().numpy(), wantf)
