"""Tables, outputs and element counts beyond 2^31 / 2^32: every offset in the kernels is 64-bit
(the reference indexes with `int`, e.g. `src/packbits.cu:24-41`, and wraps there).  The rows that
matter sit at the far end of each array, where a 32-bit product would have wrapped; they are checked
against the same operator on a small copy of those rows (an independent, small-offset run) and
against the CPU oracle."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from f2cgt_amd import capi

pytestmark = pytest.mark.gpu
RTOL = 1e-5
TAIL = 3000


def _gen(seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return g


def _rand_u8(shape, hi, seed):
    return torch.randint(0, hi, shape, dtype=torch.uint8, device="cuda", generator=_gen(seed))


def _sample_rows(n, seed):
    """Row numbers at both ends, around the 2^31 / 2^32 byte marks' neighbourhood (spread), and the tail."""
    rng = np.random.default_rng(seed)
    return torch.from_numpy(np.unique(np.concatenate([rng.integers(0, n, size=TAIL), np.arange(n - TAIL, n),
                                                      np.arange(0, 64)]))).cuda()


def _tail_graph(n_src, rows, max_deg, seed, idx=torch.int64):
    """CSC block whose source ids mostly lie in the last 2 % of the table, a few anywhere."""
    rng = np.random.default_rng(seed)
    deg = rng.integers(0, max_deg + 1, size=rows)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    e = int(indptr[-1])
    far = n_src - 1 - rng.integers(0, max(1, n_src // 50), size=e)
    anywhere = rng.integers(0, n_src, size=e)
    ids = np.where(rng.random(e) < 0.9, far, anywhere)
    ids[-1] = n_src - 1
    return torch.from_numpy(indptr).to(idx).cuda(), torch.from_numpy(ids).to(idx).cuda()


def _local(indices):
    uniq, inv = torch.unique(indices.long(), return_inverse=True)
    return uniq, inv.to(indices.dtype)


def test_pack_and_unpack_beyond_2_32_bytes():
    rows, dim = 43_100_000, 100                               # 4.31e9 bytes unpacked, 2.155e9 packed
    x = _rand_u8((rows, dim), 16, 1)
    assert x.numel() > 2 ** 32 and x.numel() // 2 > 2 ** 31
    p = capi.packbits(x, 4)
    assert p.shape == (rows, 50)
    assert torch.equal(p, x[:, 0::2] | (x[:, 1::2] << 4))
    assert torch.equal(capi.unpackbits(p, 4, dim), x)
    sel = _sample_rows(rows, 2)
    assert torch.equal(p[sel], capi.packbits(x[sel].contiguous(), 4))
    want = oc.packbits(x[rows - 200:].cpu().numpy(), 4)
    assert np.array_equal(p[rows - 200:].cpu().numpy(), want)
    del p
    x &= 1                                                    # ragged 1-bit rows: 100 -> 13 bytes
    p1 = capi.packbits(x, 1)
    assert p1.shape == (rows, 13)
    assert np.array_equal(p1[rows - 200:].cpu().numpy(), oc.packbits(x[rows - 200:].cpu().numpy(), 1))
    assert torch.equal(capi.unpackbits(p1, 1, dim), x)


def test_decoders_with_more_than_2_31_output_elements():
    rows, dim = 21_600_000, 100                               # 2.16e9 floats out
    sel = _sample_rows(rows, 3)
    codes = _rand_u8((rows, 50), 256, 4)
    params = torch.stack([torch.linspace(-2, 1, dim), torch.linspace(0.1, 0.4, dim)]).cuda()
    out = capi.sq_affine_decompress(codes, params, 4, dim)
    assert out.numel() > 2 ** 31
    assert torch.equal(out[sel], capi.sq_affine_decompress(codes[sel].contiguous(), params, 4, dim))
    want = oc.sq_affine_decompress(codes[rows - 100:].cpu().numpy(), params.cpu().numpy(), 4, dim)
    assert np.array_equal(out[rows - 100:].cpu().numpy(), want)
    del out
    logcb = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4], [0.02, 2.0, -5.643856, 1.0, 0.3]], device="cuda")
    out = capi.sq_decompress(codes, logcb, 4, 50, dim)
    assert torch.equal(out[sel], capi.sq_decompress(codes[sel].contiguous(), logcb, 4, 50, dim))
    want = oc.sq_decompress(codes[rows - 100:].cpu().numpy(), logcb.cpu().numpy(), 4, 50, dim)
    assert np.array_equal(out[rows - 100:].cpu().numpy(), want)
    del out, codes
    vrows = 17_000_000                                        # x 128 columns = 2.18e9 floats
    vsel = _sample_rows(vrows, 5)
    vcodes = _rand_u8((vrows, 16), 256, 6)
    cb = torch.randn((16, 256, 8), device="cuda", generator=_gen(7))
    out = capi.vq_decompress(vcodes, cb, 128)
    assert out.numel() > 2 ** 31
    assert torch.equal(out[vsel], capi.vq_decompress(vcodes[vsel].contiguous(), cb, 128))
    want = oc.vq_decompress(vcodes[vrows - 100:].cpu().numpy(), cb.cpu().numpy(), 128)
    assert np.array_equal(out[vrows - 100:].cpu().numpy(), want)


def test_sq_encode_with_more_than_2_31_input_elements():
    rows, dim = 21_600_000, 100
    x = torch.randn((rows, dim), device="cuda", generator=_gen(8))
    cb = torch.from_numpy(oc.sq_codebook(x[:100_000].cpu().numpy())).cuda().reshape(1, 5)
    sel = _sample_rows(rows, 9)
    packed = capi.sq_encode(x, cb, 4, dim)
    assert torch.equal(packed[sel], capi.sq_encode(x[sel].contiguous(), cb, 4, dim))
    tail = x[rows - 100:].cpu().numpy()
    want = oc.sq_codes_to_storage(oc.sq_compress(tail, cb.cpu().numpy(), 4, dim), 4)
    assert np.array_equal(packed[rows - 100:].cpu().numpy().view(np.uint8), want)
    del packed
    codes = capi.sq_compress(x, cb, 4, dim)
    assert codes.numel() > 2 ** 31
    assert torch.equal(codes[sel], capi.sq_compress(x[sel].contiguous(), cb, 4, dim))


@pytest.mark.parametrize("idx", [torch.int64, torch.int32])
def test_fused_and_plain_aggregation_from_tables_beyond_2_32_bytes(idx):
    n, dim = 43_100_000, 100
    indptr, indices = _tail_graph(n, 40_000, 12, 10, idx)
    uniq, inv = _local(indices)
    rows = np.unique(np.concatenate([np.random.default_rng(11).integers(0, 40_000, size=200), [0, 39_999]]))
    sub_ptr_np = indptr.cpu().numpy().astype(np.int64)

    def oracle_rows(dec_of):
        """oracle mean over the sampled destination rows; dec_of(ids tensor) -> numpy decoded rows"""
        pos = np.concatenate([np.arange(sub_ptr_np[r], sub_ptr_np[r + 1]) for r in rows] + [np.zeros(0, np.int64)])
        sp = np.zeros(len(rows) + 1, dtype=np.int64)
        sp[1:] = np.cumsum(sub_ptr_np[rows + 1] - sub_ptr_np[rows])
        ids = indices.long()[torch.from_numpy(pos).cuda()]
        u, iv = torch.unique(ids, return_inverse=True)
        dec = dec_of(u)
        return oc.spmm_csr(dec, sp, iv.cpu().numpy()), float(np.abs(dec).max())

    tr = torch.from_numpy(rows).cuda()
    # 8-bit affine SQ: 4.31e9 bytes of codes
    codes = _rand_u8((n, dim), 256, 12)
    assert codes.numel() > 2 ** 32
    params = torch.stack([torch.linspace(-2, 1, dim), torch.linspace(0.01, 0.04, dim)]).cuda()
    out = capi.sq_affine_decompress_spmm_csr(codes, params, indptr, indices, 8, dim)
    small = capi.sq_affine_decompress_spmm_csr(codes[uniq].contiguous(), params, indptr, inv, 8, dim)
    assert torch.equal(out, small)
    want, scale = oracle_rows(lambda u: oc.sq_affine_decompress(codes[u].cpu().numpy(), params.cpu().numpy(), 8, dim))
    assert np.allclose(out[tr].cpu().numpy(), want, rtol=RTOL, atol=RTOL * scale)
    # the same bytes as 8-bit log-domain codes (signed) and as packed 4-bit ones (200 columns)
    logcb = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
    for bits, d in ((8, dim), (4, 2 * dim)):
        out = capi.sq_decompress_spmm_csr(codes.view(torch.int8), logcb, indptr, indices, bits, d, d)
        small = capi.sq_decompress_spmm_csr(codes[uniq].contiguous().view(torch.int8), logcb, indptr, inv, bits, d, d)
        assert torch.equal(out, small)
        want, scale = oracle_rows(lambda u: oc.sq_decompress(codes[u].cpu().numpy().view(np.int8), logcb.cpu().numpy(),
                                                             bits, d, d))
        assert np.allclose(out[tr].cpu().numpy(), want, rtol=RTOL, atol=RTOL * scale)
    # the row fetch of the same table
    got = capi.fetch_rows(codes, indices)
    assert torch.equal(got, codes[indices.long()])
    # hybrid: the big table is the SQ one, the last rows of the id space are VQ rows
    n_vq = 100_000
    vq_codes = _rand_u8((n_vq, 5), 256, 13)
    vcb = torch.randn((5, 256, 20), device="cuda", generator=_gen(14))
    row_map = torch.arange(n, dtype=torch.int32, device="cuda")
    vq_ids = torch.arange(n - n_vq, n, device="cuda")[::2]
    row_map[vq_ids] = (-(vq_ids - (n - n_vq)) - 1).to(torch.int32)
    out = capi.hybrid_decompress_spmm_csr(row_map, codes, params, vq_codes, vcb, indptr, indices, dim)

    def hybrid_rows(u):
        m = row_map[u].long()
        hot = m >= 0
        local = m.cpu().numpy().copy()
        local[hot.cpu().numpy()] = np.arange(int(hot.sum()))
        return oc.hybrid_decompress(local, codes[m[hot]].cpu().numpy(), params.cpu().numpy(), vq_codes.cpu().numpy(),
                                    vcb.cpu().numpy(), dim, np.arange(u.numel()))

    want, scale = oracle_rows(hybrid_rows)
    assert np.allclose(out[tr].cpu().numpy(), want, rtol=RTOL, atol=RTOL * scale)
    del codes, out, small, got
    # plain aggregation of fp32 rows: 4.31e9 floats would be 17 GB; 2.2e9 floats cross 2^31 elements and 2^33 bytes
    nf = 22_000_000
    feat = torch.randn((nf, dim), device="cuda", generator=_gen(15))
    indptr, indices = _tail_graph(nf, 40_000, 12, 16, idx)
    uniq, inv = _local(indices)
    out = capi.spmm_csr(feat, indptr, indices)
    assert torch.equal(out, capi.spmm_csr(feat[uniq].contiguous(), indptr, inv))
    want = oc.spmm_csr(feat[uniq].cpu().numpy(), indptr.cpu().numpy().astype(np.int64), inv.cpu().numpy().astype(np.int64))
    assert np.allclose(out.cpu().numpy(), want, rtol=RTOL, atol=RTOL * 6)


@pytest.mark.parametrize("kind", ["sq_affine", "vq", "spmm"])
def test_fused_outputs_with_more_than_2_31_elements(kind):
    rows, dim, n = 17_000_000, 128, 1_000_000                 # 2.18e9 floats of output
    rng = np.random.default_rng(17)
    deg = rng.integers(0, 3, size=rows)
    indptr_np = np.zeros(rows + 1, dtype=np.int64)
    indptr_np[1:] = np.cumsum(deg)
    indices = torch.randint(0, n, (int(indptr_np[-1]),), device="cuda", generator=_gen(18))
    indptr = torch.from_numpy(indptr_np).cuda()
    if kind == "sq_affine":
        codes = _rand_u8((n, dim), 256, 19)
        params = torch.stack([torch.linspace(-2, 1, dim), torch.linspace(0.01, 0.04, dim)]).cuda()
        run = lambda ip, ix: capi.sq_affine_decompress_spmm_csr(codes, params, ip, ix, 8, dim)
        dec = lambda u: oc.sq_affine_decompress(codes[u].cpu().numpy(), params.cpu().numpy(), 8, dim)
    elif kind == "vq":
        codes = _rand_u8((n, 16), 256, 20)
        cb = torch.randn((16, 256, 8), device="cuda", generator=_gen(21))
        run = lambda ip, ix: capi.vq_decompress_spmm_csr(codes, cb, ip, ix, dim)
        dec = lambda u: oc.vq_decompress(codes[u].cpu().numpy(), cb.cpu().numpy(), dim)
    else:
        feat = torch.randn((n, dim), device="cuda", generator=_gen(22))
        run = lambda ip, ix: capi.spmm_csr(feat, ip, ix)
        dec = lambda u: feat[u].cpu().numpy()
    out = run(indptr, indices)
    assert out.numel() > 2 ** 31
    # the last rows as a block of their own (small offsets) must give the same values
    first = rows - 50_000
    e0 = int(indptr_np[first])
    tail = run((indptr[first:] - e0).contiguous(), indices[e0:].contiguous())
    if kind == "sq_affine":
        assert torch.equal(out[first:], tail)                 # integer sums: independent of the blocking
    else:
        assert torch.allclose(out[first:], tail, rtol=RTOL, atol=RTOL * 4)
    # and the oracle on the very end
    last = rows - 300
    e1 = int(indptr_np[last])
    u, iv = torch.unique(indices[e1:], return_inverse=True)
    d = dec(u)
    want = oc.spmm_csr(d, indptr_np[last:] - e1, iv.cpu().numpy())
    assert np.allclose(out[last:].cpu().numpy(), want, rtol=RTOL, atol=RTOL * float(np.abs(d).max()))
