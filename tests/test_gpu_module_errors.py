"""Error behaviour and argument handling of the F2CGTLib module on the GPU.  The reference aborts the
process on an unsupported dtype or bit width (`LOG(FATAL)`, src/common.h:29,51,64,80,102) and checks
nothing else; the replacement raises RuntimeError before any device work, accepts the reference's
keyword names (src/pybind.cu:8-28), and reads non-contiguous inputs through a contiguous copy."""
import numpy as np
import pytest
import torch

import f2cgt_amd
import f2cgt_oracle as oc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    return f2cgt_amd.load()


def _graph():
    ip = torch.tensor([0, 1, 3, 6], device="cuda")            # tests/test_fusion_decompress_spmm.py:20-21
    ix = torch.tensor([0, 1, 1, 2, 2, 0], device="cuda")
    return ip, ix


def _vq():
    g = torch.Generator(device="cuda").manual_seed(0)
    codes = torch.randint(0, 256, (3, 4), dtype=torch.uint8, device="cuda", generator=g)
    cb = torch.randn((4, 256, 8), device="cuda", generator=g)
    return codes, cb


def _sq():
    g = torch.Generator(device="cuda").manual_seed(1)
    codes = torch.randint(0, 256, (3, 16), dtype=torch.uint8, device="cuda", generator=g)
    cb = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
    return codes, cb


def test_bit_widths_outside_the_reference_set_raise(lib):
    x = torch.zeros((4, 8), dtype=torch.uint8, device="cuda")
    for bits in (0, 3, 5, 8, 16, -1):
        with pytest.raises(RuntimeError):
            lib.packbits(x, bits)
        with pytest.raises(RuntimeError):
            lib.unpackbits(x, bits, 8)
    codes, cb = _sq()
    ip, ix = _graph()
    for bits in (0, 3, 5, 7, 32):
        with pytest.raises(RuntimeError):
            lib.sq_decompress(codes, cb, bits, 16, 16)
        with pytest.raises(RuntimeError):
            lib.sq_decompress_spmm_csr(codes, cb, ip, ix, bits, 16, 16)
        with pytest.raises(RuntimeError):
            lib.sq_compress(torch.zeros((2, 16), device="cuda"), cb, bits, 16)
    with pytest.raises(RuntimeError):
        lib.unpackbits(x, 4, 17)                               # more columns than the packed row holds


def test_dtypes_outside_the_dispatch_raise(lib):
    codes, cb = _vq()
    ip, ix = _graph()
    with pytest.raises(RuntimeError):
        lib.vq_decompress(codes.to(torch.int32), cb, 32)       # int32 codes: src/common.h:68-82
    with pytest.raises(RuntimeError):
        lib.vq_decompress_spmm_csr(codes.float(), cb, ip, ix, 32)
    with pytest.raises(RuntimeError):
        lib.vq_decompress_spmm_csr(codes, cb.double(), ip, ix, 32)
    with pytest.raises(RuntimeError):
        lib.spmm_csr(torch.zeros((3, 4), dtype=torch.int32, device="cuda"), ip, ix)
    with pytest.raises(RuntimeError):
        lib.spmm_csr(torch.zeros((3, 4), device="cuda"), ip.float(), ix.float())
    with pytest.raises(RuntimeError, match="share one integer dtype"):
        lib.spmm_csr(torch.zeros((3, 4), device="cuda"), ip, ix.int())
    sq, scb = _sq()
    with pytest.raises(RuntimeError):
        lib.sq_decompress(sq, scb.double(), 4, 32, 32)
    with pytest.raises(RuntimeError):
        lib.sq_compress(torch.zeros((2, 16), dtype=torch.float64, device="cuda"), scb, 4, 16)
    with pytest.raises(RuntimeError):
        lib.pairwise_distance(torch.zeros((2, 4), dtype=torch.float64, device="cuda"), torch.zeros((2, 4), device="cuda"),
                              "l2")
    with pytest.raises(RuntimeError):
        lib.packbits(torch.zeros((2, 4), dtype=torch.int32, device="cuda"), 4)


def test_shapes_that_do_not_fit_raise(lib):
    codes, cb = _vq()
    ip, ix = _graph()
    with pytest.raises(RuntimeError):
        lib.vq_decompress(codes[:, :3], cb, 24)                # 3 code columns, 4 codebooks
    with pytest.raises(RuntimeError):
        lib.vq_decompress(codes, cb, 33)                       # more columns than the codebooks hold
    with pytest.raises(RuntimeError):
        lib.vq_decompress_spmm_csr(codes, cb[0], ip, ix, 8)    # 2-D codebooks
    with pytest.raises(RuntimeError):
        lib.vq_decompress_spmm_csr(codes, cb, ip[:0], ix, 32)  # empty indptr
    with pytest.raises(RuntimeError):
        lib.vq_decompress_spmm_csr(codes, cb, ip.reshape(2, 2), ix, 32)
    sq, scb = _sq()
    with pytest.raises(RuntimeError):
        lib.sq_decompress(sq, scb, 4, 32, 33)                  # 16 bytes hold 32 four-bit codes
    with pytest.raises(RuntimeError):
        lib.sq_decompress_spmm_csr(sq, scb, ip, ix, 4, 32, 33)
    with pytest.raises(RuntimeError):
        lib.sq_decompress(sq, scb[:, :4], 4, 32, 32)           # codebooks are [n, 5]
    with pytest.raises(RuntimeError):
        lib.sq_decompress(sq, scb, 4, 0, 32)
    with pytest.raises(RuntimeError):
        lib.sq_decompress(sq, scb, 4, 8, 32)                   # 4 column groups, 1 codebook
    with pytest.raises(RuntimeError):
        lib.pairwise_distance(torch.zeros((2, 4), device="cuda"), torch.zeros((2, 5), device="cuda"), "l2")
    with pytest.raises(RuntimeError):
        lib.KMeans(4, 8, "l2").fit(torch.zeros((3, 8), device="cuda"))      # fewer samples than clusters
    with pytest.raises(RuntimeError):
        lib.KMeans(4, 8, "l2").fit(torch.zeros((30, 7), device="cuda"))
    with pytest.raises(RuntimeError):
        lib.KMeans(0, 8, "l2")


def test_a_failed_call_leaves_the_library_usable(lib):
    codes, cb = _vq()
    ip, ix = _graph()
    want = oc.vq_decompress_spmm_csr(codes.cpu().numpy(), cb.cpu().numpy(), ip.cpu().numpy(), ix.cpu().numpy(), 32)
    with pytest.raises(RuntimeError):
        lib.vq_decompress_spmm_csr(codes, cb, ip, ix, 33)
    got = lib.vq_decompress_spmm_csr(codes, cb, ip, ix, 32)
    assert np.allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-6)


def test_non_contiguous_inputs_are_read_through_a_copy_and_inputs_are_not_modified(lib):
    g = torch.Generator(device="cuda").manual_seed(2)
    wide = torch.randint(0, 256, (3, 8), dtype=torch.uint8, device="cuda", generator=g)
    codes = wide[:, ::2]                                       # stride 2
    cb = torch.randn((256, 4, 8), device="cuda", generator=g).transpose(0, 1)       # [4, 256, 8], permuted
    ip, ix = _graph()
    ix2 = torch.stack([ix, ix], dim=1)[:, 0]                   # stride 2
    assert not codes.is_contiguous() and not cb.is_contiguous() and not ix2.is_contiguous()
    keep = (wide.clone(), cb.clone(), ip.clone(), ix2.clone())
    got = lib.vq_decompress_spmm_csr(codes, cb, ip, ix2, 32)
    want = lib.vq_decompress_spmm_csr(codes.contiguous(), cb.contiguous(), ip, ix.contiguous(), 32)
    assert torch.equal(got, want)
    assert torch.equal(lib.vq_decompress(codes, cb, 32), lib.vq_decompress(codes.contiguous(), cb.contiguous(), 32))
    feat = torch.randn((4, 3), device="cuda", generator=g).t()               # [3, 4] view of [4, 3]
    assert torch.equal(lib.spmm_csr(feat, ip, ix2), lib.spmm_csr(feat.contiguous(), ip, ix))
    assert torch.equal(wide, keep[0]) and torch.equal(cb, keep[1]) and torch.equal(ip, keep[2]) and torch.equal(ix2, keep[3])
    assert not got.requires_grad and got.is_contiguous() and got.dtype == torch.float32


def test_reference_keyword_names_and_fresh_outputs(lib):
    codes, cb = _vq()
    sq, scb = _sq()
    ip, ix = _graph()
    a = lib.vq_decompress_spmm_csr(compress_feat=codes, codebooks=cb, indptr=ip, indices=ix, feat_dim=32)
    b = lib.vq_decompress_spmm_csr(codes, cb, ip, ix, 32)
    assert torch.equal(a, b) and a.data_ptr() != b.data_ptr()  # every call returns a new tensor
    c = lib.sq_decompress_spmm_csr(compress_feat=sq, codebooks=scb, indptr=ip, indices=ix, target_bit=4,
                                   column_slice=32, feat_dim=32)
    d = lib.spmm_csr(feat=lib.sq_decompress(compress_data=sq, codebooks=scb, target_bits=4, column_slice=32,
                                            feat_dim=32), indptr=ip, indices=ix)
    assert torch.equal(c, d)
    with pytest.raises(TypeError):
        lib.sq_decompress_spmm_csr(compress_feat=sq, codebooks=scb, indptr=ip, indices=ix, target_bits=4,
                                   column_slice=32, feat_dim=32)               # the fused op's keyword is singular
    p = lib.packbits(unpack=lib.unpackbits(pack=sq, target_bits=4, unpack_dim=32), target_bits=4)
    assert torch.equal(p, sq)
    e = lib.vq_decompress(index_tensor=codes, codebooks=cb, feat_dim=30)       # feat_dim below n_cb * width truncates
    assert e.shape == (3, 30) and torch.equal(e, lib.vq_decompress(codes, cb, 32)[:, :30])
    dist = lib.pairwise_distance(x=cb[0, :5], y=cb[0], metric="anything-but-cosine")       # src/kmeans.cu:108-112
    assert torch.equal(dist, lib.pairwise_distance(cb[0, :5], cb[0], "l2"))
