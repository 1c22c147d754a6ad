"""Writes tests/golden/f2cgt_golden.npz: small input/expected-output vectors for every
operator of the path, produced by the CPU oracle (oracle/f2cgt_oracle.py).

The reference holds no expected-value fixtures for this path (its tests only compare
its own fused and unfused kernels), so these vectors are this repository's regression
lock for the oracle and a fixed target for the HIP kernels.  The literal CSC graph is
the one the reference tests use (tests/test_fusion_decompress_spmm.py:20-21).

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import f2cgt_oracle as oc  # noqa: E402


def main():
    rng = np.random.default_rng(20240521)
    out = {}

    # bit packing, ragged tails
    for bits in (1, 2, 4):
        u = rng.integers(0, 256, size=(7, 13), dtype=np.uint8)
        out["pack%d_in" % bits] = u
        out["pack%d_out" % bits] = oc.packbits(u, bits)
        out["unpack%d_out" % bits] = oc.unpackbits(out["pack%d_out" % bits], bits, 13)

    # log-domain SQ, two codebooks of 12 columns
    x = rng.uniform(-1, 1, size=(16, 24)).astype(np.float32)
    x[:, 12:] += 10
    x[0, 0] = 0.0
    cbs = np.stack([oc.sq_codebook(x[:, :12]), oc.sq_codebook(x[:, 12:])])
    out["sq_x"] = x
    out["sq_codebooks"] = cbs
    for bits in (1, 2, 4, 8, 16):
        codes = oc.sq_compress(x, cbs, bits, 12)
        store = oc.sq_codes_to_storage(codes, bits)
        out["sq%d_codes" % bits] = codes
        out["sq%d_store" % bits] = store
        out["sq%d_decoded" % bits] = oc.sq_decompress(store, cbs, bits, 12, 24)

    # the reference's literal CSC block
    indptr = np.array([0, 1, 3, 6], dtype=np.int64)
    indices = np.array([0, 1, 1, 2, 2, 0], dtype=np.int64)
    out["g_indptr"], out["g_indices"] = indptr, indices
    feat = rng.standard_normal((3, 24)).astype(np.float32)
    out["g_feat"] = feat
    out["g_spmm"] = oc.spmm_csr(feat, indptr, indices)
    for bits in (1, 2, 4, 8, 16):
        out["g_sq%d_fused" % bits] = oc.sq_decompress_spmm_csr(
            out["sq%d_store" % bits][:3], cbs, indptr, indices, bits, 12, 24)

    # VQ: 3 subspaces of width 4, feat_dim 10 (last subspace truncated)
    vq_cb = rng.standard_normal((3, 16, 4)).astype(np.float32)
    vq_idx = rng.integers(0, 16, size=(10, 3), dtype=np.uint8)
    out["vq_codebooks"], out["vq_idx"] = vq_cb, vq_idx
    out["vq_decoded"] = oc.vq_decompress(vq_idx, vq_cb, 10)
    out["g_vq_fused"] = oc.vq_decompress_spmm_csr(vq_idx, vq_cb, indptr, indices, 10)

    # affine SQ (4 and 8 bit) and the two-table hybrid
    xa = (rng.standard_normal((12, 10)) * rng.uniform(0.5, 2, size=10)).astype(np.float32)
    for bits in (4, 8):
        params = oc.sq_affine_params(xa, bits)
        codes = oc.sq_affine_compress(xa, params, bits)
        store = oc.packbits(codes, bits) if bits < 8 else codes
        out["aff%d_params" % bits] = params
        out["aff%d_store" % bits] = store
        out["aff%d_decoded" % bits] = oc.sq_affine_decompress(store, params, bits, 10)
        out["g_aff%d_fused" % bits] = oc.sq_affine_decompress_spmm_csr(store, params, indptr, indices,
                                                                     bits, 10)
    hy_cb = rng.standard_normal((2, 8, 4)).astype(np.float32)
    hy_sq = rng.integers(0, 256, size=(2, 8), dtype=np.uint8)
    hy_vq = rng.integers(0, 8, size=(3, 2), dtype=np.uint8)
    hy_params = np.stack([rng.standard_normal(8), rng.uniform(0.01, 0.05, size=8)]).astype(np.float32)
    hy_map = np.array([1, -1, -3, 0, -2], dtype=np.int32)
    hy_indptr = np.array([0, 2, 2, 5, 6], dtype=np.int64)
    hy_indices = np.array([0, 1, 4, 3, 2, 1], dtype=np.int64)
    out.update(hy_cb=hy_cb, hy_sq=hy_sq, hy_vq=hy_vq, hy_params=hy_params, hy_map=hy_map,
               hy_indptr=hy_indptr, hy_indices=hy_indices)
    out["hy_fused"] = oc.hybrid_decompress_spmm_csr(hy_map, hy_sq, hy_params, hy_vq, hy_cb, hy_indptr,
                                                    hy_indices, 8)

    # encode
    ex = rng.standard_normal((40, 8)).astype(np.float32)
    ec = rng.standard_normal((10, 8)).astype(np.float32)
    out["enc_x"], out["enc_c"] = ex, ec
    for metric in ("l2", "cosine"):
        out["enc_dist_" + metric] = oc.pairwise_distance(ex, ec, metric)
        labels, near = oc.kmeans_predict(ex, ec, metric)
        assert not near.any()
        out["enc_labels_" + metric] = labels

    # a wider encode case (24 dimensions: the matrix-core path of the distance matrix)
    wx = (rng.standard_normal((50, 24)) + 2.0).astype(np.float32)
    wc = (rng.standard_normal((40, 24)) + 2.0).astype(np.float32)
    out["enc24_x"], out["enc24_c"] = wx, wc
    for metric in ("l2", "cosine"):
        out["enc24_dist_" + metric] = oc.pairwise_distance(wx, wc, metric, dtype=np.float64)

    # row fetch of the feature cache: 50-byte rows, a third of the ids cached with other bytes
    ft = rng.integers(0, 256, size=(30, 50), dtype=np.uint8)
    fi = rng.integers(0, 30, size=21).astype(np.int64)
    fslot = np.full(30, -1, dtype=np.int32)
    fslot[::3] = np.arange(10, dtype=np.int32)
    fhot = rng.integers(0, 256, size=(10, 50), dtype=np.uint8)
    out.update(fetch_table=ft, fetch_index=fi, fetch_slot=fslot, fetch_hot=fhot)
    out["fetch_plain"] = oc.fetch_rows(ft, fi)
    out["fetch_cached"] = oc.fetch_rows(ft, fi, fhot, fslot)

    path = os.path.join(HERE, "f2cgt_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
