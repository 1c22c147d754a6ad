"""Pins of the CPU oracle for VQ decode, CSC mean aggregation, the fused compositions,
the hybrid two-table op and the encode step, against torch library routines
(index_select, sparse CSR matmul, cdist, cosine_similarity) and brute force."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc


def _graph(rng, rows, n_src, max_deg, idx=np.int64):
    deg = rng.integers(0, max_deg + 1, size=rows)
    deg[rng.integers(0, rows)] = 0
    indptr = np.zeros(rows + 1, dtype=idx)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1])).astype(idx)
    return indptr, indices


def test_vq_decompress_is_index_select_cat():
    # the statement of tests/test_vq.py:17-19,63-65 incl. the zero padded second codebook
    rng = np.random.default_rng(0)
    c1 = rng.standard_normal((256, 60)).astype(np.float32)
    c2 = rng.standard_normal((256, 50)).astype(np.float32)
    l1 = rng.integers(0, 256, size=1000, dtype=np.uint8)
    l2 = rng.integers(0, 256, size=1000, dtype=np.uint8)
    want = torch.cat([torch.index_select(torch.from_numpy(c1), 0, torch.from_numpy(l1).long()),
                      torch.index_select(torch.from_numpy(c2), 0, torch.from_numpy(l2).long())], dim=1)
    cb = np.zeros((2, 256, 60), dtype=np.float32)
    cb[0] = c1
    cb[1, :, :50] = c2
    got = oc.vq_decompress(np.stack([l1, l2], axis=1), cb, 110)
    assert np.array_equal(got, want.numpy())


def test_vq_decompress_int16_and_fp16():
    rng = np.random.default_rng(1)
    cb = rng.standard_normal((2, 700, 4)).astype(np.float16)
    idx = rng.integers(0, 700, size=(50, 2)).astype(np.int16)
    got = oc.vq_decompress(idx, cb, 8)
    for r in (0, 17, 49):
        want = np.concatenate([cb[0, idx[r, 0]], cb[1, idx[r, 1]]]).astype(np.float32)
        assert np.array_equal(got[r], want)


@pytest.mark.parametrize("idx", [np.int32, np.int64])
def test_spmm_csr_is_sparse_mean_matmul(idx):
    rng = np.random.default_rng(2)
    feat = rng.standard_normal((300, 20)).astype(np.float32)
    indptr, indices = _graph(rng, 120, 300, 9, idx)
    got = oc.spmm_csr(feat, indptr, indices)
    deg = np.diff(indptr.astype(np.int64))
    vals = np.repeat(1.0 / np.maximum(deg, 1), deg)
    a = torch.sparse_csr_tensor(torch.from_numpy(indptr.astype(np.int64)),
                                torch.from_numpy(indices.astype(np.int64)),
                                torch.from_numpy(vals), size=(120, 300))
    want = (a @ torch.from_numpy(feat).double()).numpy()
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    assert not got[deg == 0].any()
    # index_add statement
    acc = torch.zeros(120, 20, dtype=torch.float64)
    rows = torch.from_numpy(np.repeat(np.arange(120), deg))
    acc.index_add_(0, rows, torch.from_numpy(feat).double()[torch.from_numpy(indices.astype(np.int64))])
    assert np.allclose(got, (acc / torch.from_numpy(np.maximum(deg, 1))[:, None]).numpy(), rtol=1e-5, atol=1e-6)


def test_spmm_csr_literal_graph_by_hand():
    # indptr/indices literal of tests/test_fusion_decompress_spmm.py:20-21
    indptr = np.array([0, 1, 3, 6])
    indices = np.array([0, 1, 1, 2, 2, 0])
    f = np.array([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]], dtype=np.float32)
    want = np.array([[1, 10], [(2 + 2) / 2, (20 + 20) / 2], [(4 + 4 + 1) / 3, (40 + 40 + 10) / 3]],
                    dtype=np.float32)
    assert np.array_equal(oc.spmm_csr(f, indptr, indices), want)


def test_spmm_csr_sequential_order_is_bitwise():
    # sums that depend on the order of addition: edge order must be honoured
    f = np.array([[1e8], [1.0], [-1e8], [1.0]], dtype=np.float32)
    indptr = np.array([0, 4, 8])
    indices = np.array([0, 1, 2, 3, 1, 3, 0, 2])
    got = oc.spmm_csr(f, indptr, indices)
    s1 = np.float32(np.float32(np.float32(np.float32(1e8) + np.float32(1)) + np.float32(-1e8)) + np.float32(1))
    s2 = np.float32(np.float32(np.float32(np.float32(1) + np.float32(1)) + np.float32(1e8)) + np.float32(-1e8))
    assert got[0, 0] == s1 / np.float32(4) and got[1, 0] == s2 / np.float32(4)


def test_fused_equals_composition_on_random_graphs():
    rng = np.random.default_rng(3)
    indptr, indices = _graph(rng, 200, 500, 12)
    # VQ, truncated feat_dim as in tests/test_fusion_decompress_spmm.py:67-70
    cb = rng.standard_normal((16, 256, 8)).astype(np.float32)
    codes = rng.integers(0, 256, size=(500, 16), dtype=np.uint8)
    fused = oc.vq_decompress_spmm_csr(codes, cb, indptr, indices, 100)
    assert np.array_equal(fused, oc.spmm_csr(oc.vq_decompress(codes, cb, 100), indptr, indices))
    # SQ, every width
    x = rng.uniform(-1, 1, size=(500, 64)).astype(np.float32)
    cbs = np.stack([oc.sq_codebook(x[:, :32]), oc.sq_codebook(x[:, 32:])])
    for bits in (1, 2, 4, 8, 16):
        store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, 32), bits)
        fused = oc.sq_decompress_spmm_csr(store, cbs, indptr, indices, bits, 32, 64)
        unfused = oc.spmm_csr(oc.sq_decompress(store, cbs, bits, 32, 64), indptr, indices)
        assert np.array_equal(fused, unfused)


def test_hybrid_dispatch_by_hand():
    rng = np.random.default_rng(4)
    D = 8
    sq = rng.integers(0, 256, size=(3, D), dtype=np.uint8)
    params = np.stack([rng.standard_normal(D), rng.uniform(0.01, 0.1, D)]).astype(np.float32)
    cb = rng.standard_normal((2, 16, 4)).astype(np.float32)
    vq = rng.integers(0, 16, size=(4, 2), dtype=np.uint8)
    row_map = np.array([0, -1, 2, -4, 1, -2], dtype=np.int32)
    ids = np.arange(6)
    dec = oc.hybrid_decompress(row_map, sq, params, vq, cb, D, ids)
    for i, m in enumerate(row_map):
        if m >= 0:
            want = (params[0] + (sq[m].astype(np.float32) * params[1]).astype(np.float32)).astype(np.float32)
        else:
            r = -m - 1
            want = np.concatenate([cb[0, vq[r, 0]], cb[1, vq[r, 1]]])
        assert np.array_equal(dec[i], want)
    indptr = np.array([0, 3, 3, 6])
    indices = np.array([0, 1, 5, 2, 3, 4])
    assert np.array_equal(oc.hybrid_decompress_spmm_csr(row_map, sq, params, vq, cb, indptr, indices, D),
                          oc.spmm_csr(dec, indptr, indices))


def test_pairwise_distance_against_torch():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((70, 33)).astype(np.float32)
    y = rng.standard_normal((19, 33)).astype(np.float32)
    tx, ty = torch.from_numpy(x), torch.from_numpy(y)
    l2 = oc.pairwise_distance(x, y, "l2")
    assert np.allclose(l2, (torch.cdist(tx.double(), ty.double()) ** 2).numpy(), rtol=1e-5, atol=1e-5)
    # the statement of examples/my_kmeans.py:43-48
    stmt = ((tx.unsqueeze(1) - ty.unsqueeze(0)) ** 2.0).sum(dim=-1)
    assert np.allclose(l2, stmt.numpy(), rtol=1e-6, atol=1e-6)
    # any string but "cosine" is squared L2 (src/kmeans.cu:108-112)
    assert np.array_equal(l2, oc.pairwise_distance(x, y, "euclidean"))
    cos = oc.pairwise_distance(x, y, "cosine")
    stmt = 1 - torch.nn.functional.cosine_similarity(tx.unsqueeze(1), ty.unsqueeze(0), dim=2)
    assert np.allclose(cos, stmt.numpy(), rtol=1e-5, atol=1e-6)
    assert abs(oc.pairwise_distance(x[:1], x[:1], "l2")[0, 0]) == 0.0


def test_kmeans_predict_first_minimum_and_near_ties():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((200, 8)).astype(np.float32)
    c = rng.standard_normal((16, 8)).astype(np.float32)
    c[9] = c[3]  # exact duplicate: the first index must win
    labels, near = oc.kmeans_predict(x, c, "l2")
    brute = np.array([np.argmin([((xi.astype(np.float64) - cj) ** 2).sum() for cj in c]) for xi in x])
    assert np.array_equal(labels, brute)
    assert not (labels == 9).any()
    assert np.array_equal(near, np.isin(labels, [3]))  # rows whose best is the duplicated centre
    labels_c, _ = oc.kmeans_predict(x, c, "cosine")
    cosine = 1 - (x.astype(np.float64) @ c.T.astype(np.float64)) / (
        np.linalg.norm(x.astype(np.float64), axis=1)[:, None] * np.linalg.norm(c.astype(np.float64), axis=1)[None])
    assert np.array_equal(labels_c, cosine.argmin(axis=1))


def test_golden_fixtures_reproduce(golden):
    g = golden
    for bits in (1, 2, 4):
        assert np.array_equal(oc.packbits(g["pack%d_in" % bits], bits), g["pack%d_out" % bits])
        assert np.array_equal(oc.unpackbits(g["pack%d_out" % bits], bits, 13), g["unpack%d_out" % bits])
    for bits in (1, 2, 4, 8, 16):
        assert np.array_equal(oc.sq_compress(g["sq_x"], g["sq_codebooks"], bits, 12), g["sq%d_codes" % bits])
        assert np.array_equal(oc.sq_decompress(g["sq%d_store" % bits], g["sq_codebooks"], bits, 12, 24),
                              g["sq%d_decoded" % bits])
        assert np.array_equal(oc.sq_decompress_spmm_csr(g["sq%d_store" % bits][:3], g["sq_codebooks"],
                                                        g["g_indptr"], g["g_indices"], bits, 12, 24),
                              g["g_sq%d_fused" % bits])
    assert np.array_equal(oc.vq_decompress(g["vq_idx"], g["vq_codebooks"], 10), g["vq_decoded"])
    assert np.array_equal(oc.spmm_csr(g["g_feat"], g["g_indptr"], g["g_indices"]), g["g_spmm"])
    assert np.array_equal(oc.hybrid_decompress_spmm_csr(g["hy_map"], g["hy_sq"], g["hy_params"], g["hy_vq"],
                                                        g["hy_cb"], g["hy_indptr"], g["hy_indices"], 8),
                          g["hy_fused"])
    for metric in ("l2", "cosine"):
        assert np.array_equal(oc.kmeans_predict(g["enc_x"], g["enc_c"], metric)[0], g["enc_labels_" + metric])
        assert np.array_equal(oc.pairwise_distance(g["enc24_x"], g["enc24_c"], metric, dtype=np.float64),
                              g["enc24_dist_" + metric])
    assert np.array_equal(oc.fetch_rows(g["fetch_table"], g["fetch_index"]), g["fetch_plain"])
    assert np.array_equal(oc.fetch_rows(g["fetch_table"], g["fetch_index"], g["fetch_hot"], g["fetch_slot"]),
                          g["fetch_cached"])
    assert np.array_equal(g["fetch_plain"], g["fetch_table"][g["fetch_index"]])


# ---- row fetch of the feature cache --------------------------------------------------------
def test_fetch_rows_is_index_select_and_a_cache_of_copies_changes_nothing():
    rng = np.random.default_rng(21)
    table = rng.integers(0, 256, size=(500, 7), dtype=np.uint8)
    index = rng.integers(0, 500, size=300)
    want = torch.index_select(torch.from_numpy(table), 0, torch.from_numpy(index)).numpy()
    assert np.array_equal(oc.fetch_rows(table, index), want)
    hot_ids = rng.permutation(500)[:120]
    slot_map = np.full(500, -1, dtype=np.int32)
    slot_map[hot_ids] = np.arange(120, dtype=np.int32)
    assert np.array_equal(oc.fetch_rows(table, index, table[hot_ids], slot_map), want)
    # rows that have a slot come from the cache, the others from the table
    marked = oc.fetch_rows(table, index, np.zeros((120, 7), dtype=np.uint8), slot_map)
    cached = slot_map[index] >= 0
    assert not marked[cached].any() and np.array_equal(marked[~cached], want[~cached])
