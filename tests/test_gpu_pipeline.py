"""The Python callers around the operator library (f2cgt_amd/pipeline.py) against the CPU oracle:
the offline SQ / VQ encode pipeline, the compression manager and the fused GraphSAGE layer."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _graph(rng, rows, n_src, max_deg):
    deg = rng.integers(0, max_deg + 1, size=rows)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    indptr[1:] = np.cumsum(deg)
    indices = rng.integers(0, n_src, size=int(indptr[-1])).astype(np.int64)
    return indptr, indices


@pytest.mark.parametrize("bits", [1, 2, 4, 8, 16])
def test_sq_compress_pipeline_matches_oracle(bits):
    from f2cgt_amd import pipeline
    rng = np.random.default_rng(bits)
    x = np.concatenate([rng.uniform(-1, 1, size=(4000, 60)), rng.uniform(-1, 1, size=(4000, 50)) + 10],
                       axis=1).astype(np.float32)
    every_row = torch.arange(x.shape[0])
    store, cbs = pipeline.sq_compress(torch.from_numpy(x), bits, 60, sample_index=every_row, batch_rows=1500)
    want_cb = np.stack([oc.sq_codebook(x[:, :60]), oc.sq_codebook(x[:, 60:])])
    got_cb = cbs.cpu().numpy()
    assert np.array_equal(got_cb[:, :4], want_cb[:, :4])              # percentiles and exponents: exact
    assert np.allclose(got_cb[:, 4], want_cb[:, 4], rtol=1e-6)        # mean: summation order is free
    want = oc.sq_codes_to_storage(oc.sq_compress(x, got_cb, bits, 60), bits)
    got = store.cpu().numpy()
    assert got.dtype == (np.int16 if bits == 16 else np.int8)
    assert np.array_equal(got.view(want.dtype) if got.dtype != want.dtype else got, want)


def test_vq_compress_pipeline_labels_are_nearest_cosine_centres():
    from f2cgt_amd import pipeline
    rng = np.random.default_rng(0)
    x = rng.standard_normal((6000, 20)).astype(np.float32)   # slices of 8, 8 and a zero-padded 4
    torch.manual_seed(0)
    codes, cbs = pipeline.vq_compress(torch.from_numpy(x), 64, 8, sample_index=torch.arange(6000), batch_rows=2500)
    assert codes.dtype == torch.uint8 and tuple(codes.shape) == (6000, 3) and tuple(cbs.shape) == (3, 64, 8)
    cb = cbs.cpu().numpy()
    assert not cb[2, :, 4:].any()
    for i, (lo, hi) in enumerate([(0, 8), (8, 16), (16, 20)]):
        data = np.zeros((6000, 8), dtype=np.float32)
        data[:, :hi - lo] = x[:, lo:hi]
        want, tie = oc.kmeans_predict(data, cb[i], "cosine")
        got = codes[:, i].cpu().numpy().astype(np.int64)
        assert np.array_equal(got[~tie], want[~tie])
    # decode of the codes is what the manager serves
    dec = oc.vq_decompress(codes.cpu().numpy(), cb, 20)
    assert dec.shape == (6000, 20)


def _reference_layer(h_self, agg, conv):
    w_n = conv.fc_neigh.weight.detach().cpu().double().numpy()
    w_s = conv.fc_self.weight.detach().cpu().double().numpy()
    b_s = conv.fc_self.bias.detach().cpu().double().numpy()
    return h_self.astype(np.float64) @ w_s.T + b_s + agg.astype(np.float64) @ w_n.T


@pytest.mark.parametrize("method", ["sq", "vq"])
def test_one_level_manager_and_fused_layer(method):
    from f2cgt_amd import pipeline
    rng = np.random.default_rng(7)
    n, d = 3000, 64
    x = rng.standard_normal((n, d)).astype(np.float32)
    torch.manual_seed(1)
    if method == "sq":
        table, cbs = pipeline.sq_compress(torch.from_numpy(x), 4, 32, sample_index=torch.arange(n))
        configs = [(32, 4)]
        decode = lambda rows: oc.sq_decompress_per_byte_codebook(rows, cbs.cpu().numpy(), 4, 32, d)
    else:
        table, cbs = pipeline.vq_compress(torch.from_numpy(x), 256, 8, sample_index=torch.arange(n))
        configs = [(8, 256)]
        decode = lambda rows: oc.vq_decompress(rows, cbs.cpu().numpy(), d)
    meta = {"methods": [method], "feat_dim": d, "configs": configs, "codebooks": [cbs], "compression_data": table}
    # a sampled block: 500 destination rows, 1200 source rows (destinations first)
    src_ids = torch.from_numpy(rng.permutation(n)[:1200]).cuda()
    indptr, indices = _graph(rng, 500, 1200, 9)
    for fusion in (True, False):
        sm = pipeline.CompressionManager(meta, fusion=fusion)
        conv = pipeline.MySAGEConv(d, 16, "mean", sm).cuda()
        all_feat = sm.get_all_data(src_ids)
        h_self = sm.reorganize_seeds_data(sm.get_seeds_data(src_ids[:500]), all_feat, 500)
        if not fusion:
            assert h_self is None            # one level, no fusion: the layer slices h_neigh itself
        out = conv((torch.from_numpy(indptr).cuda(), torch.from_numpy(indices).cuda()), (h_self, all_feat))
        rows = table[src_ids].cpu().numpy()
        dec = decode(rows.view(np.uint8) if rows.dtype == np.int8 else rows)
        agg = oc.spmm_csr(dec, indptr, indices)
        want = _reference_layer(dec[:500], agg, conv)
        got = out.detach().cpu().numpy()
        assert np.allclose(got, want, rtol=1e-4, atol=1e-4 * np.abs(want).max())


def test_two_level_manager_serves_seeds_from_the_first_table():
    from f2cgt_amd import pipeline
    rng = np.random.default_rng(11)
    n, d = 2000, 32
    x = rng.standard_normal((n, d)).astype(np.float32)
    seeds = torch.from_numpy(np.sort(rng.permutation(n)[:300]))
    torch.manual_seed(2)
    seed_table, sq_cb = pipeline.sq_compress(torch.from_numpy(x)[seeds], 8, d, sample_index=torch.arange(300))
    table, vq_cb = pipeline.vq_compress(torch.from_numpy(x), 128, 8, sample_index=torch.arange(n))
    meta = {"methods": ["sq", "vq"], "feat_dim": d, "configs": [(d, 8), (8, 128)], "codebooks": [sq_cb, vq_cb],
            "compression_data": table, "seeds_compression_data": seed_table, "seeds": seeds}
    sm = pipeline.CompressionManager(meta, fusion=True)
    # block: the first 100 destinations are seeds, the other 150 are not; 700 sources in total
    others = np.setdiff1d(np.arange(n), seeds.numpy())
    src = np.concatenate([seeds.numpy()[:100], others[:600]])
    src_ids = torch.from_numpy(src).cuda()
    indptr, indices = _graph(rng, 250, 700, 6)
    seeds_feature = sm.get_seeds_data(src_ids[:100])
    all_feat = sm.get_all_data(src_ids)
    assert all_feat.dtype == table.dtype                       # fusion: still compressed
    h_self = sm.reorganize_seeds_data(seeds_feature, all_feat, 250)
    want_seed = oc.sq_decompress(seed_table.cpu().numpy()[:100], sq_cb.cpu().numpy(), 8, d, d)
    want_rest = oc.vq_decompress(table.cpu().numpy()[src[100:250]], vq_cb.cpu().numpy(), d)
    assert np.array_equal(h_self.cpu().numpy(), np.concatenate([want_seed, want_rest]))
    conv = pipeline.MySAGEConv(d, 8, "mean", sm, activation=torch.relu).cuda()
    out = conv((torch.from_numpy(indptr).cuda(), torch.from_numpy(indices).cuda()), (h_self, all_feat))
    dec = oc.vq_decompress(table.cpu().numpy()[src], vq_cb.cpu().numpy(), d)
    want = np.maximum(_reference_layer(np.concatenate([want_seed, want_rest]), oc.spmm_csr(dec, indptr, indices), conv), 0)
    assert np.allclose(out.detach().cpu().numpy(), want, rtol=1e-4, atol=1e-4 * np.abs(want).max())
    with pytest.raises(KeyError):
        sm.get_seeds_data(src_ids[100:110])


@pytest.mark.parametrize("ratio,with_seeds", [(8, False), (32, False), (64, True), (128, True)])
def test_artefact_files_round_trip_into_the_manager(tmp_path, ratio, with_seeds):
    # ratio 8 / 32: SQ at 4 / 1 bits per fp32 value; 64 / 128: VQ, 16 / 32 columns per code byte,
    # with the seed rows in an SQ table of their own (4-bit)
    from f2cgt_amd import pipeline
    rng = np.random.default_rng(ratio)
    n, d = 5000, 64
    x = rng.standard_normal((n, d)).astype(np.float32)
    seeds = torch.from_numpy(np.sort(rng.permutation(n)[:400])) if with_seeds else None
    torch.manual_seed(3)
    np.random.seed(3)
    meta = pipeline.run(str(tmp_path), torch.from_numpy(x), seeds=seeds, target_compression_ratio=ratio,
                        n_clusters=64)
    names = {"compression_meta.pt", "compression_data.pt"} | ({"seeds_compression_data.pt"} if with_seeds else set())
    assert {p.name for p in tmp_path.iterdir()} == names
    loaded = pipeline.load_compress_data(str(tmp_path))
    assert loaded["methods"] == (["sq"] if with_seeds else []) + (["sq"] if ratio <= 32 else ["vq"])
    assert loaded["feat_dim"] == d and loaded["configs"] == meta["configs"]
    if ratio <= 32:
        bits = 32 // ratio
        assert loaded["configs"][-1] == (64, bits)
        assert tuple(loaded["compression_data"].shape) == (n, d * bits // 8) and loaded["compression_data"].dtype == torch.int8
    else:
        w = ratio // 4
        assert loaded["configs"][-1] == (w, -1)
        assert tuple(loaded["compression_data"].shape) == (n, d // w) and loaded["compression_data"].dtype == torch.uint8
        assert tuple(loaded["codebooks"][-1].shape) == (d // w, 64, w)
    if with_seeds:
        assert loaded["configs"][0] == (64, 4) and torch.equal(loaded["seeds"], seeds)
        assert tuple(loaded["seeds_compression_data"].shape) == (400, d // 2)

    sm = pipeline.CompressionManager(loaded, fusion=True)
    src = np.concatenate([seeds.numpy()[:50], np.setdiff1d(np.arange(n), seeds.numpy())[:450]]) if with_seeds \
        else rng.permutation(n)[:500]
    src_ids = torch.from_numpy(src).cuda()
    indptr, indices = _graph(rng, 120, 500, 7)
    all_feat = sm.get_all_data(src_ids)
    n_seed_dst = 50 if with_seeds else 120
    h_self = sm.reorganize_seeds_data(sm.get_seeds_data(src_ids[:n_seed_dst]), all_feat, 120)
    conv = pipeline.MySAGEConv(d, 8, "mean", sm).cuda()
    out = conv((torch.from_numpy(indptr).cuda(), torch.from_numpy(indices).cuda()), (h_self, all_feat))

    table = loaded["compression_data"].numpy()[src]
    cb = loaded["codebooks"][-1].numpy()
    if ratio <= 32:
        dec = oc.sq_decompress_per_byte_codebook(table.view(np.uint8), cb, 32 // ratio, 64, d)
    else:
        dec = oc.vq_decompress(table, cb, d)
    want_self = dec[:120].copy()
    if with_seeds:
        seed_rows = loaded["seeds_compression_data"].numpy()[:50].view(np.uint8)
        want_self[:50] = oc.sq_decompress(seed_rows, loaded["codebooks"][0].numpy(), 4, 64, d)
    assert np.array_equal(h_self.cpu().numpy(), want_self)
    want = _reference_layer(want_self, oc.spmm_csr(dec, indptr, indices), conv)
    assert np.allclose(out.detach().cpu().numpy(), want, rtol=1e-4, atol=1e-4 * np.abs(want).max())
