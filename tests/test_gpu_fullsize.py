"""Full-size runs of the benchmark configurations (C1..C5 and the C5 encode step) on the GPU,
checked through size-independent properties:

  * sampled destination rows against the CPU oracle (exact decode of the rows they touch);
  * fused == unfused composition on the GPU (decode of the gathered unique rows, then spmm_csr);
  * a checksum of checksums: sum_r deg_r * out[r, :] == sum_e decoded[indices[e], :]  (fp64);
  * rows without edges are zero, rows with one edge equal the decoded source row bit for bit.
"""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc
from parity_bars import assert_mean_aggregate
from f2cgt_amd import capi, synth

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _decode_rows(wl, ids):
    """GPU decode (standalone ops) of the source rows `ids` (int64 tensor on the GPU)."""
    if wl["kind"] == "sq_affine":
        return capi.sq_affine_decompress(wl["codes"][ids].contiguous(), wl["params"], wl["bits"], wl["feat_dim"])
    if wl["kind"] == "vq":
        return capi.vq_decompress(wl["codes"][ids].contiguous(), wl["codebooks"], wl["feat_dim"])
    m = wl["row_map"][ids].long()
    out = torch.empty((ids.numel(), wl["feat_dim"]), dtype=torch.float32, device=ids.device)
    hot = m >= 0
    out[hot] = capi.sq_affine_decompress(wl["sq_codes"][m[hot]].contiguous(), wl["sq_params"], 8, wl["feat_dim"])
    out[~hot] = capi.vq_decompress(wl["vq_codes"][-m[~hot] - 1].contiguous(), wl["vq_codebooks"], wl["feat_dim"])
    return out


def _fused(wl):
    if wl["kind"] == "sq_affine":
        return capi.sq_affine_decompress_spmm_csr(wl["codes"], wl["params"], wl["indptr"], wl["indices"], wl["bits"],
                                                  wl["feat_dim"])
    if wl["kind"] == "vq":
        return capi.vq_decompress_spmm_csr(wl["codes"], wl["codebooks"], wl["indptr"], wl["indices"], wl["feat_dim"])
    return capi.hybrid_decompress_spmm_csr(wl["row_map"], wl["sq_codes"], wl["sq_params"], wl["vq_codes"],
                                           wl["vq_codebooks"], wl["indptr"], wl["indices"], wl["feat_dim"])


def _oracle_rows(wl, rows):
    """CPU oracle output for the destination rows `rows` (numpy ints)."""
    indptr = wl["indptr"].cpu().numpy().astype(np.int64)
    starts, ends = indptr[rows], indptr[rows + 1]
    sub_ptr = np.zeros(len(rows) + 1, dtype=np.int64)
    sub_ptr[1:] = np.cumsum(ends - starts)
    pos = np.concatenate([np.arange(s, e) for s, e in zip(starts, ends)]) if sub_ptr[-1] else np.zeros(0, np.int64)
    ids = wl["indices"][torch.from_numpy(pos).to(wl["indices"].device)].cpu().numpy().astype(np.int64)
    uniq, inv = np.unique(ids, return_inverse=True)
    tu = torch.from_numpy(uniq).to(wl["indices"].device)
    if wl["kind"] == "sq_affine":
        dec = oc.sq_affine_decompress(wl["codes"][tu].cpu().numpy(), wl["params"].cpu().numpy(), wl["bits"],
                                      wl["feat_dim"])
    elif wl["kind"] == "vq":
        dec = oc.vq_decompress(wl["codes"][tu].cpu().numpy(), wl["codebooks"].cpu().numpy(), wl["feat_dim"])
    else:
        m = wl["row_map"][tu].cpu().numpy().astype(np.int64)
        dec = np.empty((len(uniq), wl["feat_dim"]), dtype=np.float32)
        hot = m >= 0
        if hot.any():
            sq = wl["sq_codes"][torch.from_numpy(m[hot]).to(tu.device)].cpu().numpy()
            dec[hot] = oc.sq_affine_decompress(sq, wl["sq_params"].cpu().numpy(), 8, wl["feat_dim"])
        if (~hot).any():
            vq = wl["vq_codes"][torch.from_numpy(-m[~hot] - 1).to(tu.device)].cpu().numpy()
            dec[~hot] = oc.vq_decompress(vq, wl["vq_codebooks"].cpu().numpy(), wl["feat_dim"])
    return oc.spmm_csr(dec, sub_ptr, inv), oc.spmm_csr(dec.astype(np.float64), sub_ptr, inv), float(np.abs(dec).max())


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
@pytest.mark.parametrize("idx", [torch.int64, torch.int32])
def test_full_size_workload(name, idx):
    wl = synth.WORKLOADS[name](device="cuda", idx_dtype=idx)
    R, D = wl["R"], wl["feat_dim"]
    out = _fused(wl)
    torch.cuda.synchronize()
    assert out.shape == (R, D) and bool(torch.isfinite(out).all())

    # sampled rows against the CPU oracle
    rng = np.random.default_rng(0)
    rows = np.unique(np.concatenate([rng.integers(0, R, size=300), [0, R - 1]]))
    want, exact, scale = _oracle_rows(wl, rows)
    got = out[torch.from_numpy(rows).cuda()].cpu().numpy()
    # 1e-5 of each row's magnitude, and no further from the float64 mean than the reference's fp32 sum
    assert_mean_aggregate(got, want, exact, scale)

    # fused == unfused on the GPU: decode the unique source rows, aggregate with the plain kernel
    uniq, inv = torch.unique(wl["indices"].long(), return_inverse=True)
    dec = _decode_rows(wl, uniq)
    unfused = capi.spmm_csr(dec, wl["indptr"].long(), inv)
    torch.cuda.synchronize()
    row_scale = unfused.abs().amax(dim=1, keepdim=True).clamp_min(1e-30)
    assert bool(((out - unfused).abs() <= RTOL * row_scale).all())

    # checksum of checksums in fp64: sum_r deg_r * out[r] == sum_e decoded[index_e]
    deg = (wl["indptr"][1:] - wl["indptr"][:-1]).double()
    lhs = (out.double() * deg[:, None]).sum(dim=0)
    counts = torch.bincount(inv, minlength=uniq.numel()).double()
    rhs = (dec.double() * counts[:, None]).sum(dim=0)
    denom = (dec.double().abs() * counts[:, None]).sum(dim=0) + 1e-30
    assert float(((lhs - rhs).abs() / denom).max()) < 1e-6

    # rows with a single neighbour reproduce the decoded source row exactly
    one = torch.nonzero(deg == 1).flatten()[:5000]
    if one.numel():
        src = inv[wl["indptr"].long()[one]]
        assert torch.equal(out[one], dec[src])
    zero = torch.nonzero(deg == 0).flatten()
    if zero.numel():
        assert not bool(out[zero].any())


def test_full_size_encode():
    enc = synth.c5_encode(device="cuda")
    labels = capi.kmeans_predict(enc["x"], enc["centers"], "l2", u8=True)
    torch.cuda.synchronize()
    # every label is a true arg-min: compare against torch on the GPU in fp64, in slices
    x, c = enc["x"].double(), enc["centers"].double()
    bad = 0
    near = 0
    for s in range(0, enc["m"], 100_000):
        d = torch.cdist(x[s:s + 100_000], c) ** 2
        best2 = torch.topk(d, 2, dim=1, largest=False)
        ref = best2.indices[:, 0]
        gap = (best2.values[:, 1] - best2.values[:, 0]) / best2.values[:, 1].clamp_min(1e-30)
        tie = gap < 1e-6
        near += int(tie.sum())
        bad += int(((labels[s:s + 100_000].long() != ref) & ~tie).sum())
    assert bad == 0
    assert near < enc["m"] * 1e-3
    # sampled rows against the CPU oracle
    rows = np.random.default_rng(1).integers(0, enc["m"], size=2000)
    want, tie = oc.kmeans_predict(enc["x"][torch.from_numpy(rows).cuda()].cpu().numpy(), enc["centers"].cpu().numpy(), "l2")
    got = labels[torch.from_numpy(rows).cuda()].cpu().numpy().astype(np.int64)
    assert np.array_equal(got[~tie], want[~tie])
    # idempotence: assigning the centres to themselves gives the identity
    ident = capi.kmeans_predict(enc["centers"], enc["centers"], "l2")
    assert torch.equal(ident.cpu(), torch.arange(enc["n"]))


@pytest.mark.parametrize("name", ["c2", "c3", "c5"])
def test_full_size_fetch_then_fused_equals_fused_on_global_ids(name):
    """The reference's flow (fetch the code rows of the block's source nodes, run the fused
    operator on local indices) against the fused operator on global ids, at full size."""
    wl = synth.WORKLOADS[name](device="cuda")
    uniq, inv = torch.unique(wl["indices"], return_inverse=True)
    rows = capi.fetch_rows(wl["codes"], uniq)
    assert torch.equal(rows, wl["codes"][uniq])
    if wl["kind"] == "vq":
        local = capi.vq_decompress_spmm_csr(rows, wl["codebooks"], wl["indptr"], inv, wl["feat_dim"])
    else:
        local = capi.sq_affine_decompress_spmm_csr(rows, wl["params"], wl["indptr"], inv, wl["bits"], wl["feat_dim"])
    assert torch.equal(local, _fused(wl))


@pytest.mark.parametrize("form", ["affine", "log"])
def test_outputs_beyond_the_last_level_cache_take_the_streaming_stores(form):
    """Above 220 MB of output (140 MB for whole-line rows or denser graphs) the row-block kernels switch to non-temporal stores; the result must
    be what the same kernel writes with plain stores, which is how each half of the rows is run."""
    wl = synth.c2_sq4_affine(device="cuda", R=800_000)              # 320 MB of output
    indptr, indices, d = wl["indptr"], wl["indices"], wl["feat_dim"]
    if form == "affine":
        run = lambda ip, ix: capi.sq_affine_decompress_spmm_csr(wl["codes"], wl["params"], ip, ix, 4, d)
    else:
        logcb = torch.tensor([[0.01, 3.0, -6.643856, 1.5849625, 0.4]], device="cuda")
        run = lambda ip, ix: capi.sq_decompress_spmm_csr(wl["codes"], logcb, ip, ix, 4, d, d)
    full = run(indptr, indices)
    half = wl["R"] // 2
    e_half = int(indptr[half])
    first = run(indptr[:half + 1].contiguous(), indices[:e_half].contiguous())
    second = run((indptr[half:] - e_half).contiguous(), indices[e_half:].contiguous())
    assert full.shape[0] * d * 4 > 220_000_000 > first.shape[0] * d * 4
    assert torch.equal(full, torch.cat([first, second]))
