"""The reference's CPU-runnable flow for the aggregation path, in plain torch on host
cores: decompress the gathered rows, then a sparse mean matmul.

TEST/BENCHMARK INFRASTRUCTURE ONLY (the `cpu_baseline` leg of bench.py and the tests
that check it against the numpy oracle).  Never imported by the product.

Steps mirror the unfused composition of the reference (examples/compress.py:58-72 then
examples/conv.py:53-54):
  1. unique + relabel of `indices`   (the reference does this in its sampler; timed
                                      separately)
  2. gather the code rows of the unique ids
  3. torch dequantise: affine min + code*scale; VQ index_select per subspace + cat
     (tests/test_vq.py:17-19); hybrid = per-row dispatch of the two
  4. torch.sparse_csr_tensor(indptr, relabelled, 1/deg) @ X
"""
from __future__ import annotations

import time

import torch


def relabel(indices):
    uniq, inv = torch.unique(indices.long(), return_inverse=True)
    return uniq, inv


def dequant_affine(codes, params, bits, feat_dim):
    if bits < 8:
        per = 8 // bits
        shifts = torch.arange(per, dtype=torch.uint8) * bits
        un = (codes.unsqueeze(-1) >> shifts) & ((1 << bits) - 1)
        codes = un.reshape(codes.shape[0], -1)[:, :feat_dim]
    return params[0, :feat_dim] + codes[:, :feat_dim].float() * params[1, :feat_dim]


def dequant_vq(codes, codebooks, feat_dim):
    parts = [torch.index_select(codebooks[c], 0, codes[:, c].long()) for c in range(codebooks.shape[0])]
    return torch.cat(parts, dim=1)[:, :feat_dim]


def mean_spmm(indptr, inv, x, rows):
    indptr = indptr.long()
    deg = (indptr[1:] - indptr[:-1]).clamp_min(1).float()
    vals = torch.repeat_interleave(1.0 / deg, indptr[1:] - indptr[:-1])
    a = torch.sparse_csr_tensor(indptr, inv, vals, size=(rows, x.shape[0]))
    return a @ x


def run(wl, rows=None):
    """One pass over the first `rows` destination rows of workload `wl` (CPU tensors).
    Returns (output, seconds for steps 2-4, seconds for step 1)."""
    indptr = wl["indptr"].long()
    rows = wl["R"] if rows is None else min(rows, wl["R"])
    indptr = indptr[:rows + 1]
    indices = wl["indices"][:int(indptr[-1])]
    t0 = time.perf_counter()
    uniq, inv = relabel(indices)
    t1 = time.perf_counter()
    kind = wl["kind"]
    if kind == "sq_affine":
        x = dequant_affine(wl["codes"][uniq], wl["params"], wl["bits"], wl["feat_dim"])
    elif kind == "vq":
        x = dequant_vq(wl["codes"][uniq], wl["codebooks"], wl["feat_dim"])
    elif kind == "hybrid":
        m = wl["row_map"][uniq].long()
        x = torch.empty((uniq.numel(), wl["feat_dim"]), dtype=torch.float32)
        hot = m >= 0
        x[hot] = dequant_affine(wl["sq_codes"][m[hot]], wl["sq_params"], 8, wl["feat_dim"])
        x[~hot] = dequant_vq(wl["vq_codes"][-m[~hot] - 1], wl["vq_codebooks"], wl["feat_dim"])
    else:
        raise ValueError(kind)
    out = mean_spmm(indptr, inv, x, rows)
    t2 = time.perf_counter()
    return out, t2 - t1, t1 - t0
