"""Seeded synthetic workloads of the benchmark configurations (C1..C5).

Plain torch tensor generation, on any device; it defines the samplers in code so the
edge counts are reproducible:

  * Zipf(s) over ids [0, n): inverse CDF of the continuous density x^-s on [1, n+1),
    id = floor(x) - 1 (rank == id, id 0 is the hottest);
  * degree ~ discrete power law P(d) ~ d^-a for d >= 1, capped at `cap` (a row whose
    drawn degree exceeds the cap keeps `cap` neighbours): mean 2.24 for a=2.1, cap=12;
  * affine codes: clamp(round((x - min_c) / scale_c), 0, 2^bits - 1),
    scale_c = (max_c - min_c) / (2^bits - 1).

Every workload is a dict with the operator inputs, `E` (edges), `R` (rows) and
`algo_bytes` = E*(B_row + b_idx [+ 4 map]) + (R+1)*b_idx + R*D*4 + codebook bytes.

`compulsory_bytes(wl)` is the same sum with every *distinct* source row (and row-map entry)
counted once: what a launch must move through HBM at least, however well its caches work.
`algo_bytes` charges a hot row once per edge and can therefore exceed what moves.
"""
from __future__ import annotations

import math

import torch


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def zipf_ids(n_ids, size, s, gen, device, dtype=torch.int64):
    u = torch.rand(size, generator=gen, device=device, dtype=torch.float64)
    one_minus_s = 1.0 - s
    hi = float(n_ids + 1) ** one_minus_s
    x = (1.0 + u * (hi - 1.0)) ** (1.0 / one_minus_s)
    ids = x.floor().to(torch.int64) - 1
    return ids.clamp_(0, n_ids - 1).to(dtype)


def powerlaw_degrees(rows, exponent, cap, gen, device):
    d = torch.arange(1, cap, dtype=torch.float64)
    weights = d ** (-exponent)
    # Hurwitz tail sum_{d >= cap} d^-a, by direct summation plus an integral remainder
    far = torch.arange(cap, 200000, dtype=torch.float64)
    tail = (far ** (-exponent)).sum() + (200000.0 ** (1.0 - exponent)) / (exponent - 1.0)
    p = torch.cat([weights, tail.reshape(1)])
    p = (p / p.sum()).to(torch.float32).to(device)
    return torch.multinomial(p, rows, replacement=True, generator=gen) + 1


def csc_from_degrees(deg, idx_dtype):
    indptr = torch.zeros(deg.numel() + 1, dtype=torch.int64, device=deg.device)
    indptr[1:] = torch.cumsum(deg, 0)
    return indptr.to(idx_dtype)


def affine_quantise(x, bits):
    """-> (codes uint8 [N,D] unpacked, params fp32 [2,D])."""
    lo = x.min(dim=0).values
    hi = x.max(dim=0).values
    scale = (hi - lo) / float((1 << bits) - 1)
    scale = torch.where(scale > 0, scale, torch.ones_like(scale))
    q = torch.round((x - lo) / scale).clamp_(0, (1 << bits) - 1).to(torch.uint8)
    return q, torch.stack([lo, scale]).contiguous()


def pack_low_first(codes, bits):
    """torch-only packing (element i of a group in bits [bits*i, bits*(i+1)))."""
    per = 8 // bits
    n, d = codes.shape
    pad = (-d) % per
    if pad:
        codes = torch.cat([codes, torch.zeros((n, pad), dtype=torch.uint8, device=codes.device)], 1)
    grouped = codes.reshape(n, -1, per).to(torch.int32)
    shifts = (torch.arange(per, device=codes.device, dtype=torch.int32) * bits)
    return (grouped << shifts).sum(dim=2).to(torch.uint8).contiguous()


def _idx_bytes(dtype):
    return 8 if dtype == torch.int64 else 4


def c1_sq8_affine(device="cpu", idx_dtype=torch.int64, N=100_000, D=128, R=10_000, fanout=10, seed=0):
    g = _gen(seed, device)
    x = torch.randn((N, D), generator=g, device=device, dtype=torch.float32)
    codes, params = affine_quantise(x, 8)
    deg = torch.full((R,), fanout, dtype=torch.int64, device=device)
    indptr = csc_from_degrees(deg, idx_dtype)
    E = R * fanout
    indices = torch.randint(0, N, (E,), generator=g, device=device, dtype=torch.int64).to(idx_dtype)
    b = _idx_bytes(idx_dtype)
    return dict(name="c1_sq8_affine", kind="sq_affine", bits=8, codes=codes, params=params,
                indptr=indptr, indices=indices, feat_dim=D, R=R, E=E, N=N,
                algo_bytes=E * (D + b) + (R + 1) * b + R * D * 4 + 2 * D * 4)


def c2_sq4_affine(device="cpu", idx_dtype=torch.int64, N=2_400_000, D=100, R=250_000, cap=12,
                  exponent=2.1, zipf_s=1.1, seed=0, chunk=400_000):
    g = _gen(seed, device)
    col_scale = 0.5 + 1.5 * torch.rand((D,), generator=g, device=device, dtype=torch.float32)
    # two passes over a regenerable stream keep peak memory at one chunk of fp32 rows
    state = g.get_state()
    lo = torch.full((D,), float("inf"), device=device)
    hi = torch.full((D,), float("-inf"), device=device)
    for s in range(0, N, chunk):
        x = torch.randn((min(chunk, N - s), D), generator=g, device=device) * col_scale
        lo = torch.minimum(lo, x.min(dim=0).values)
        hi = torch.maximum(hi, x.max(dim=0).values)
    scale = (hi - lo) / 15.0
    scale = torch.where(scale > 0, scale, torch.ones_like(scale))
    params = torch.stack([lo, scale]).contiguous()
    g.set_state(state)
    packed = torch.empty((N, (D + 1) // 2), dtype=torch.uint8, device=device)
    for s in range(0, N, chunk):
        x = torch.randn((min(chunk, N - s), D), generator=g, device=device) * col_scale
        q = torch.round((x - lo) / scale).clamp_(0, 15).to(torch.uint8)
        packed[s:s + q.shape[0]] = pack_low_first(q, 4)
    deg = powerlaw_degrees(R, exponent, cap, g, device)
    indptr = csc_from_degrees(deg, idx_dtype)
    E = int(deg.sum().item())
    indices = zipf_ids(N, (E,), zipf_s, g, device, idx_dtype)
    b = _idx_bytes(idx_dtype)
    return dict(name="c2_sq4_affine", kind="sq_affine", bits=4, codes=packed, params=params,
                indptr=indptr, indices=indices, feat_dim=D, R=R, E=E, N=N,
                algo_bytes=E * (packed.shape[1] + b) + (R + 1) * b + R * D * 4 + 2 * D * 4)


def c3_vq(device="cpu", idx_dtype=torch.int64, N=10_000_000, n_cb=16, K=256, w=8, R=500_000, fanout=15,
          zipf_s=1.1, seed=0):
    g = _gen(seed, device)
    D = n_cb * w
    codebooks = torch.randn((n_cb, K, w), generator=g, device=device, dtype=torch.float32)
    codes = torch.randint(0, K, (N, n_cb), generator=g, device=device, dtype=torch.uint8)
    deg = torch.full((R,), fanout, dtype=torch.int64, device=device)
    indptr = csc_from_degrees(deg, idx_dtype)
    E = R * fanout
    indices = zipf_ids(N, (E,), zipf_s, g, device, idx_dtype)
    b = _idx_bytes(idx_dtype)
    return dict(name="c3_vq_%dx%d" % (n_cb, w), kind="vq", codes=codes, codebooks=codebooks,
                indptr=indptr, indices=indices, feat_dim=D, R=R, E=E, N=N,
                algo_bytes=E * (n_cb + b) + (R + 1) * b + R * D * 4 + n_cb * K * w * 4)


def c4_hybrid(device="cpu", idx_dtype=torch.int64, N=100_000_000, D=128, hot_frac=0.05, n_cb=8, K=256,
              w=16, R=1_000_000, fanout=12, zipf_s=1.2, seed=0):
    g = _gen(seed, device)
    n_hot = max(1, int(N * hot_frac))
    n_cold = max(1, N - n_hot)
    # rank == id, so the hottest 5 % are ids [0, n_hot)
    row_map = torch.empty((N,), dtype=torch.int32, device=device)
    row_map[:n_hot] = torch.arange(n_hot, dtype=torch.int32, device=device)
    row_map[n_hot:] = -torch.arange(N - n_hot, dtype=torch.int32, device=device) - 1
    sq_codes = torch.randint(0, 256, (n_hot, D), generator=g, device=device, dtype=torch.uint8)
    lo = torch.randn((D,), generator=g, device=device) - 3.0
    scale = (0.5 + torch.rand((D,), generator=g, device=device)) * (6.0 / 255.0)
    sq_params = torch.stack([lo, scale]).contiguous()
    vq_codes = torch.randint(0, K, (n_cold, n_cb), generator=g, device=device, dtype=torch.uint8)
    vq_codebooks = torch.randn((n_cb, K, w), generator=g, device=device, dtype=torch.float32)
    deg = torch.full((R,), fanout, dtype=torch.int64, device=device)
    indptr = csc_from_degrees(deg, idx_dtype)
    E = R * fanout
    indices = zipf_ids(N, (E,), zipf_s, g, device, idx_dtype)
    b = _idx_bytes(idx_dtype)
    hot_edges = int((indices < n_hot).sum().item())
    row_bytes = hot_edges * D + (E - hot_edges) * n_cb
    return dict(name="c4_hybrid", kind="hybrid", row_map=row_map, sq_codes=sq_codes, sq_params=sq_params,
                vq_codes=vq_codes, vq_codebooks=vq_codebooks, indptr=indptr, indices=indices,
                feat_dim=D, R=R, E=E, N=N, hot_edges=hot_edges,
                algo_bytes=row_bytes + E * (b + 4) + (R + 1) * b + R * D * 4 + n_cb * K * w * 4 + 2 * D * 4)


def c5_vq_wide(device="cpu", idx_dtype=torch.int64, N=240_000_000, n_cb=24, K=256, w=32, R=600_000,
               fanout=10, zipf_s=1.1, seed=0):
    wl = c3_vq(device, idx_dtype, N, n_cb, K, w, R, fanout, zipf_s, seed)
    wl["name"] = "c5_vq_%dx%d" % (n_cb, w)
    return wl


def c5_encode(device="cpu", m=1_000_000, k=32, n=256, seed=0):
    g = _gen(seed, device)
    x = torch.randn((m, k), generator=g, device=device, dtype=torch.float32)
    centers = torch.randn((n, k), generator=g, device=device, dtype=torch.float32)
    return dict(name="c5_encode", kind="encode", x=x, centers=centers, m=m, n=n, k=k,
                flops=2.0 * m * n * k, algo_bytes=m * k * 4 + n * k * 4 + m)


def scatter_ids(wl, mult=2_654_435_761):
    """The same workload with every source id passed through a fixed bijection of [0, N)
    (id -> id * mult mod N, mult coprime with N), so hot rows are no longer neighbours in the
    table.  Only the id stream changes; row contents are i.i.d., so the tables stay as they are
    (for the hybrid workload the row map is permuted with the ids)."""
    n = wl["N"]
    while math.gcd(mult, n) != 1:
        mult += 2
    idx = wl["indices"]
    perm = (idx.to(torch.int64) * (mult % n)) % n if n < (1 << 31) else ((idx.to(torch.int64) % n) * (mult % n)) % n
    out = dict(wl)
    out["indices"] = perm.to(idx.dtype)
    out["name"] = wl["name"] + "_scattered"
    if wl["kind"] == "hybrid":
        inv = torch.empty_like(wl["row_map"])
        src = torch.arange(n, device=idx.device, dtype=torch.int64)
        inv[(src * (mult % n)) % n] = wl["row_map"]
        out["row_map"] = inv
    return out


def compulsory_bytes(wl):
    """Bytes a launch cannot avoid moving: distinct source rows (and distinct row-map entries)
    once each, plus indices, row offsets, output and codebooks / column parameters."""
    idx = wl["indices"]
    b = _idx_bytes(idx.dtype)
    R, E, D = wl["R"], wl["E"], wl["feat_dim"]
    uniq = torch.unique(idx)
    if wl["kind"] == "hybrid":
        hot = int((wl["row_map"][uniq.to(torch.int64)] >= 0).sum().item())
        cb = wl["vq_codebooks"]
        rows = hot * D + (uniq.numel() - hot) * cb.shape[0] + uniq.numel() * 4
        fixed = cb.numel() * 4 + 2 * D * 4
    elif wl["kind"] == "vq":
        rows = uniq.numel() * wl["codes"].shape[1]
        fixed = wl["codebooks"].numel() * 4
    else:
        rows = uniq.numel() * wl["codes"].shape[1]
        fixed = 2 * D * 4
    return int(rows + E * b + (R + 1) * b + R * D * 4 + fixed)


def extra_blocks(wl, count, seed=1000):
    """`count` further CSC blocks over the same tables, drawn like the workload's own (same degree
    law, same id distribution, other seeds): lets a benchmark rotate graphs and outputs so that
    nothing but the tables' hot rows is still cached when a buffer comes round again."""
    dev = wl["indices"].device
    out = []
    for i in range(count):
        g = _gen(seed + i, dev)
        nb = dict(wl)
        if wl["name"].startswith("c2"):
            deg = powerlaw_degrees(wl["R"], 2.1, 12, g, dev)
            zs = 1.1
        else:
            deg = torch.full((wl["R"],), wl["E"] // wl["R"], dtype=torch.int64, device=dev)
            zs = 1.2 if wl["kind"] == "hybrid" else 1.1
        nb["indptr"] = csc_from_degrees(deg, wl["indptr"].dtype)
        nb["E"] = int(deg.sum().item())
        if wl["name"].startswith("c1"):
            nb["indices"] = torch.randint(0, wl["N"], (nb["E"],), generator=g, device=dev).to(wl["indices"].dtype)
        else:
            nb["indices"] = zipf_ids(wl["N"], (nb["E"],), zs, g, dev, wl["indices"].dtype)
        row_b = wl["codes"].shape[1] if "codes" in wl else None
        if row_b is not None:
            b = _idx_bytes(wl["indices"].dtype)
            fixed = wl["codebooks"].numel() * 4 if "codebooks" in wl else 2 * wl["feat_dim"] * 4
            nb["algo_bytes"] = nb["E"] * (row_b + b) + (wl["R"] + 1) * b + wl["R"] * wl["feat_dim"] * 4 + fixed
        elif wl["kind"] == "hybrid":
            b = _idx_bytes(wl["indices"].dtype)
            cb, D = wl["vq_codebooks"], wl["feat_dim"]
            hot = int((nb["indices"] < wl["sq_codes"].shape[0]).sum().item())
            nb["hot_edges"] = hot
            nb["algo_bytes"] = (hot * D + (nb["E"] - hot) * cb.shape[0] + nb["E"] * (b + 4) + (wl["R"] + 1) * b
                                + wl["R"] * D * 4 + cb.numel() * 4 + 2 * D * 4)
        out.append(nb)
    return out


WORKLOADS = {"c1": c1_sq8_affine, "c2": c2_sq4_affine, "c3": c3_vq, "c4": c4_hybrid, "c5": c5_vq_wide}
