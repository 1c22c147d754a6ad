"""CPU oracle for the fused feature-decompression + neighbour-aggregation path.

TEST INFRASTRUCTURE ONLY.  This module is the checker that the parity tests, the
smoke test and the `cpu_baseline` leg of the benchmark compare the HIP library
against.  Nothing in the product (`f2cgt_amd/`) may import it, and it must never be
used as a fallback for a missing HIP extension.

Every function is a from-scratch numpy restatement of the algorithm in the reference
source it cites (paths relative to the reference checkout).  The arithmetic is fp32
with the operation order of the reference kernel text; fp64 is used only where
stated (to define a correctly rounded fp32 `log2`/`exp2`, and for brute-force
classification of near-ties).

What pins each function (tests/test_oracle_*.py):
  packbits/unpackbits   numpy.packbits(bitorder="little") for 1 bit, exhaustive byte
                        tables for 2/4 bits, round trips, ragged tails.
  sq_compress           invariants of the kernel text (range, monotone in |x|, code
                        symmetry, saturation) + exact powers of two.
  sq_decompress         brute force of every code against exact powers of two,
                        <=1 ulp against torch.exp2 on fp32, +-mean for 1 bit.
  vq_decompress         torch.index_select + cat (tests/test_vq.py:17-19,63-65).
  spmm_csr              torch.sparse_csr_tensor(indptr, indices, 1/deg) @ X and
                        index_add_; deg-0 rows.
  fused ops             == spmm_csr(decompress(.)) bit for bit
                        (tests/test_fusion_decompress_spmm.py:27-33,113-120).
  pairwise_distance     torch.cdist**2 / 1-cosine_similarity, fp64 brute force.
  fetch_rows            torch.index_select on the full table; a cache of any subset of
                        rows must not change the result.
  sq_affine_*, hybrid   closed forms stated by the benchmark configuration.
  kmeans_update         per-cluster means by boolean masks in fp64, a hand-computed case, and the
                        invariants of a Lloyd step (inertia never rises, a fixed point stays put).
  sq_lut(fma=True)      the same table with the product and sum of the exponent fused into one
                        rounding (what a contracting compiler makes of the kernel text); the test
                        counts the entries on which the two readings differ.

PARITY UNPINNED (nothing in the reference or in this container fixes them):
  * last-ulp behaviour of CUDA `exp2f`/`log2f` inside the reference kernels.  This
    oracle defines both as the correctly rounded fp32 function (fp64 libm result
    rounded once to fp32); the reference's GPU result may differ by an ulp.
  * raft 23.10's internal rounding and tie rule in `kmeans_predict` /
    `pairwise_distance` (third-party, not vendored).  This oracle follows the torch
    statement in examples/my_kmeans.py:43-55,116-125 (first minimum wins).
  * `KMeans.fit` (raft k-means++/random initialisation and RNG stream): only the update step and
    the stopping rules are restated here.
  * whether the reference's CUDA build contracts `fabs(value) * k + emin`
    (src/sq_quantization.cu:146-151, src/fusion_spmm.cu:203-207) into one fused multiply-add:
    nvcc does so by default, the torch statement of the same formula (tests/test_sq.py:96-106)
    cannot.  `sq_lut` follows the torch statement; `sq_lut(..., fma=True)` gives the other reading.
"""
from __future__ import annotations

import numpy as np

F32 = np.float32


# --------------------------------------------------------------------------- #
# packbits / unpackbits                                                        #
# --------------------------------------------------------------------------- #
def packbits(unpack: np.ndarray, target_bits: int) -> np.ndarray:
    """uint8 [R,U] -> uint8 [R, ceil(U / (8/bits))].

    Follows src/packbits.cu:24-41: element i of a group lands in bits
    [bits*i, bits*(i+1)) of the output byte ("small end"), the tail group is
    zero padded, values are masked to `bits` bits first.
    """
    assert target_bits in (1, 2, 4)
    unpack = np.ascontiguousarray(unpack).view(np.uint8)
    rows, udim = unpack.shape
    per = 8 // target_bits
    pdim = (udim + per - 1) // per
    mask = (1 << target_bits) - 1
    padded = np.zeros((rows, pdim * per), dtype=np.uint8)
    padded[:, :udim] = unpack & mask
    grouped = padded.reshape(rows, pdim, per).astype(np.uint16)
    shifts = (np.arange(per, dtype=np.uint16) * target_bits)
    return (grouped << shifts).sum(axis=2).astype(np.uint8)


def unpackbits(pack: np.ndarray, target_bits: int, unpack_dim: int) -> np.ndarray:
    """Inverse of packbits; src/packbits.cu:84-94 and src/cuda_utils.cuh:5-9:
    out[r][o] = (pack[r][o / n] >> (bits * (o % n))) & mask, n = 8 / bits."""
    assert target_bits in (1, 2, 4)
    pack = np.ascontiguousarray(pack).view(np.uint8)
    per = 8 // target_bits
    mask = (1 << target_bits) - 1
    cols = np.arange(unpack_dim)
    src = pack[:, cols // per]
    return ((src >> ((cols % per) * target_bits).astype(np.uint8)) & mask).astype(np.uint8)


# --------------------------------------------------------------------------- #
# log-domain scalar quantisation (the reference's SQ)                          #
# --------------------------------------------------------------------------- #
def log2_f32(x: np.ndarray) -> np.ndarray:
    """Correctly rounded fp32 log2 (stands in for the kernel's log2f,
    src/sq_quantization.cu:52)."""
    return np.log2(np.asarray(x, dtype=F32).astype(np.float64)).astype(F32)


def exp2_f32(x: np.ndarray) -> np.ndarray:
    """Correctly rounded fp32 exp2 (stands in for the kernel's exp2f,
    src/sq_quantization.cu:150)."""
    return np.exp2(np.asarray(x, dtype=F32).astype(np.float64)).astype(F32)


def sq_codebook(sample: np.ndarray) -> np.ndarray:
    """[fmin, fmax, emin, emax, mean] as fp32[5].

    Follows tests/test_sq.py:8-21 and examples/process_compress.py:55-68.  With a
    float32 sample numpy's percentile returns float32 and torch.tensor() keeps it, so
    the statement runs in fp32 throughout: emin = log2(fmin), emax = log2(fmax) + 1e-5
    (log2 taken as the correctly rounded fp32 function).  Helper for building test
    inputs; the operators receive the finished [n,5] tensor.
    """
    epsilon = 1e-5
    s = np.abs(np.asarray(sample, dtype=F32))
    fmin = F32(max(np.percentile(s, 0.5), epsilon))
    fmax = F32(max(np.percentile(s, 99.5), 2 * epsilon))
    emin = log2_f32(fmin)
    emax = F32(log2_f32(fmax) + F32(epsilon))
    mean = s.mean(dtype=F32)
    if mean < 0.1:
        mean = F32(mean + F32(0.1))
    return np.array([fmin, fmax, emin, emax, mean], dtype=F32)


def sq_compress(src: np.ndarray, codebooks: np.ndarray, target_bits: int,
                column_slice: int) -> np.ndarray:
    """fp32 [R,D] -> fp32 [R,D] holding integer code values.

    Follows src/sq_quantization.cu:33-60 (and tests/test_sq.py:24-45).  Column j
    uses codebook j // column_slice.  Quirks reproduced on purpose: x == 0 is
    encoded as negative; a value at or below fmin can floor to -1 when
    log2f(fmin_f32) lands one ulp below emin.
    """
    src = np.asarray(src, dtype=F32)
    codebooks = np.asarray(codebooks, dtype=F32)
    if target_bits == 1:
        return np.where(src <= 0, F32(0), F32(1)).astype(F32)
    drange = F32(1 << (target_bits - 1))
    cb = np.arange(src.shape[1]) // column_slice
    fmin, fmax = codebooks[cb, 0], codebooks[cb, 1]
    emin, emax = codebooks[cb, 2], codebooks[cb, 3]
    neg = src <= 0
    v = np.abs(src)
    v = np.minimum(np.maximum(v, fmin), fmax)
    v = log2_f32(v)
    v = ((v - emin) / (emax - emin)).astype(F32) * drange
    v = np.floor(v.astype(F32))
    v = np.where(neg, F32(-1) - v, v).astype(F32)
    if target_bits < 8:
        v = v + drange
    return v.astype(F32)


def sq_codes_to_storage(codes_f32: np.ndarray, target_bits: int) -> np.ndarray:
    """What the caller does with sq_compress' output
    (examples/process_compress.py:128-139): cast, and pack when bits < 8."""
    if target_bits < 8:
        return packbits(codes_f32.astype(np.uint8), target_bits)
    if target_bits == 8:
        return codes_f32.astype(np.int8)
    return codes_f32.astype(np.int16)


def sq_lut(codebooks: np.ndarray, target_bits: int, fma: bool = False) -> np.ndarray:
    """Decoded value of every raw code, per codebook: fp32 [n_cb, 2**bits].

    fma=True: the exponent |v| * k + emin rounded once (the product of two fp32 values is exact in
    fp64, the sum is formed there and rounded to fp32), which is what a compiler that contracts
    the kernel's `fabs(value) * k + emin` (src/sq_quantization.cu:146-151) into a fused multiply-add
    evaluates.  Not used by any parity check: it measures how far the two readings are apart.

    The index is the raw bit pattern as stored (unsigned for bits < 8, the
    two's-complement pattern of the signed code for 8/16 bits).  Formula:
    src/sq_quantization.cu:136-152 / tests/test_sq.py:96-106, evaluated in fp32
    without FMA: k = (emax - emin) / drange; v = code' + 0.5;
    out = exp2(|v| * k + emin) * sign(v).
    """
    codebooks = np.asarray(codebooks, dtype=F32)
    n = 1 << target_bits
    raw = np.arange(n, dtype=np.int64)
    if target_bits == 1:
        mean = codebooks[:, 4:5]
        return ((raw.astype(F32) - F32(0.5))[None, :] * (F32(2) * mean)).astype(F32)
    drange = F32(1 << (target_bits - 1))
    if target_bits < 8:
        signed = raw.astype(F32) - drange
    else:
        signed = np.where(raw >= n // 2, raw - n, raw).astype(F32)
    v = signed + F32(0.5)
    sign = np.where(v >= 0, F32(1), F32(-1))
    emin, emax = codebooks[:, 2:3], codebooks[:, 3:4]
    k = ((emax - emin) / drange).astype(F32)
    if fma:
        t = (np.abs(v)[None, :].astype(np.float64) * k.astype(np.float64) + emin.astype(np.float64)).astype(F32)
    else:
        t = (np.abs(v)[None, :] * k).astype(F32) + emin
    return (exp2_f32(t.astype(F32)) * sign[None, :]).astype(F32)


def _sq_raw_codes(compress_data: np.ndarray, target_bits: int, feat_dim: int) -> np.ndarray:
    """Raw unsigned bit pattern of every column's code, int64 [R, feat_dim]."""
    if target_bits < 8:
        return unpackbits(compress_data, target_bits, feat_dim).astype(np.int64)
    if target_bits == 8:
        return np.ascontiguousarray(compress_data).view(np.uint8)[:, :feat_dim].astype(np.int64)
    return np.ascontiguousarray(compress_data).view(np.uint16)[:, :feat_dim].astype(np.int64)


def sq_decompress(compress_data: np.ndarray, codebooks: np.ndarray, target_bits: int,
                  column_slice: int, feat_dim: int) -> np.ndarray:
    """codes -> fp32 [R, feat_dim]; src/sq_quantization.cu:123-153.  Column j uses
    codebook j // column_slice (per OUTPUT column)."""
    raw = _sq_raw_codes(compress_data, target_bits, feat_dim)
    lut = sq_lut(codebooks, target_bits)
    cb = np.arange(feat_dim) // column_slice
    return lut[cb[None, :], raw]


def sq_decompress_per_byte_codebook(compress_data, codebooks, target_bits, column_slice,
                                    feat_dim):
    """The fused kernel's codebook choice (src/fusion_spmm.cu:180): per PACKED BYTE j,
    codebook = j * pack / column_slice.  Equal to sq_decompress iff
    column_slice % pack == 0."""
    pack = max(8 // target_bits, 1)
    raw = _sq_raw_codes(compress_data, target_bits, feat_dim)
    lut = sq_lut(codebooks, target_bits)
    cols = np.arange(feat_dim)
    cb = ((cols // pack) * pack) // column_slice
    return lut[cb[None, :], raw]


# --------------------------------------------------------------------------- #
# per-column affine scalar quantisation (benchmark-defined extension)          #
# --------------------------------------------------------------------------- #
def sq_affine_params(x: np.ndarray, target_bits: int) -> np.ndarray:
    """fp32 [2, D]: row 0 = per-column min, row 1 = per-column scale
    = (max - min) / (2**bits - 1)."""
    x = np.asarray(x, dtype=F32)
    lo = x.min(axis=0)
    hi = x.max(axis=0)
    scale = ((hi - lo) / F32((1 << target_bits) - 1)).astype(F32)
    scale = np.where(scale > 0, scale, F32(1)).astype(F32)
    return np.stack([lo, scale]).astype(F32)


def sq_affine_compress(x: np.ndarray, params: np.ndarray, target_bits: int) -> np.ndarray:
    """codes = clamp(round((x - min) / scale), 0, 2**bits - 1), uint8 [R,D]
    (packed by the caller with packbits when bits < 8)."""
    x = np.asarray(x, dtype=F32)
    q = np.rint(((x - params[0]) / params[1]).astype(F32))
    return np.clip(q, 0, (1 << target_bits) - 1).astype(np.uint8)


def sq_affine_decompress(compress_data: np.ndarray, params: np.ndarray, target_bits: int,
                         feat_dim: int) -> np.ndarray:
    """x = min_c + code * scale_c in fp32, product rounded before the sum (no FMA).
    Codes are unsigned; sub-byte codes are packed low bits first
    (same packing as src/packbits.cu:37-38)."""
    if target_bits < 8:
        raw = unpackbits(compress_data, target_bits, feat_dim)
    else:
        raw = np.ascontiguousarray(compress_data).view(np.uint8)[:, :feat_dim]
    prod = (raw.astype(F32) * params[1][None, :feat_dim]).astype(F32)
    return (params[0][None, :feat_dim] + prod).astype(F32)


# --------------------------------------------------------------------------- #
# vector quantisation decode                                                   #
# --------------------------------------------------------------------------- #
def vq_decompress(index_tensor: np.ndarray, codebooks: np.ndarray, feat_dim: int) -> np.ndarray:
    """out[i][j] = codebooks[j // w][idx[i][j // w]][j % w], j < feat_dim;
    src/vq_quantization.cu:18-31.  fp16 codebooks are widened to fp32."""
    codebooks = np.asarray(codebooks)
    n_cb, _, w = codebooks.shape
    idx = np.asarray(index_tensor).astype(np.int64)
    parts = [codebooks[c][idx[:, c]] for c in range(n_cb)]
    return np.concatenate(parts, axis=1)[:, :feat_dim].astype(F32)


# --------------------------------------------------------------------------- #
# CSC mean aggregation                                                         #
# --------------------------------------------------------------------------- #
def spmm_csr(feat: np.ndarray, indptr: np.ndarray, indices: np.ndarray) -> np.ndarray:
    """out[r] = (sum over edges of row r, in edge order, of feat[indices[e]]) /
    max(deg, 1); src/fusion_spmm.cu:24-42.  The sum runs sequentially in the
    feature dtype, then one division; rows without edges give 0."""
    feat = np.asarray(feat)
    indptr = np.asarray(indptr).astype(np.int64)
    indices = np.asarray(indices).astype(np.int64)
    rows = indptr.shape[0] - 1
    deg = indptr[1:] - indptr[:-1]
    acc = np.zeros((rows, feat.shape[1]), dtype=feat.dtype)
    max_deg = int(deg.max()) if rows else 0
    for k in range(max_deg):
        live = np.nonzero(deg > k)[0]
        acc[live] = acc[live] + feat[indices[indptr[live] + k]]
    denom = np.where(deg == 0, 1, deg).astype(F32).astype(feat.dtype)
    return (acc / denom[:, None]).astype(feat.dtype)


def vq_decompress_spmm_csr(compress_feat, codebooks, indptr, indices, feat_dim):
    """src/fusion_spmm.cu:83-104: spmm_csr with vq_decompress inlined."""
    uniq, inv = np.unique(np.asarray(indices).astype(np.int64), return_inverse=True)
    table = vq_decompress(np.asarray(compress_feat)[uniq], codebooks, feat_dim)
    return spmm_csr(table, indptr, inv)


def sq_decompress_spmm_csr(compress_feat, codebooks, indptr, indices, target_bit,
                           column_slice, feat_dim):
    """src/fusion_spmm.cu:173-236: spmm_csr with SQ decode inlined; the codebook is
    picked per packed byte (:180)."""
    uniq, inv = np.unique(np.asarray(indices).astype(np.int64), return_inverse=True)
    table = sq_decompress_per_byte_codebook(np.asarray(compress_feat)[uniq], codebooks,
                                            target_bit, column_slice, feat_dim)
    return spmm_csr(table, indptr, inv)


def sq_affine_decompress_spmm_csr(compress_feat, params, indptr, indices, target_bit,
                                  feat_dim):
    uniq, inv = np.unique(np.asarray(indices).astype(np.int64), return_inverse=True)
    table = sq_affine_decompress(np.asarray(compress_feat)[uniq], params, target_bit, feat_dim)
    return spmm_csr(table, indptr, inv)


def hybrid_decompress(row_map, sq_codes, sq_params, vq_codes, vq_codebooks, feat_dim, ids):
    """Two-table decode of the rows `ids`: row_map[id] >= 0 selects row row_map[id]
    of the 8-bit affine SQ table, row_map[id] < 0 selects row -row_map[id]-1 of
    the VQ table."""
    ids = np.asarray(ids).astype(np.int64)
    m = np.asarray(row_map)[ids].astype(np.int64)
    out = np.empty((ids.shape[0], feat_dim), dtype=F32)
    hot = m >= 0
    if hot.any():
        out[hot] = sq_affine_decompress(np.asarray(sq_codes)[m[hot]], sq_params, 8, feat_dim)
    if (~hot).any():
        out[~hot] = vq_decompress(np.asarray(vq_codes)[-m[~hot] - 1], vq_codebooks, feat_dim)
    return out


def hybrid_decompress_spmm_csr(row_map, sq_codes, sq_params, vq_codes, vq_codebooks,
                               indptr, indices, feat_dim):
    """Mean aggregation where every source row is decoded from the table its
    row_map entry names (benchmark-defined two-level extension; the reference's
    closest form is examples/compress.py:39-54,74-106)."""
    uniq, inv = np.unique(np.asarray(indices).astype(np.int64), return_inverse=True)
    table = hybrid_decompress(row_map, sq_codes, sq_params, vq_codes, vq_codebooks,
                              feat_dim, uniq)
    return spmm_csr(table, indptr, inv)


# --------------------------------------------------------------------------- #
# Row fetch in front of the operators (examples/tensor_cache.py:49-58)
# --------------------------------------------------------------------------- #
def fetch_rows(table: np.ndarray, index: np.ndarray, hot: np.ndarray = None,
               slot_map: np.ndarray = None) -> np.ndarray:
    """TensorCache.__getitem__: row `index[i]` of the table, taken from the cache of hot rows
    where the id has a slot (shmtensor cache_fetch) and from the table itself otherwise
    (uva_fetch).  The cache holds copies (`gpu_data = data[cache_candidates]`,
    examples/tensor_cache.py:79), so the result equals `table[index]` whenever it does."""
    index = np.asarray(index).astype(np.int64)
    out = np.empty((index.size,) + table.shape[1:], dtype=table.dtype)
    for i, key in enumerate(index):
        slot = -1 if slot_map is None else int(slot_map[key])
        out[i] = hot[slot] if slot >= 0 else table[key]
    return out


# --------------------------------------------------------------------------- #
# VQ encode: pairwise distance + argmin                                        #
# --------------------------------------------------------------------------- #
def pairwise_distance(x: np.ndarray, y: np.ndarray, metric: str, dtype=F32) -> np.ndarray:
    """[m,k] x [n,k] -> [m,n].  "cosine" -> 1 - x.y / (|x||y|); every other string
    -> squared L2, sum((x - y)**2), no square root (src/kmeans.cu:108-112,
    examples/my_kmeans.py:43-55)."""
    x = np.asarray(x).astype(dtype)
    y = np.asarray(y).astype(dtype)
    if metric == "cosine":
        xn = np.sqrt((x * x).sum(axis=1, dtype=dtype))
        yn = np.sqrt((y * y).sum(axis=1, dtype=dtype))
        dot = x @ y.T
        denom = np.maximum(xn[:, None] * yn[None, :], dtype(1e-8))
        return (dtype(1) - dot / denom).astype(dtype)
    out = np.empty((x.shape[0], y.shape[0]), dtype=dtype)
    step = max(1, (1 << 24) // max(1, y.shape[0] * x.shape[1]))
    for s in range(0, x.shape[0], step):
        d = x[s:s + step, None, :] - y[None, :, :]
        out[s:s + step] = (d * d).sum(axis=2, dtype=dtype)
    return out


def kmeans_predict(x: np.ndarray, centers: np.ndarray, metric: str):
    """labels int64 [m] = first minimum of the distance row
    (examples/my_kmeans.py:116-125), plus a mask of rows that are NEAR-TIES:
    relative gap between the two smallest fp64 distances below 1e-6.  Labels are
    only specified outside the mask."""
    d = pairwise_distance(x, centers, metric, dtype=np.float64)
    labels = d.argmin(axis=1)
    if d.shape[1] < 2:
        return labels.astype(np.int64), np.zeros(d.shape[0], dtype=bool)
    part = np.partition(d, 1, axis=1)[:, :2]
    gap = part[:, 1] - part[:, 0]
    scale = np.maximum(np.abs(part[:, 1]), 1e-30)
    return labels.astype(np.int64), (gap / scale) < 1e-6


def kmeans_update(x: np.ndarray, labels: np.ndarray, centers: np.ndarray):
    """One Lloyd centre update (examples/my_kmeans.py:128-147, compute_new_centers): a centre becomes
    the plain mean of the rows assigned to it, whatever the metric; a centre without members keeps
    its value.  -> (new centres fp32, sum_c |dc|, sum_c |dc|^2): the centre shift of :100-103 and its
    squared form (the quantity raft's fit tests, src/kmeans.cu:61-75).  The sums run in fp64: the
    GPU adds in fp32 in an order of its own, so the comparison carries a tolerance."""
    x64 = x.astype(np.float64)
    n, k = centers.shape
    sums = np.zeros((n, k), dtype=np.float64)
    np.add.at(sums, labels.astype(np.int64), x64)
    counts = np.bincount(labels.astype(np.int64), minlength=n).astype(np.float64)
    new = centers.astype(np.float64).copy()
    has = counts > 0
    new[has] = sums[has] / counts[has, None]
    new = new.astype(F32)
    d2 = ((new.astype(np.float64) - centers.astype(np.float64)) ** 2).sum(axis=1)
    return new, float(np.sqrt(d2).sum()), float(d2.sum())


def kmeans_stop(shift_abs: float, shift_sq: float, tol: float, rule: int) -> bool:
    """Stopping rules: 1 = raft (sum of squared centre shifts below tol, src/kmeans.cu:61-75 via
    KMeansParams.tol), 2 = the reference's own trainer ((sum of centre shifts)^2 < tol,
    examples/my_kmeans.py:105), with its tol growing by 1.2 per iteration (:111) left to the caller."""
    if rule == 1:
        return shift_sq < tol
    if rule == 2:
        return shift_abs * shift_abs < tol
    return False
