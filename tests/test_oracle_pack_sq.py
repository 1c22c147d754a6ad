"""Pins of the CPU oracle for packbits/unpackbits and the scalar quantisers, against
independent statements: numpy.packbits, exhaustive byte tables, exact powers of two,
torch.exp2 and the invariants of the reference kernel text."""
import numpy as np
import pytest
import torch

import f2cgt_oracle as oc


# ---- packbits / unpackbits -------------------------------------------------------------
@pytest.mark.parametrize("udim", [1, 7, 8, 9, 64, 100])
def test_pack_1bit_is_numpy_packbits_little(udim):
    rng = np.random.default_rng(udim)
    u = rng.integers(0, 2, size=(5, udim), dtype=np.uint8)
    assert np.array_equal(oc.packbits(u, 1), np.packbits(u, axis=1, bitorder="little"))


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_unpack_every_byte_value(bits):
    # a byte b holds 8/bits codes, code i = (b >> bits*i) & mask: check by python ints
    per = 8 // bits
    pack = np.arange(256, dtype=np.uint8).reshape(256, 1)
    got = oc.unpackbits(pack, bits, per)
    for b in range(256):
        assert [int(v) for v in got[b]] == [(b >> (bits * i)) & ((1 << bits) - 1) for i in range(per)]


@pytest.mark.parametrize("bits", [1, 2, 4])
@pytest.mark.parametrize("udim", [1, 3, 8, 13, 50, 100])
def test_pack_roundtrip_and_tail(bits, udim):
    rng = np.random.default_rng(bits * 100 + udim)
    u = rng.integers(0, 256, size=(9, udim), dtype=np.uint8)  # high bits must be masked off
    p = oc.packbits(u, bits)
    per = 8 // bits
    assert p.shape == (9, (udim + per - 1) // per)
    assert np.array_equal(oc.unpackbits(p, bits, udim), u & ((1 << bits) - 1))
    # zero padded tail: unpacking past unpack_dim gives zeros
    full = oc.unpackbits(p, bits, p.shape[1] * per)
    assert not full[:, udim:].any()


def test_pack_4bit_low_nibble_first_literal():
    u = np.array([[0x1, 0x2, 0xF, 0x0, 0x7]], dtype=np.uint8)
    assert oc.packbits(u, 4).tolist() == [[0x21, 0x0F, 0x07]]
    u2 = np.array([[1, 2, 3, 0, 3]], dtype=np.uint8)
    assert oc.packbits(u2, 2).tolist() == [[0b00111001, 0b11]]


def test_pack_empty():
    assert oc.packbits(np.zeros((0, 5), np.uint8), 4).shape == (0, 3)
    assert oc.unpackbits(np.zeros((0, 3), np.uint8), 4, 5).shape == (0, 5)


# ---- log-domain SQ ------------------------------------------------------------------------
def _codebook(fmin, fmax, mean=0.3):
    return np.array([[fmin, fmax, np.log2(fmin), np.log2(fmax), mean]], dtype=np.float32)


@pytest.mark.parametrize("bits", [2, 4, 8, 16])
def test_sq_decompress_exact_powers_of_two(bits):
    # emin = 0, emax = drange  ->  k = 1, value(code') = 2^(|code' + 0.5|) * sign: every
    # exponent is a half-integer; with emin = 0.5 they are integers -> exact powers of two
    drange = 1 << (bits - 1)
    if drange > 64:
        emax = 64.5  # k = 64/drange keeps exponents representable for 8/16 bits
    else:
        emax = drange + 0.5
    cb = np.array([[1.0, 2.0, 0.5, emax, 0.3]], dtype=np.float32)
    lut = oc.sq_lut(cb, bits)[0]
    k = np.float32(np.float32(emax - 0.5) / np.float32(drange))
    n = 1 << bits
    for raw in range(0, n, max(1, n // 512)):
        signed = raw - drange if bits < 8 else (raw - n if raw >= n // 2 else raw)
        v = signed + 0.5
        expo = np.float32(np.float32(abs(v)) * k) + np.float32(0.5)
        want = np.float32(np.sign(v)) * np.float32(2.0 ** float(expo))
        assert lut[raw] == want, (bits, raw)
    if drange <= 64:  # integer exponents: exact powers of two
        assert lut[drange if bits < 8 else 0] == np.float32(2.0)       # code' = 0  -> 2^(0.5+0.5)
        assert lut[(drange - 1) if bits < 8 else n - 1] == np.float32(-2.0)  # code' = -1


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_sq_lut_within_one_ulp_of_torch_exp2(bits):
    rng = np.random.default_rng(bits)
    x = rng.uniform(-1, 1, size=(4000, 3)).astype(np.float32)
    cb = np.stack([oc.sq_codebook(x)])
    drange = np.float32(1 << (bits - 1))
    n = 1 << bits
    raw = np.arange(n)
    signed = (raw - drange) if bits < 8 else np.where(raw >= n // 2, raw - n, raw)
    v = torch.tensor(signed, dtype=torch.float32) + 0.5
    k = torch.tensor((cb[0, 3] - cb[0, 2]) / drange)
    t = v.abs().mul(k).add(torch.tensor(cb[0, 2])).exp2().mul(torch.sign(v)).numpy()
    lut = oc.sq_lut(cb, bits)[0]
    ulp = np.spacing(np.abs(lut))
    assert np.all(np.abs(lut - t) <= ulp)
    assert np.array_equal(np.sign(lut), np.sign(t))


def test_sq_1bit_is_plus_minus_mean():
    cb = np.array([[0.1, 1.0, -3.0, 0.0, 0.37], [0.1, 1.0, -3.0, 0.0, 1.5]], dtype=np.float32)
    lut = oc.sq_lut(cb, 1)
    assert lut.tolist() == [[-np.float32(0.37), np.float32(0.37)], [-1.5, 1.5]]
    x = np.array([[-2.0, 0.0, 0.5, 3.0]], dtype=np.float32)
    assert oc.sq_compress(x, cb, 1, 2).tolist() == [[0, 0, 1, 1]]  # x == 0 encodes as negative


@pytest.mark.parametrize("bits", [2, 4, 8, 16])
def test_sq_compress_invariants(bits):
    rng = np.random.default_rng(bits + 10)
    x = rng.uniform(-1, 1, size=(3000, 8)).astype(np.float32)
    cb = np.stack([oc.sq_codebook(x)])
    fmin, fmax = cb[0, 0], cb[0, 1]
    inner = (np.abs(x) > fmin * 1.001) & (np.abs(x) < fmax)
    codes = oc.sq_compress(x, cb, bits, 8)
    drange = 1 << (bits - 1)
    assert np.array_equal(codes, np.round(codes))
    lo, hi = (0, 2 * drange - 1) if bits < 8 else (-drange, drange - 1)
    assert codes[inner].min() >= lo and codes[inner].max() <= hi
    # sign symmetry: code(-x) = 2*drange-1-code(x) (bits<8) / -1-code(x) (bits>=8), x != 0
    neg = oc.sq_compress(-x, cb, bits, 8)
    if bits < 8:
        assert np.array_equal(neg, 2 * drange - 1 - codes)
    else:
        assert np.array_equal(neg, -1 - codes)
    # monotone in |x| for positive inputs
    xs = np.sort(np.abs(x[:, 0]))[:, None].repeat(8, axis=1)
    cs = oc.sq_compress(xs, cb, bits, 8)[:, 0]
    assert np.all(np.diff(cs) >= 0)
    # saturation at and beyond fmax
    big = np.full((1, 8), fmax * 4, dtype=np.float32)
    assert np.array_equal(oc.sq_compress(big, cb, bits, 8), oc.sq_compress(np.full((1, 8), fmax, np.float32), cb, bits, 8))


@pytest.mark.parametrize("bits", [2, 4, 8, 16])
def test_sq_compress_bucket_edges_exact(bits):
    # fmin = 1, fmax = 2^drange: emin = 0, emax = drange -> code' = floor(log2 x):
    # x = 2^j lands exactly on the lower edge of bucket j (needs a correct log2 at powers of two)
    drange = 1 << (bits - 1)
    top = min(drange, 100)
    cb = np.array([[1.0, 2.0 ** top, 0.0, float(drange), 0.3]], dtype=np.float32)
    j = np.arange(0, top)
    x = (2.0 ** j).astype(np.float32)[None, :]
    codes = oc.sq_compress(x, cb, bits, x.shape[1])[0]
    bias = drange if bits < 8 else 0
    assert np.array_equal(codes, j + bias)
    # a little below the edge (one ulp below is not enough: fp32 log2 rounds it back up)
    just_below = (x * np.float32(1 - 2.0 ** -12))[:, 1:]
    codes_b = oc.sq_compress(just_below, cb, bits, x.shape[1])[0]
    assert np.array_equal(codes_b, j[1:] - 1 + bias)


@pytest.mark.parametrize("bits", [1, 2, 4, 8, 16])
def test_sq_roundtrip_error_bound_and_multi_codebook(bits):
    # the shape of tests/test_sq.py:162-185: two column groups with different ranges
    rng = np.random.default_rng(bits + 77)
    a = rng.uniform(-1, 1, size=(2000, 60)).astype(np.float32)
    b = (rng.uniform(-1, 1, size=(2000, 50)) + 10).astype(np.float32)
    x = np.concatenate([a, b], axis=1)
    cbs = np.stack([oc.sq_codebook(a), oc.sq_codebook(b)])
    store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, 60), bits)
    dec = oc.sq_decompress(store, cbs, bits, 60, 110)
    # per-group decode equals the single-codebook decode of that group
    store_a = oc.sq_codes_to_storage(oc.sq_compress(a, cbs[:1], bits, 60), bits)
    assert np.array_equal(dec[:, :60], oc.sq_decompress(store_a, cbs[:1], bits, 60, 60))
    assert np.array_equal(np.sign(dec), np.where(x <= 0, -1, 1))
    if bits >= 8:  # fine quantiser: relative error bounded by the bucket width
        inner = (np.abs(x) > cbs[0, 0] * 1.01) & (np.abs(x) < cbs[0, 1])
        inner[:, 60:] = (np.abs(b) > cbs[1, 0] * 1.01) & (np.abs(b) < cbs[1, 1])
        width = (cbs[:, 3] - cbs[:, 2]) / (1 << (bits - 1))
        tol = np.where(np.arange(110) < 60, 2.0 ** width[0] - 1, 2.0 ** width[1] - 1)
        rel = np.abs(dec - x) / np.abs(x)
        assert np.all(rel[inner] <= np.broadcast_to(tol, x.shape)[inner] * 1.001)


def test_sq_fused_codebook_choice_equals_standalone_when_aligned():
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, size=(50, 32)).astype(np.float32)
    cbs = np.stack([oc.sq_codebook(x[:, :16]), oc.sq_codebook(x[:, 16:] * 3)])
    for bits in (1, 2, 4, 8):
        store = oc.sq_codes_to_storage(oc.sq_compress(x, cbs, bits, 16), bits)
        assert np.array_equal(oc.sq_decompress(store, cbs, bits, 16, 32),
                              oc.sq_decompress_per_byte_codebook(store, cbs, bits, 16, 32))


def test_sq_codebook_follows_the_torch_statement():
    # the statement of tests/test_sq.py:8-21, executed with torch on the same sample
    rng = np.random.default_rng(3)
    s = rng.uniform(-1, 1, size=(5000, 4)).astype(np.float32)
    cb = oc.sq_codebook(s)
    sample = torch.from_numpy(s).float().abs()
    fmin = max(np.percentile(sample.numpy(), 0.5), 1e-5)
    fmax = max(np.percentile(sample.numpy(), 99.5), 2e-5)
    fmin_t, fmax_t = torch.tensor(fmin), torch.tensor(fmax)
    emin, emax = torch.log2(fmin_t), torch.log2(fmax_t).add(1e-5)
    want = np.array([fmin_t.item(), fmax_t.item(), emin.item(), emax.item(), sample.mean().item()],
                    dtype=np.float32)
    assert cb[0] == want[0] and cb[1] == want[1]
    assert np.all(np.abs(cb[2:4] - want[2:4]) <= np.spacing(np.abs(want[2:4])))
    assert abs(cb[4] - want[4]) <= 4 * np.spacing(want[4])
    tiny = oc.sq_codebook(np.full((10, 2), 1e-7, dtype=np.float32))
    assert tiny[0] == np.float32(1e-5) and tiny[1] == np.float32(2e-5)
    assert tiny[4] == np.float32(np.float32(1e-7) + np.float32(0.1))


# ---- affine SQ ----------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_affine_closed_form(bits):
    rng = np.random.default_rng(bits)
    x = (rng.standard_normal((500, 11)) * 3).astype(np.float32)
    params = oc.sq_affine_params(x, bits)
    codes = oc.sq_affine_compress(x, params, bits)
    store = oc.packbits(codes, bits) if bits < 8 else codes
    dec = oc.sq_affine_decompress(store, params, bits, 11)
    # independent statement with python floats rounded through fp32 at each step
    for r, c in [(0, 0), (3, 10), (499, 5), (17, 7)]:
        prod = np.float32(np.float32(codes[r, c]) * params[1, c])
        assert dec[r, c] == np.float32(params[0, c] + prod)
    # endpoints decode to min and (up to rounding) max; error at most half a step
    assert np.all(np.abs(dec - x) <= params[1] * 0.5 * 1.0001 + 1e-6)
    assert np.array_equal(dec.min(axis=0), params[0])


def test_fused_multiply_add_reading_of_the_decode_differs_on_few_codes():
    # nvcc contracts `fabs(value) * k + emin` into one FMA by default; the torch statement the oracle
    # follows rounds the product first.  How many table entries the two readings disagree on, and by
    # how much: reported (and bounded) here, nothing else depends on the fma form.
    rng = np.random.default_rng(3)
    x = rng.uniform(-3, 3, size=(20000, 64)).astype(np.float32)
    cbs = np.stack([oc.sq_codebook(x[:, :32]), oc.sq_codebook(x[:, 32:] * 40),
                    np.array([0.01, 3.0, np.log2(0.01), np.log2(3.0) + 1e-5, 0.4], dtype=np.float32)])
    report = {}
    for bits in (2, 4, 8, 16):
        plain, fused = oc.sq_lut(cbs, bits), oc.sq_lut(cbs, bits, fma=True)
        differ = plain != fused
        report[bits] = (int(differ.sum()), plain.size)
        # the exponent moves by at most one fp32 rounding, so a differing entry is off by a few ulp of
        # the decoded value (the slope of exp2 times one rounding of an exponent of up to ~7 bits)
        rel = np.abs(plain.astype(np.float64) - fused.astype(np.float64)) / np.abs(plain.astype(np.float64))
        assert rel.max() < 2e-6, (bits, rel.max())
        assert differ.mean() < 0.5
    print("sq_lut entries that change under FMA contraction (differing, total):", report)
    assert report[2][0] <= report[2][1] and report[16][0] > 0      # the readings do differ somewhere at 16 bits
