"""Pins the CPU oracle (oracle/) before anything is compared with it.

The reference stores no golden vectors for this path (its tests recompute everything against
compute_ref), so the oracle is pinned by hand-derived vectors, by closed forms evaluated
independently in numpy, by special cases with known answers and by brute force on tiny inputs.
"""
import json
import os

import numpy as np
import pytest

from oracle import quantizer as Q

HERE = os.path.dirname(os.path.abspath(__file__))
COMBOS = [(2, 2), (3, 3), (4, 4), (5, 5), (6, 6), (7, 7), (8, 8), (4, 2), (6, 2), (8, 2), (8, 4), (8, 3)]


def rand_vals(rng, rows, k, bits, signed):
    lo, hi = (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if signed else (0, (1 << bits) - 1)
    return rng.integers(lo, hi + 1, size=(rows, k), dtype=np.int32)


# ------------------------------------------------------------------ packing

def test_pack_hand_vectors(oracle):
    cases = json.load(open(os.path.join(HERE, "golden", "pack_vectors.json")))["cases"]
    for c in cases:
        v = np.array(c["values"], dtype=np.int32).reshape(1, 32)
        got = oracle.pack_i32(v, c["bits"])
        want = np.array([int(h, 16) for h in c["planes_hex"]], dtype=np.uint32).reshape(c["bits"], 1, 1)
        assert np.array_equal(got, want), c["name"]
        assert np.array_equal(oracle.np_pack(v, c["bits"]), want), c["name"]


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8, 12, 16])
def test_pack_matches_closed_form_and_round_trips(oracle, bits):
    rng = np.random.default_rng(bits)
    for signed in (False, True):
        v = rand_vals(rng, 7, 256, bits, signed)
        planes = oracle.pack_i32(v, bits)
        assert planes.shape == (bits, 7, 8)
        assert np.array_equal(planes, oracle.np_pack(v, bits))
        assert np.array_equal(oracle.unpack(planes, signed), v)


def test_pack_planes_above_width_are_zero(oracle):
    rng = np.random.default_rng(0)
    v = rand_vals(rng, 3, 128, 3, False)
    planes = oracle.pack_i32(v, 8)
    assert not planes[3:].any() and planes[:3].any()


def nibble_pack(values):
    """8 four-bit elements per uint32, first element in the top nibble (pack.cu:26-40)."""
    v = (np.asarray(values).astype(np.int64) & 0xF).reshape(-1, 8)
    shifts = (4 * (7 - np.arange(8))).astype(np.int64)
    return (v << shifts).sum(axis=1).astype(np.uint32)


def test_pack_u4_equals_pack_i32_on_same_values(oracle):
    rng = np.random.default_rng(4)
    v = rand_vals(rng, 5, 128, 4, False)
    assert np.array_equal(oracle.pack_u4(nibble_pack(v), 5, 128, 4), oracle.pack_i32(v, 4))
    # hand vector: word 0 = 0xF0000001 -> first element 15, eighth element 1
    words = np.zeros(4, dtype=np.uint32)
    words[0] = 0xF0000001
    planes = oracle.pack_u4(words, 1, 32, 4)
    assert [int(x) for x in planes[:, 0, 0]] == [0x81000000, 0x80000000, 0x80000000, 0x80000000]


@pytest.mark.parametrize("scale", [1.0, 0.5, 3.0, 127.0 / 6.0, 1e-3, 100.0])
def test_pack_f16_all_bit_patterns(oracle, scale):
    """Every fp16 input against numpy float16 arithmetic: product rounded to fp16, then truncated."""
    bits_all = np.arange(65536, dtype=np.uint16)
    x = bits_all.view(np.float16)
    finite = np.isfinite(x)
    x = np.where(finite, x, np.float16(0)).astype(np.float16).reshape(512, 128)
    with np.errstate(over="ignore", invalid="ignore"):
        prod = (x * np.float16(scale)).astype(np.float16)  # numpy rounds the fp16 product once
    ok = np.isfinite(prod)
    want = np.where(ok, np.trunc(prod.astype(np.float64)), 0).astype(np.int64)
    planes = oracle.pack_f16(x, scale, 17)
    got = oracle.unpack(planes, True).astype(np.int64)
    assert np.array_equal(got[ok], want[ok])


def test_f16_conversions_match_numpy(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(1)
    f = np.concatenate([rng.normal(0, 1, 2000), rng.normal(0, 1e-6, 500), rng.normal(0, 3e4, 500),
                        [0.0, -0.0, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25]]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([L.abq_oracle_f32_to_f16(float(v)) for v in f], dtype=np.uint16)
    assert np.array_equal(got, want)
    hb = np.arange(0, 65536, 7, dtype=np.uint16)
    back = np.array([L.abq_oracle_f16_to_f32(int(h)) for h in hb], dtype=np.float32)
    ref = hb.view(np.float16).astype(np.float32)
    assert np.array_equal(np.isnan(back), np.isnan(ref))
    assert np.array_equal(back[~np.isnan(ref)], ref[~np.isnan(ref)])


# ------------------------------------------------------------------ GEMM

@pytest.mark.parametrize("q,p", COMBOS)
@pytest.mark.parametrize("signed", [True, False])
def test_three_gemms_agree_with_numpy(oracle, q, p, signed):
    rng = np.random.default_rng(100 * q + p + (7 if signed else 0))
    M, N, K = 5, 9, 256
    x, w = rand_vals(rng, M, K, q, signed), rand_vals(rng, N, K, p, signed)
    xp, wp = oracle.pack_i32(x, q), oracle.pack_i32(w, p)
    want = oracle.np_gemm(x, w)
    assert np.array_equal(oracle.gemm_bitserial(xp, wp, signed), want)
    assert np.array_equal(oracle.gemm_popc(xp, wp, signed)[0], want)
    assert np.array_equal(oracle.gemm_int(x, w), want)


def test_sign_rule_brute_force(oracle):
    """All value pairs for q, p <= 3 placed on distinct K positions."""
    for q in (1, 2, 3):
        for p in (1, 2, 3):
            for signed in (True, False):
                if signed and (q == 1 or p == 1):
                    continue
                xlo, xhi = oracle.value_range(q, signed)
                wlo, whi = oracle.value_range(p, signed)
                xv, wv = np.arange(xlo, xhi + 1), np.arange(wlo, whi + 1)
                K = 128
                x = np.zeros((len(xv), K), dtype=np.int32)
                w = np.zeros((len(wv), K), dtype=np.int32)
                x[:, 31] = xv  # bit 0 of the word: the position the reference extracts with 1<<31 ... >>31
                w[:, 31] = wv
                x[:, 0] = xv
                w[:, 0] = wv
                want = 2 * np.outer(xv, wv).astype(np.int32)
                got = oracle.gemm_bitserial(oracle.pack_i32(x, q), oracle.pack_i32(w, p), signed)
                assert np.array_equal(got, want), (q, p, signed)


def test_all_ones_planes_closed_form(oracle):
    """All planes all-ones: D = K * (sum_i s_i 2^i) * (sum_j s_j 2^j)."""
    K = 384
    for q, p in COMBOS:
        for signed in (True, False):
            xp = np.full((q, 2, K // 32), 0xFFFFFFFF, dtype=np.uint32)
            wp = np.full((p, 3, K // 32), 0xFFFFFFFF, dtype=np.uint32)
            sx = -1 if signed else (1 << q) - 1
            sw = -1 if signed else (1 << p) - 1
            for fn in (lambda: oracle.gemm_bitserial(xp, wp, signed), lambda: oracle.gemm_popc(xp, wp, signed)[0]):
                assert np.all(fn() == K * sx * sw)


def test_single_bit_gives_single_product(oracle):
    K = 128
    x = np.zeros((1, K), dtype=np.int32)
    w = np.zeros((1, K), dtype=np.int32)
    x[0, 77], w[0, 77] = -128, -2
    w[0, 3] = 1  # unmatched position contributes nothing
    d = oracle.gemm_popc(oracle.pack_i32(x, 8), oracle.pack_i32(w, 2), True)[0]
    assert d[0, 0] == 256
    assert oracle.gemm_bitserial(oracle.pack_i32(x, 8), oracle.pack_i32(w, 2), True)[0, 0] == 256


def test_configs0_shape_reduced(oracle):
    """BASELINE configs[0] (W4A4 unsigned, seed 0) at a reduced N so the bit-serial path runs in seconds."""
    rng = np.random.default_rng(0)
    M, N, K = 64, 96, 4096
    x, w = rand_vals(rng, M, K, 4, False), rand_vals(rng, N, K, 4, False)
    xp, wp = oracle.pack_i32(x, 4), oracle.pack_i32(w, 4)
    want = oracle.np_gemm(x, w)
    assert np.array_equal(oracle.gemm_bitserial(xp, wp, False), want)
    assert np.array_equal(oracle.gemm_popc(xp, wp, False)[0], want)


def test_int32_range_of_largest_baseline_case(oracle):
    # W8A8 unsigned, K = 13824: the largest |D| any configuration can produce
    assert 13824 * 255 * 255 < 2 ** 31


# ------------------------------------------------------------------ epilogue and scales

def test_epilogue_f16_matches_numpy(oracle):
    rng = np.random.default_rng(5)
    acc = np.concatenate([rng.integers(-70000, 70000, 4000), rng.integers(-3000, 3000, 4000),
                          [0, 1, -1, 2047, 2049, 65504, 65519, 65520, -65520, 1 << 24, (1 << 24) + 1]]).astype(np.int32)
    for scale in (np.float16(0.0123), np.float16(1.0), np.float16(7.5e-4)):
        got = oracle.epilogue_f16(acc, scale)
        with np.errstate(over="ignore", invalid="ignore"):
            want = acc.astype(np.float64).astype(np.float16) * scale  # int -> fp16 rounds once from exact
        assert np.array_equal(got.view(np.uint16), want.astype(np.float16).view(np.uint16))


def test_quantizer_closed_forms():
    rng = np.random.default_rng(9)
    x = rng.normal(0, 1, (6, 256))
    # symmetric, no zero point: max |x| of a row maps to +/- qmax, error <= scale / 2
    qp = Q.QuantParams(8, symmetric=True, disable_zero_point=True)
    scale, zp = Q.calibrate(x, qp)
    assert zp is None and scale.shape == (6, 1)
    xi = Q.quantize(x, qp, scale, zp)
    assert np.all(np.abs(xi).max(axis=1) == 127)
    assert np.all(np.abs(Q.dequantize(xi, qp, scale, zp) - x) <= scale / 2 + 1e-12)
    # asymmetric with zero point: row min -> qmin, row max -> qmax
    qp = Q.QuantParams(4)
    scale, zp = Q.calibrate(x, qp)
    xi = Q.quantize(x, qp, scale, zp)
    assert np.all(xi.min(axis=1) == 0) and np.all(xi.max(axis=1) == 15)
    # grouped: one scale per (row, group)
    qp = Q.QuantParams(2, symmetric=True, disable_zero_point=True, group_size=128)
    scale, zp = Q.calibrate(x, qp)
    assert scale.shape == (12, 1)
    xi = Q.quantize(x, qp, scale, zp)
    assert xi.min() >= -2 and xi.max() <= 1
    # exactly representable rows quantize to themselves
    qp = Q.QuantParams(8, symmetric=True, disable_zero_point=True)
    ints = rng.integers(-127, 128, (3, 64)).astype(np.float64)
    ints[:, 0] = 127
    assert np.allclose(Q.fake_quant(ints * 0.25, qp), ints * 0.25)
    # two-bit "bit balance": asymmetric 2-bit range is widened to five levels (quantizer.py:66-68)
    qp = Q.QuantParams(2)
    assert (qp.qmin, qp.qmax) == (0, 4)


def test_per_token_codes_f32_agrees_with_the_fp64_restatement():
    rng = np.random.default_rng(21)
    x = rng.normal(0, 1, (8, 512)).astype(np.float16)
    # symmetric: same codes as calibrate/quantize in fp64 except where x/scale sits on a rounding tie
    codes, scale, zero = Q.per_token_codes_f32(x, 8, True)
    qp = Q.QuantParams(8, symmetric=True, disable_zero_point=True)
    s64, _ = Q.calibrate(x, qp)
    c64 = Q.quantize(x, qp, s64, None)
    assert np.allclose(scale, s64[:, 0], rtol=1e-6) and not zero.any()
    assert np.abs(codes - c64).max() <= 1 and (codes != c64).mean() < 1e-3
    assert np.all(np.abs(codes).max(axis=1) == 127)
    # asymmetric: unsigned code = code + 2^(n-1), zero point = zero + 2^(n-1)
    for bits in (8, 4):
        codes, scale, zero = Q.per_token_codes_f32(x, bits, False)
        qp = Q.QuantParams(bits)
        s64, z64 = Q.calibrate(x, qp)
        c64 = Q.quantize(x, qp, s64, z64)
        half = 1 << (bits - 1)
        assert np.allclose(scale, s64[:, 0], rtol=1e-6)
        assert np.array_equal(zero + half, z64[:, 0])
        assert np.abs(codes + half - c64).max() <= 1 and (codes + half != c64).mean() < 2e-3
        assert (codes + half).min() == 0 and (codes + half).max() == 2 * half - 1
        # dequantisation error at most scale / 2 inside the clamp range
        deq = (codes - zero[:, None]) * scale[:, None]
        assert np.all(np.abs(deq - x.astype(np.float32)) <= scale[:, None] * 0.5001)


def test_group_affine_codes_and_dequant_matmul():
    rng = np.random.default_rng(22)
    w = rng.normal(0, 0.02, (12, 256))
    codes, scale, zero = Q.group_affine_codes(w, 2, 128)
    assert codes.shape == (12, 256) and scale.shape == (12, 2) and zero.shape == (12, 2)
    assert codes.min() == -2 and codes.max() == 1
    # every group's min and max land on the ends of the code range
    g = codes.reshape(12, 2, 128)
    assert np.all(g.min(axis=2) == -2) and np.all(g.max(axis=2) == 1)
    # same codes as the general restatement with a 4-level range (bit balance switched off)
    qp = Q.QuantParams(2, group_size=128)
    qp.qmax = 3
    s = np.clip((w.reshape(-1, 128).max(1) - w.reshape(-1, 128).min(1)) / 3, Q.CLIPMIN, 1e4)[:, None]
    z = np.round(-w.reshape(-1, 128).min(1)[:, None] / s)
    assert np.array_equal(Q.quantize(w, qp, s, z), codes + 2)
    # dequant_matmul against an element-by-element loop
    xc = rng.integers(-128, 128, (3, 256)).astype(np.int32)
    xs, xz = rng.uniform(0.01, 0.1, 3), rng.integers(-5, 5, 3).astype(np.float64)
    got = Q.dequant_matmul(xc, xs, xz, codes, scale, zero, 128)
    want = np.zeros((3, 12))
    for m in range(3):
        for n in range(12):
            for k in range(256):
                want[m, n] += (xc[m, k] - xz[m]) * xs[m] * (codes[n, k] - zero[n, k // 128]) * scale[n, k // 128]
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)


def test_quantizer_bit_balance_closed_forms():
    """quantizer.py:66-68,169-171: asymmetric 1- and 2-bit ranges are widened by one level.  A row holding the
    exact multiples 0, s, 2s, 3s, 4s of a step s is quantised to 0..4 with scale s and dequantises to itself; with
    the plain range (3 bits) the same row would use scale 4s/7."""
    from oracle import quantizer as Q
    s = 0.125
    x = np.array([[0.0, s, 2 * s, 3 * s, 4 * s, 2 * s, s, 4 * s]])
    qp = Q.QuantParams(2)
    assert (qp.qmin, qp.qmax) == (0, 4)
    scale, zp = Q.calibrate(x, qp)
    assert scale[0, 0] == s and zp[0, 0] == 0
    assert np.array_equal(Q.quantize(x, qp, scale, zp), np.array([[0, 1, 2, 3, 4, 2, 1, 4]], dtype=np.float64))
    assert np.array_equal(Q.fake_quant(x, qp), x)
    assert Q.QuantParams(1).qmax == 2 and Q.QuantParams(3).qmax == 7 and Q.QuantParams(2, disable_zero_point=True).qmax == 1
    # shifted row: the zero point takes the offset, the codes stay
    scale, zp = Q.calibrate(x - 2 * s, qp)
    assert scale[0, 0] == s and zp[0, 0] == 2
    assert np.array_equal(Q.quantize(x - 2 * s, qp, scale, zp), np.array([[0, 1, 2, 3, 4, 2, 1, 4]], dtype=np.float64))
    codes, sc, zero, bits = Q.group_affine_codes_bit_balance(np.tile(x - 2 * s, (2, 16)), 2, 64)
    assert bits == 3 and codes.min() == -4 and codes.max() == 0 and np.all(sc == s) and np.all(zero == 2 - 4)
    # x ~ scale * (code - zero) reproduces the row
    assert np.array_equal((codes - np.repeat(zero, 64, axis=1)) * np.repeat(sc, 64, axis=1), np.tile(x - 2 * s, (2, 16)))


def test_quantizer_pads_rows_to_whole_groups():
    """quantizer.py:82-91,112-118,151-156: a row whose length is no multiple of the group size is padded with zeros
    (symmetric quantisation only); the padded group's scale comes from its real elements and the padding is cut off."""
    from oracle import quantizer as Q
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, (3, 100))
    qp = Q.QuantParams(4, symmetric=True, disable_zero_point=True, group_size=64)
    scale, zp = Q.calibrate(x, qp)
    assert zp is None and scale.shape == (6, 1)
    want = np.stack([np.abs(x[:, :64]).max(axis=1), np.abs(x[:, 64:]).max(axis=1)], axis=1).reshape(-1, 1) / 7
    assert np.allclose(scale, want, rtol=0, atol=0)
    q = Q.quantize(x, qp, scale, zp)
    assert q.shape == x.shape and np.array_equal(q[:, :64], np.clip(np.round(x[:, :64] / scale[0::2]), -8, 7))
    assert np.array_equal(q[:, 64:], np.clip(np.round(x[:, 64:] / scale[1::2]), -8, 7))
    assert Q.fake_quant(x, qp).shape == x.shape
    with pytest.raises(AssertionError):
        Q.calibrate(x, Q.QuantParams(4, symmetric=False, group_size=64))
