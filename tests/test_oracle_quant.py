"""Pins the oracle's conversions, quantizer and blob layout against the
reference's own test expectations and against brute force."""
import numpy as np

import oracle as O


def test_bf16_round_to_nearest_even_and_roundtrip():
    # Quantization.swift:17-23 is RNE on the top 16 bits.
    cases = {1.0: 0x3F80, -1.0: 0xBF80, 0.5: 0x3F00, 0.0: 0x0000}
    for v, bits in cases.items():
        assert O.lib.orc_bf16_bits(v) == bits
    # exact ties: 1 + 2^-8 is halfway between 0x3F80 and 0x3F81 -> even (0x3F80);
    # 1 + 3*2^-8 is halfway between 0x3F81 and 0x3F82 -> even (0x3F82).
    assert O.lib.orc_bf16_bits(1.0 + 2.0 ** -8) == 0x3F80
    assert O.lib.orc_bf16_bits(1.0 + 3 * 2.0 ** -8) == 0x3F82
    # QuantizationAffineTests.swift:47-58: relative error <= 2^-7
    for v in [0.0, 1.0, -1.0, 0.5, -0.5, 1.0 / 3.0, 12345.0]:
        back = O.lib.orc_bf16_to_float(O.lib.orc_bf16_bits(v))
        assert abs(back - v) / max(abs(v), 1e-6) < 8e-3
    # the vectorised numpy twin used by the tests agrees with the C function
    r = np.random.default_rng(0).standard_normal(4096).astype(np.float32)
    c = np.array([O.lib.orc_bf16_bits(float(x)) for x in r], np.uint16)
    assert np.array_equal(O.bf16_bits(r), c)


def test_f16_conversion_matches_numpy_everywhere_it_matters():
    r = np.random.default_rng(1)
    vals = np.concatenate([
        r.standard_normal(20000).astype(np.float32),
        (r.standard_normal(20000) * 1e-5).astype(np.float32),   # subnormal range
        (r.standard_normal(2000) * 3e4).astype(np.float32),     # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8,
                  2.9802322e-8, 8.9406967e-8, np.inf, -np.inf], np.float32)])
    ours = np.array([O.lib.orc_f16_bits(float(v)) for v in vals], np.uint16)
    with np.errstate(over="ignore"):
        ref = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(ours, ref)
    back = np.array([O.lib.orc_f16_to_float(int(b)) for b in ours], np.float32)
    assert np.array_equal(back, ref.view(np.float16).astype(np.float32))


def test_splitmix64_and_seedtree_known_values():
    # SplitMix64 with seed 0: first outputs of the published reference generator.
    g = O.SplitMix64(0)
    assert [g.next() for _ in range(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4,
                                           0x06C45D188009454F]
    # FNV-1a 64 of "a" is 0xAF63DC4C8601EC8C (published test vector)
    assert O.lib.orc_seedtree_key(0, b"a") == 0xAF63DC4C8601EC8C
    assert O.lib.orc_seedtree_key(0, b"") == 0xCBF29CE484222325


def test_quantizer_reference_property_tests():
    # QuantizationAffineTests.swift:8-29
    row = np.concatenate([0.10 + np.arange(64, dtype=np.float32) * np.float32(0.01),
                          -0.50 - np.arange(64, dtype=np.float32) * np.float32(0.005)])
    p, s, b = O.quantize_affine(row, 4)
    assert p.shape == (1, 64) and s.shape == (1, 2) and b.shape == (1, 2)
    assert np.abs(O.dequantize_affine(p, s, b, 128, 4)[0] - row).max() < 0.025
    # :31-46
    row8 = (-0.3 + np.arange(64, dtype=np.float32) * np.float32(0.02)).astype(np.float32)
    p, s, b = O.quantize_affine(row8, 8)
    assert np.abs(O.dequantize_affine(p, s, b, 64, 8)[0] - row8).max() < 0.008
    # :61-72 flat group reproduces bf16(v) exactly with scale 1
    flat = np.full(64, 0.42, np.float32)
    p, s, b = O.quantize_affine(flat, 4)
    assert s[0, 0] == 0x3F80 and not p.any()
    assert np.array_equal(O.dequantize_affine(p, s, b, 64, 4)[0], O.round_bf16(flat))
    # :76-88 positive-only range uses codes 0 and 15
    pos = (np.arange(64, dtype=np.float32) / np.float32(63.0) + np.float32(1.0))
    codes = O.unpack_codes(O.quantize_affine(pos, 4)[0], 4)
    assert codes.min() == 0 and codes.max() == 15


def test_nibble_order_low_is_even():
    # QuantizationTests.swift:35-50 plus the exact layout statement of
    # nvmai_kernels.h:13 (element 2k in the low half of byte k).
    row = np.arange(64, dtype=np.float32) - np.float32(31.5)
    p, s, b = O.quantize_affine(row, 4)
    scale, bias = O.bf16_to_float(s)[0, 0], O.bf16_to_float(b)[0, 0]
    lo, hi = int(p[0, 0] & 0x0F), int(p[0, 0] >> 4)
    assert abs(lo * scale + bias - row[0]) <= scale + 1e-3
    assert abs(hi * scale + bias - row[1]) <= scale + 1e-3
    codes = O.unpack_codes(p, 4)
    assert np.array_equal(codes[0::2], p[0] & 0x0F) and np.array_equal(codes[1::2], p[0] >> 4)
    # monotone input -> monotone codes, so even/odd cannot be swapped unnoticed
    assert np.all(np.diff(codes.astype(int)) >= 0) and codes[0] == 0 and codes[-1] == 15


def _brute_force_codes(w, scales, biases, bits):
    """Independent restatement in vectorised float32 numpy: nearest code with
    exact halves going away from zero (numpy's rint is half-to-even, so the
    halves are handled separately)."""
    levels = (1 << bits) - 1
    s = O.bf16_to_float(scales).repeat(64, axis=1)
    b = O.bf16_to_float(biases).repeat(64, axis=1)
    inv = np.where(s == 0, np.float32(0), np.float32(1.0) / s).astype(np.float32)
    t = ((w - b).astype(np.float32) * inv).astype(np.float32)
    frac = t - np.trunc(t)
    r = np.where(np.abs(frac) == 0.5, np.trunc(t) + np.sign(t), np.rint(t))
    return np.clip(r, 0, levels).astype(np.uint8)


def test_quantizer_matches_brute_force_and_error_bound():
    # DequantInt4GEMVReferenceTests.swift:59-76 / Int8 :48-65: error <= one step
    for bits in (4, 8):
        for n in (128, 256, 2816):
            label = ("int4" if bits == 4 else "int8") + "-affine-roundtrip-n%d" % n
            g = O.seed_tree(0xF5, label)
            row = g.uniform_array(n, -1.0, 1.0)[None, :]
            p, s, b = O.quantize_affine(row, bits)
            rec = O.dequantize_affine(p, s, b, n, bits)
            step = O.bf16_to_float(s).repeat(64, axis=1)
            assert np.all(np.abs(rec - row) <= step + 1e-4)
            codes = O.unpack_codes(p, bits).reshape(1, n)
            assert np.array_equal(codes, _brute_force_codes(row, s, b, bits))
    # gaussian weights of the benchmark shape, many rows
    w = (np.random.default_rng(3).standard_normal((64, 2048)) * 0.02).astype(np.float32)
    w = O.round_bf16(w)
    for bits in (4, 8):
        p, s, b = O.quantize_affine(w, bits)
        assert np.array_equal(O.unpack_codes(p, bits).reshape(w.shape),
                              _brute_force_codes(w, s, b, bits))
        # scale/bias are bf16 of (max-min)/levels and min
        wg = w.reshape(64, 32, 64)
        lv = np.float32((1 << bits) - 1)
        assert np.array_equal(s, O.bf16_bits((wg.max(2) - wg.min(2)) / lv))
        assert np.array_equal(b, O.bf16_bits(wg.min(2)))


def _assert_codes_are_argmin(w, codes, scale, bias, levels, what):
    """The property itself, in float64 and without any rounding rule: the chosen code is at least as
    close to the value as both neighbouring codes (|w - (q s + b)| <= |w - ((q +- 1) s + b)|), except
    within a hair of an exact tie, where the fp32 product decides.  Clamped ends only have one
    neighbour inside the range.  A quantizer that truncates, rounds the wrong way, is off by one
    code or swaps scale and bias fails this for most elements."""
    w, s, b, q = (np.asarray(a, np.float64) for a in (w, scale, bias, codes))
    err = np.abs(w - (q * s + b))
    tol = 1e-4 * np.abs(s) + 1e-12
    up_ok = (q >= levels) | (err <= np.abs(w - ((q + 1) * s + b)) + tol)
    down_ok = (q <= 0) | (err <= np.abs(w - ((q - 1) * s + b)) + tol)
    bad = ~(up_ok & down_ok) & (s > 0)
    assert not bad.any(), "%s: %d codes are not the nearest" % (what, int(bad.sum()))
    # and values outside the representable range sit on the clamped end
    assert np.all(q[(w < b) & (s > 0)] == 0) and np.all(q[(w > levels * s + b) & (s > 0)] == levels)


def test_quantizer_codes_are_the_nearest_codes():
    # argmin over codes against the STORED (bf16) scale and bias: that is what makes the packed
    # codes the reference's (Quantization.swift:80-99 quantizes against the rounded pair)
    rng = np.random.default_rng(17)
    for bits in (4, 8):
        levels = (1 << bits) - 1
        for w in (O.round_bf16((rng.standard_normal((48, 2048)) * 0.02).astype(np.float32)),
                  rng.uniform(-1, 1, (16, 512)).astype(np.float32),
                  (rng.standard_normal((8, 256)) * 30 + 100).astype(np.float32)):      # positive-only groups
            p, s, b = O.quantize_affine(w, bits)
            codes = O.unpack_codes(p, bits).reshape(w.shape)
            _assert_codes_are_argmin(w, codes, O.bf16_to_float(s).repeat(64, axis=1),
                                     O.bf16_to_float(b).repeat(64, axis=1), levels, "weights %d bit" % bits)


def test_expert_offsets_known_answers():
    # CPUExpertFFNTests.swift:56-67
    o = O.expert_offsets(2048, 512, 4)
    assert int(o[9]) == 1_769_472
    assert [int(o[0]), int(o[1]), int(o[3]), int(o[6])] == [0, 524_288, 589_824, 1_179_648]
    assert list(o[:9]) == sorted(o[:9])
    assert list(map(int, o)) == [0, 524288, 557056, 589824, 1114112, 1146880, 1179648,
                                 1703936, 1736704, 1769472]
    # RuntimeConfiguration.swift:195-197: the 8-bit expert stride
    assert int(O.expert_offsets(2048, 512, 8)[9]) == 3_342_336
