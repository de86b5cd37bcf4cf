"""Pins the oracle's RMSNorm, embedding lookup and greedy LM head against the known answers the
reference's own tests hold and against float64 recomputation."""
import numpy as np

import oracle as O


def _bitstream_table(bits, rows, cols):
    # AffineQuantTests.swift:7-32: value = (row*11 + col*3) & mask packed as a bit stream
    mask = (1 << bits) - 1
    values = np.array([[(r * 11 + c * 3) & mask for c in range(cols)] for r in range(rows)], np.uint32)
    packed = np.zeros((rows, cols * bits // 8), np.uint8)
    for r in range(rows):
        for c in range(cols):
            packed[r, c * bits // 8] |= (int(values[r, c]) << ((c * bits) % 8)) & 0xFF
    return packed, values


# ------------------------------------------------------------------ RMSNorm
def test_rmsnorm_matches_float64_recomputation():
    # RMSNormReferenceTests.swift:26-44: d in {256, 512, 2816}, x ~ U(-1,1), w ~ U(0.5,1.5), eps 1e-6
    for d, seed in [(256, 0xA1), (512, 0xB2), (2816, 0xC3), (100, 7)]:
        rng = np.random.default_rng(seed)
        x = rng.uniform(-1, 1, (3, d)).astype(np.float32)
        w = O.round_bf16(rng.uniform(0.5, 1.5, d).astype(np.float32))
        got = O.rmsnorm(x, O.bf16_bits(w), 1e-6)
        x64 = x.astype(np.float64)
        inv = 1.0 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-6)
        want = x64 * inv * w.astype(np.float64)
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-6
        # no weight == unit weight (rmsnorm.metal:152-175)
        unit = O.bf16_bits(np.ones(d, np.float32))
        assert np.array_equal(O.rmsnorm(x, None, 1e-6), O.rmsnorm(x, unit, 1e-6))


def test_rmsnorm_constant_heads_known_answer_and_isolation():
    # RMSNormTests.swift:119-165: head h is the constant h+1, unit weights -> every output is 1
    heads, hd = 16, 256
    x = np.repeat(np.arange(1, heads + 1, dtype=np.float32)[:, None], hd, axis=1)
    y = O.rmsnorm(x, O.bf16_bits(np.ones(hd, np.float32)), 1e-6)
    assert np.abs(y - 1.0).max() < 1e-2
    assert np.abs(y - 1.0).max() < 1e-5          # what the formula gives: c / sqrt(c^2 + 1e-6)
    # a row depends on nothing but itself
    x2 = x.copy()
    x2[5] = -3.0
    y2 = O.rmsnorm(x2, None, 1e-6)
    assert np.array_equal(np.delete(y2, 5, 0), np.delete(O.rmsnorm(x, None, 1e-6), 5, 0))
    assert np.abs(y2[5] + 1.0).max() < 1e-5      # sign preserved
    # zeros stay finite (RMSNormReferenceTests.swift:46-52: small magnitudes)
    assert np.isfinite(O.rmsnorm(np.zeros((1, 64), np.float32), None, 1e-6)).all()
    small = np.array([[1e-4, -1e-4, 2e-4, -2e-4, 1e-4, -1e-4, 2e-4, -2e-4]], np.float32)
    assert np.isfinite(O.rmsnorm(small, None, 1e-6)).all()


# ------------------------------------------------------------------ embedding lookup
def test_embed_lookup_bitstream_known_answer():
    # AffineQuantTests.swift:58-79: scale 1, bias 0, token 1 -> the packed values exactly
    for bits in (4, 8):
        rows, cols = 3, 128
        packed, values = _bitstream_table(bits, rows, cols)
        one = np.full((rows, cols // 64), 0x3F80, np.uint16)
        zero = np.zeros((rows, cols // 64), np.uint16)
        for tok in range(rows):
            assert np.array_equal(O.embed_lookup(packed, one, zero, bits, tok), values[tok].astype(np.float32))
        # dequant_int4.metal:77-80: a token id at or past vocab gives zeros
        assert not O.embed_lookup(packed, one, zero, bits, rows).any()
        assert not O.embed_lookup(packed, one, zero, bits, 0xFFFFFFFF).any()


def test_embed_lookup_equals_dequantizer_times_scale():
    rng = np.random.default_rng(3)
    for bits in (4, 8):
        w = (rng.standard_normal((9, 192)) * 0.05).astype(np.float32)
        p, s, b = O.quantize_affine(w, bits)
        deq = O.dequantize_affine(p, s, b, 192, bits).reshape(9, 192)
        for tok in (0, 4, 8):
            assert np.array_equal(O.embed_lookup(p, s, b, bits, tok), deq[tok])
            assert np.array_equal(O.embed_lookup(p, s, b, bits, tok, 45.25), deq[tok] * np.float32(45.25))


# ------------------------------------------------------------------ greedy LM head
def _const_rows(v, d, special, hi, lo, bits=4):
    w = np.full((v, d), lo, np.float32)
    for r in special:
        w[r] = hi
    return O.quantize_affine(w, bits)


def test_greedy_head_reference_known_answers():
    d = 64
    unit = O.bf16_bits(np.ones(d, np.float32))
    # LMHeadChainInt4Tests.swift:153-175: the one row of ones wins, at v - 3
    hidden = O.f16_to_float(O.f16_bits((0.25 + (np.arange(d) % 7) * 0.01).astype(np.float32)))
    for v in (1024, 2048, 4096):
        p, s, b = _const_rows(v, d, [v - 3], 1.0, -0.5)
        assert O.lm_head_greedy(hidden, unit, p, s, b, 4, act=1) == v - 3
    # :177-193: equal rows 17 and 311 -> the lower index
    hidden = O.f16_to_float(O.f16_bits((0.2 + (np.arange(d) % 5) * 0.02).astype(np.float32)))
    p, s, b = _const_rows(1024, d, [17, 311], 1.0, -0.25)
    assert O.lm_head_greedy(hidden, unit, p, s, b, 4, act=1) == 17
    # :136-151: NaN hidden -> no finite logit -> token 0
    p, s, b = _const_rows(1024, d, [], 0.25, 0.25)
    assert O.lm_head_greedy(np.full(d, np.nan, np.float32), unit, p, s, b, 4, act=1) == 0


def test_greedy_head_matches_float64_argmax_on_separated_rows():
    rng = np.random.default_rng(21)
    for bits, d, v in [(4, 256, 700), (8, 192, 300), (8, 2048, 64)]:
        w = (rng.standard_normal((v, d)) * 0.02).astype(np.float32)
        target = int(rng.integers(v))
        hidden = O.round_bf16(rng.standard_normal(d).astype(np.float32))
        w[target] += 0.05 * np.sign(hidden)            # a clear winner
        p, s, b = O.quantize_affine(w, bits)
        nw = O.bf16_bits(O.round_bf16(rng.uniform(0.5, 1.5, d).astype(np.float32)))
        tok, logits = O.lm_head_greedy(hidden, nw, p, s, b, bits, act=0, want_logits=True)
        xn = O.round_bf16(O.rmsnorm(hidden[None], nw, 1e-6)[0]).astype(np.float64)
        deq = O.dequantize_affine(p, s, b, d, bits).reshape(v, d).astype(np.float64)
        want = deq @ xn
        assert tok == int(np.argmax(want)) == target
        assert np.abs(logits - want).max() / np.abs(want).max() < 1e-5
        # without a norm weight the hidden row is used as it is
        tok2, logits2 = O.lm_head_greedy(hidden, None, p, s, b, bits, act=0, want_logits=True)
        want2 = deq @ hidden.astype(np.float64)
        assert tok2 == int(np.argmax(want2))
        assert np.abs(logits2 - want2).max() / np.abs(want2).max() < 1e-5


# ------------------------------------------------------------------ elementwise helpers
def test_elementwise_special_values_and_float64():
    # the reference holds no test for utility.metal's helpers: what the mathematics fixes
    z = np.zeros(4, np.float32)
    one = np.ones(4, np.float32)
    assert np.array_equal(O.elementwise(O.EW_SILU_MUL, z, one), z)                         # silu(0) = 0
    assert np.array_equal(O.elementwise(O.EW_SIGMOID_MUL, one, z), one * np.float32(0.5))  # sigmoid(0) = 1/2
    big = np.full(4, 40.0, np.float32)
    assert np.array_equal(O.elementwise(O.EW_SIGMOID_MUL, one, big), one)                  # saturates to 1
    assert np.abs(O.elementwise(O.EW_SIGMOID_MUL, one, -big)).max() < 1e-15                # and to 0
    assert np.array_equal(O.elementwise(O.EW_SILU_MUL, big, one), big)                     # silu(x) -> x
    rng = np.random.default_rng(8)
    a = (rng.standard_normal(4096) * 3).astype(np.float32)
    b = (rng.standard_normal(4096) * 3).astype(np.float32)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    for op, want in [(O.EW_SILU_MUL, a64 / (1 + np.exp(-a64)) * b64), (O.EW_SIGMOID_MUL, a64 / (1 + np.exp(-b64))),
                     (O.EW_SIGMOID_SCALAR, a64 / (1 + np.exp(-b64[0]))), (O.EW_ADD, a64 + b64)]:
        got = O.elementwise(op, a, b)
        assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
    assert np.array_equal(O.elementwise(O.EW_ADD, a, b), a + b)                            # one IEEE addition
    # sigmoid(-g) = 1 - sigmoid(g)
    s_pos = O.elementwise(O.EW_SIGMOID_MUL, np.ones_like(b), b)
    s_neg = O.elementwise(O.EW_SIGMOID_MUL, np.ones_like(b), -b)
    assert np.abs(s_pos + s_neg - 1.0).max() < 1e-6


def test_split_and_concat_are_inverse_layouts():
    heads, dim = 5, 12
    packed = np.arange(heads * 2 * dim, dtype=np.float32).reshape(heads, 2 * dim)
    q, g = O.split_q_gate(packed, heads, dim)
    assert q[2, 3] == packed[2, 3] and g[2, 3] == packed[2, dim + 3]          # utility.metal:90-91
    assert np.array_equal(O.concat_rows(q, g), packed)
