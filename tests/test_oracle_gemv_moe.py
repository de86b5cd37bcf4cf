"""Pins the oracle's GEMV, expert FFN, router and MoE layer."""
import math

import numpy as np
import pytest

import oracle as O


def _lcg_rows(count, n, seed):
    """CPUExpertFFNTests.swift:16-27: rows quantized from the test's own LCG."""
    g = O.Lcg(seed)
    return np.stack([g.array(n) for _ in range(count)])


def test_int4_gemv_bit_exact_against_reference_c_kernel():
    ref = O.load_reference_gemv()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(7)
    for rows, n in [(64, 128), (512, 2048), (2048, 512), (3, 64), (1, 2816)]:
        w = rng.standard_normal((rows, n)).astype(np.float32) * np.float32(0.02)
        p, s, b = O.quantize_affine(w, 4)
        x = rng.standard_normal(n).astype(np.float32)
        ours = O.affine_gemv(p, s, b, x, 4)
        theirs = np.zeros(rows, np.float32)
        ref(p, s, b, x, rows, n, theirs)
        assert np.array_equal(ours.view(np.uint32), theirs.view(np.uint32))


def test_gemv_bitstream_known_answer():
    # AffineQuantTests.swift:7-56: value = (row*11 + col*3) & mask, scale 1,
    # bias 0, x = 1  =>  y[row] = sum(values)   (exact in fp32 at this size)
    for bits in (4, 8):
        rows, cols = 3, 128
        mask = (1 << bits) - 1
        values = np.array([[(r * 11 + c * 3) & mask for c in range(cols)] for r in range(rows)])
        packed = np.zeros((rows, cols * bits // 8), np.uint8)
        for r in range(rows):
            for c in range(cols):                       # the test's own bit-stream packing
                bit = c * bits
                packed[r, bit // 8] |= (int(values[r, c]) << (bit % 8)) & 0xFF
        one = np.full((rows, cols // 64), 0x3F80, np.uint16)
        zero = np.zeros_like(one)
        y = O.affine_gemv(packed, one, zero, np.ones(cols, np.float32), bits)
        assert np.array_equal(y, values.sum(1).astype(np.float32))
        assert np.array_equal(O.unpack_codes(packed, bits).reshape(rows, cols), values)
        assert np.array_equal(O.dequantize_affine(packed, one, zero, cols, bits), values)


def test_factored_gemv_matches_unfactored_and_float64():
    rng = np.random.default_rng(11)
    for bits in (4, 8):
        w = rng.standard_normal((96, 1024)).astype(np.float32) * np.float32(0.05)
        p, s, b = O.quantize_affine(w, bits)
        x = rng.standard_normal(1024).astype(np.float32)
        fact = O.affine_gemv(p, s, b, x, bits)
        unf = O.affine_gemv(p, s, b, x, bits, unfactored=True)
        dense = O.dequantize_affine(p, s, b, 1024, bits).astype(np.float64) @ x.astype(np.float64)
        assert O.rel_error(fact, dense) < 2e-5
        assert O.rel_error(unf, dense) < 2e-5


def test_expert_ffn_matches_reference_test_setup():
    # CPUExpertFFNTests.swift:69-113 (d=128, f=64, seeds 1,2,3, x from seed 99 inc 1)
    d, f = 128, 64
    gate, up, down = _lcg_rows(f, d, 1), _lcg_rows(f, d, 2), _lcg_rows(d, f, 3)
    blob = O.pack_expert(gate, up, down, 4)
    x = O.Lcg(99, inc=1).array(d)
    out = O.expert_ffn_accumulate(blob, 4, x, d, f, 1.0, np.zeros(d, np.float32))
    # independent float64 restatement from the decoded rows
    deq = lambda m, n: O.dequantize_affine(*O.quantize_affine(m, 4), n, 4).astype(np.float64)
    g = deq(gate, d) @ x
    u = deq(up, d) @ x
    act = g / (1 + np.exp(-g)) * u
    expected = deq(down, f) @ act
    scale = max(np.abs(expected).max(), 1)
    assert np.abs(out - expected).max() <= 2e-4 * scale
    # :117-152 accumulate linearity 0.75 + 0.25 == 1.0
    blob2 = O.pack_expert(_lcg_rows(f, d, 7), _lcg_rows(f, d, 8), _lcg_rows(d, f, 9), 4)
    x2 = np.full(d, 0.05, np.float32)
    once = O.expert_ffn_accumulate(blob2, 4, x2, d, f, 1.0, np.zeros(d, np.float32))
    twice = np.zeros(d, np.float32)
    O.expert_ffn_accumulate(blob2, 4, x2, d, f, 0.75, twice)
    O.expert_ffn_accumulate(blob2, 4, x2, d, f, 0.25, twice)
    assert np.abs(once - twice).max() <= 1e-4 * max(np.abs(once).max(), 1)


def _constant_blob(d, f, bits):
    """MoEFusedFFNTests.swift:238-270: all codes 0, scales 0, biases 1/64, .5/64, 1/64."""
    off = O.expert_offsets(d, f, bits)
    blob = np.zeros(int(off[9]), np.uint8)
    bf = lambda v: int(np.float32(v).view(np.uint32)) >> 16

    def fill(o, count, v):
        blob[o:o + 2 * count].view(np.uint16)[:] = bf(v)
    fill(int(off[2]), f * d // 64, 1.0 / 64)
    fill(int(off[5]), f * d // 64, 0.5 / 64)
    fill(int(off[8]), d * f // 64, 1.0 / 64)
    return blob


def test_moe_layer_constant_blob_known_answer():
    # MoEFusedFFNTests.swift:17-54: x = 1, 8 experts x weight 0.125 => silu(2)
    d, f = 128, 64
    expected = 2.0 / (1.0 + math.exp(-2.0))
    for bits in (4, 8):
        blob = _constant_blob(d, f, bits)
        y = np.zeros(d, np.float32)
        for _ in range(8):
            O.expert_ffn_accumulate(blob, bits, np.ones(d, np.float32), d, f, 0.125, y)
        assert np.abs(y - expected).max() < 1e-5


def _router_reference(weights, hidden, eff, expert_scale, k=8):
    """RouterTopKTests.swift:72-97 restated in float64."""
    scaled = (hidden * eff).astype(np.float32)
    p, s, b = O.quantize_affine(weights, 8)
    logits = O.dequantize_affine(p, s, b, weights.shape[1], 8).astype(np.float64) @ scaled
    order = sorted(range(len(logits)), key=lambda e: (-logits[e], e))[:k]
    ex = np.exp(logits[order] - logits[order[0]])
    return np.array(order, np.uint32), ex / ex.sum() * expert_scale[order], (p, s, b)


def test_router_matches_reference_tests():
    E, D = 16, 128
    # productionRouterMatchesReference (RouterTopKTests.swift:19-44)
    g = O.SplitMix64(0xA5B61234)
    weights = np.stack([g.uniform_array(D, -0.05, 0.05) + np.float32(e) * np.float32(0.01)
                        for e in range(E)])
    hidden = g.uniform_array(D, -1.0, 1.0)
    inv = np.float32(1.0) / np.sqrt(np.float32(D))
    eff = g.uniform_array(D, 0.5, 1.5) * inv
    escale = g.uniform_array(E, 0.6, 1.4)
    # the kernel reads hidden as fp16 and both scales as bf16
    hidden16 = O.f16_to_float(O.f16_bits(hidden))
    eff_bits, es_bits = O.bf16_bits(eff), O.bf16_bits(escale)
    idx_ref, w_ref, (p, s, b) = _router_reference(weights, hidden, eff, escale)
    logits = O.router_logits(8, p, s, b, hidden16, eff_bits)
    idx, w = O.router_topk(logits, 8, es_bits)
    assert np.array_equal(idx, idx_ref)
    assert np.abs(O.f16_to_float(w) - w_ref).max() < 5e-3

    # productionRouterResolvesNearTieLikeReference (:46-70)
    g = O.SplitMix64(0x71E0F4A)
    pattern = g.uniform_array(D, 0.2, 1.0)
    hidden = g.uniform_array(D, 0.5, 1.5)
    gains = np.zeros(E, np.float32)
    for e in range(7):
        gains[e] = np.float32(1.0) - np.float32(e) * np.float32(0.05)
    gains[7] = 0.5
    gains[8] = np.float32(0.5) * (np.float32(1.0) + np.float32(1e-4))
    for e in range(9, E):
        gains[e] = np.float32(0.4) - np.float32(e - 9) * np.float32(0.02)
    weights = np.stack([pattern * gn for gn in gains])
    ones_d, ones_e = np.ones(D, np.float32), np.ones(E, np.float32)
    idx_ref, _, (p, s, b) = _router_reference(weights, hidden, ones_d, ones_e)
    hidden16 = O.f16_to_float(O.f16_bits(hidden))
    idx, _ = O.router_topk(O.router_logits(8, p, s, b, hidden16, None), 8)
    idx_ref16, _, _ = _router_reference(weights, hidden16, ones_d, ones_e)
    assert np.array_equal(idx, idx_ref16)
    assert list(idx[:7]) == list(range(7))     # gains 1.0 .. 0.7 dominate


def test_router_topk_is_stable_sort_and_softmax():
    rng = np.random.default_rng(5)
    for k in (1, 2, 8):
        for _ in range(50):
            logits = rng.standard_normal(256).astype(np.float32)
            logits[rng.integers(0, 256, 40)] = logits[rng.integers(0, 256, 40)]  # exact ties
            idx, w = O.router_topk(logits, k)
            order = sorted(range(256), key=lambda e: (-logits[e], e))[:k]
            assert list(idx) == order
            ex = np.exp(logits[order].astype(np.float64) - float(logits[order[0]]))
            assert np.abs(O.f16_to_float(w) - ex / ex.sum()).max() < 1e-3
    # all-equal logits: the lowest indices win, in order
    idx, w = O.router_topk(np.zeros(256, np.float32), 8)
    assert list(idx) == list(range(8)) and np.all(O.f16_to_float(w) == 0.125)


def test_router_logits_all_kinds_match_float64_dot():
    rng = np.random.default_rng(9)
    E, D = 64, 2048
    w = O.round_bf16((rng.standard_normal((E, D)) * 0.02).astype(np.float32))
    x = O.round_bf16(rng.standard_normal(D).astype(np.float32))
    dense = O.router_logits(16, O.bf16_bits(w), None, None, x)
    assert O.rel_error(dense, w.astype(np.float64) @ x.astype(np.float64)) < 1e-5
    for bits in (4, 8):
        p, s, b = O.quantize_affine(w, bits)
        got = O.router_logits(bits, p, s, b, x)
        want = O.dequantize_affine(p, s, b, D, bits).astype(np.float64) @ x.astype(np.float64)
        assert O.rel_error(got, want) < 1e-5
        # and agrees with the plain GEMV up to summation order
        assert O.rel_error(got, O.affine_gemv(p, s, b, x, bits)) < 1e-5


def test_moe_layer_forward_matches_float64_dense_model():
    rng = np.random.default_rng(21)
    d, f, E, k, T = 256, 128, 16, 4, 3
    for bits in (4, 8):
        mk = lambda r, c: O.round_bf16((rng.standard_normal((r, c)) * 0.05).astype(np.float32))
        experts = [(mk(f, d), mk(f, d), mk(d, f)) for _ in range(E)]
        blobs = np.stack([O.pack_expert(g, u, dn, bits) for g, u, dn in experts])
        shared = O.pack_expert(mk(f, d), mk(f, d), mk(d, f), bits)
        router_w = O.bf16_bits(mk(E, d))
        gate_row = O.quantize_affine(mk(1, d), 8)
        x = O.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
        idx, w, y = O.moe_layer_forward(x, d, f, k, bits, (16, router_w, None, None), blobs,
                                        shared, (8,) + gate_row)
        off = O.expert_offsets(d, f, bits)

        def dense_ffn(blob, xv):
            m = lambda wo, so, bo, r, c: O.dequantize_affine(
                blob[wo:wo + r * c * bits // 8].reshape(r, -1),
                blob[so:so + r * c // 32].view(np.uint16).reshape(r, -1),
                blob[bo:bo + r * c // 32].view(np.uint16).reshape(r, -1), c, bits).astype(np.float64)
            g = m(off[0], off[1], off[2], f, d) @ xv
            u = m(off[3], off[4], off[5], f, d) @ xv
            return m(off[6], off[7], off[8], d, f) @ (g / (1 + np.exp(-g)) * u)
        for t in range(T):
            xv = x[t].astype(np.float64)
            logits = O.bf16_to_float(router_w).astype(np.float64) @ xv
            order = sorted(range(E), key=lambda e: (-logits[e], e))[:k]
            assert list(idx[t]) == order
            gl = O.dequantize_affine(*gate_row, d, 8).astype(np.float64)[0] @ xv
            want = dense_ffn(shared, xv) / (1 + np.exp(-gl))
            for slot, e in enumerate(order):
                want = want + float(O.f16_to_float(w[t, slot])) * dense_ffn(blobs[e], xv)
            assert O.rel_error(y[t], want) < 2e-5
