"""Pins the oracle's softmax, RNG and samplers."""
import numpy as np

import oracle as O
import ctypes as C


def test_xorshift64star_textbook_values_and_seed_for():
    s = C.c_uint64(1)
    # state after one step from 1: 1 ^ (1<<13) = 0x2001; ^ >>7 = 0x2041; ^ <<17 = 0x40822041
    assert O.lib.orc_xorshift64star(C.byref(s)) == (0x40822041 * 2685821657736338717) % 2**64
    assert s.value == 0x40822041
    s = C.c_uint64(42)
    u = O.lib.orc_uniform01(C.byref(s))
    assert 0.0 <= u < 1.0 and u * 16777216.0 == int(u * 16777216.0)
    # Sampler.swift:304-325: splitmix64(seed + position), 0 -> golden ratio
    assert O.seed_for(0, 0) == 0xE220A8397B1DCDAF        # splitmix64 finalizer of 0+gamma
    assert O.seed_for(7, 5) == O.seed_for(12, 0) == O.seed_for(0, 12)


def test_softmax_matches_float64_and_tiled_matches_single():
    rng = np.random.default_rng(8)
    for v in (1003, 4096, 248320):
        logits = O.f16_to_float(O.f16_bits(rng.standard_normal(v).astype(np.float32) * 4))
        p = O.f16_to_float(O.softmax_f16(logits))
        z = logits.astype(np.float64)
        want = np.exp(z - z.max())
        want /= want.sum()
        assert np.abs(p - want).max() < 1e-3 * want.max() + 1e-7
        # LogitSoftcapSoftmaxTests.swift:119-160 bounds tiled-vs-single by 1e-5 on
        # its inputs; here large probabilities occur, so the bound is one fp16 ulp.
        bt = O.softmax_f16(logits, tiled=True).astype(np.int32)
        assert np.abs(bt - O.softmax_f16(logits).astype(np.int32)).max() <= 1
    capped = O.f16_to_float(O.softmax_f16(np.array([1e3, 0, -1e3], np.float32), softcap=30.0))
    want = np.exp(np.array([30.0, 0, -30.0]) - 30)
    assert np.abs(capped - want / want.sum()).max() < 1e-3


def _lcg_probs(v):
    # SampleTopK64Tests.swift:118-121
    i = np.arange(v, dtype=np.uint64)
    mixed = i * np.uint64(6364136223846793005) + np.uint64(1442695040888963407)
    p = ((mixed >> np.uint64(40)).astype(np.uint32).astype(np.float32) + np.float32(1)) \
        * np.float32(1.0 / 16777217.0)
    return O.f16_bits(p)


def test_top64_is_exact_top64_of_vocab():
    probs = _lcg_probs(262144)
    _, idx, val = O.sample_topk64(probs, 1.0, 0.95, 1, 64, want_top64=True)
    pv = O.f16_to_float(probs)
    order = np.lexsort((np.arange(pv.size), -pv))[:64]
    assert np.array_equal(idx, order.astype(np.uint32))
    assert np.array_equal(val, pv[order])


def test_tiled_sampler_equals_generic_on_reference_inputs():
    probs = _lcg_probs(262144)
    # productionVocabularyMatchesCurrentSampler (:115-130)
    for t in (0.7, 0.85, 1.0):
        for seed in (1, 2, 0x123456789ABCDEF0, 2**64 - 1):
            assert O.sample_topk64(probs, t, 0.95, seed, 64) == O.sample_generic(probs, t, 64, 0.95, seed)
    # everyKUpToSixtyFourMatchesTheGenericSampler (:168-187)
    for k in (1, 2, 7, 20, 33, 63, 64):
        for t in (0.6, 1.0):
            for seed in (1, 42, 0x123456789ABCDEF0):
                assert O.sample_topk64(probs, t, 0.95, seed, k) == O.sample_generic(probs, t, k, 0.95, seed)


def test_sampler_ties_flat_and_geometric_cases():
    ones = O.f16_bits(np.ones(1003, np.float32))
    for seed in range(1, 9):                                   # :132-142
        a = O.sample_topk64(ones, 1.0, 0.95, seed, 64)
        assert a == O.sample_generic(ones, 1.0, 64, 0.95, seed) and a < 64
    flat = O.f16_bits(np.full(1003, 1.0 / 1003.0, np.float32))
    seen = set()
    for seed in range(1, 257):                                 # :144-159
        a = O.sample_topk64(flat, 1.0, 0.95, seed, 64)
        assert a == O.sample_generic(flat, 1.0, 64, 0.95, seed) and a < 64
        seen.add(a)
    assert any(a >= 61 for a in seen)
    geo = np.zeros(1003, np.float32)
    geo[:128] = (0.85 ** np.arange(128)).astype(np.float32)
    geo = O.f16_bits(geo)
    for k in (3, 8, 20, 64):                                   # :196-213
        for seed in (1, 5, 99, 4242):
            a = O.sample_topk64(geo, 1.0, 0.95, seed, k)
            assert a == O.sample_generic(geo, 1.0, k, 0.95, seed) and a < k


def test_sampler_distribution_and_greedy():
    # inverse-CDF draw over a known 3-point distribution: frequencies follow p^(1/T)
    p = np.zeros(512, np.float32)
    p[[10, 20, 30]] = [0.5, 0.25, 0.25]
    pb = O.f16_bits(p)
    counts = {10: 0, 20: 0, 30: 0}
    n = 4000
    for seed in range(1, n + 1):
        counts[O.sample_topk64(pb, 0.5, 1.0, O.seed_for(123, seed), 20)] += 1
    w = np.array([0.25, 0.0625, 0.0625])
    w /= w.sum()
    got = np.array([counts[10], counts[20], counts[30]]) / n
    assert np.abs(got - w).max() < 0.03
    assert O.sample_generic(pb, 0.0, 20, 0.95, 1) == 10          # greedy argmax
    # nothing above -inf: the reference's reduction starts every lane at index 0 and ends there
    # (logit.metal:340-382); an out-of-range id must never reach the generation loop
    nan_bits = np.full(512, 0x7E00, np.uint16)
    assert O.sample_generic(nan_bits, 0.0, 20, 0.95, 1) == 0
    assert O.sample_generic(np.full(512, 0xFC00, np.uint16), 0.0, 0, 1.0, 1) == 0      # all -inf
    assert O.sample_topk64(pb, 1.0, 0.4, 77, 20) == 10           # nucleus cut at the first entry


def _splitmix_gumbel_u(seed, position, row):
    """logit.metal:296-313 in Python integers: the 24-bit draw behind one Gumbel value."""
    m = (1 << 64) - 1
    x = (seed ^ ((position * 0xD2B74407B1CE6E93) & m) ^ row) & m
    x = (x + 0x9E3779B97F4A7C15) & m
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & m
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & m
    x = x ^ (x >> 31)
    return x >> 40


def test_gumbel_noise_closed_form_and_path_choice():
    # the draw: SplitMix64 of (seed ^ position * C ^ row), top 24 bits, (bits + 0.5) / 2^24
    for seed, pos, row in [(1, 0, 0), (42, 17, 248319), (0x123456789ABCDEF0, 4095, 7), (0, 0, 0)]:
        bits = _splitmix_gumbel_u(seed, pos, row)
        u = np.float32(np.float32(bits) + np.float32(0.5)) * np.float32(1.0 / 16777216.0)
        want = -np.log(-np.log(np.float64(u)))
        assert abs(O.gumbel_for(seed, pos, row) - want) <= 4e-7 * max(1.0, abs(want))
    # SplitMix64's first output for state 0 is a published constant
    assert _splitmix_gumbel_u(0, 0, 0) == 0xE220A8397B1DCDAF >> 40
    rng = np.random.default_rng(3)
    p = O.softmax_f16(rng.standard_normal(1003).astype(np.float32) * 2)
    # the kernel's choice of path (logit.metal:340, 391, 431)
    assert O.sample(p, 0.0, 0, 1.0, 5, 9) == O.sample_generic(p, 0.0, 0, 1.0, 5)
    assert O.sample(p, 0.8, 0, 1.0, 5, 9) == O.sample_gumbel(p, 0.8, 5, 9)
    assert O.sample(p, 0.8, 0, 0.0, 5, 9) == O.sample_gumbel(p, 0.8, 5, 9)
    assert O.sample(p, 0.8, 20, 1.0, 5, 9) == O.sample_generic(p, 0.8, 20, 1.0, 5)
    assert O.sample(p, 0.8, 0, 0.9, 5, 9) == O.sample_generic(p, 0.8, 0, 0.9, 5)
    # position and seed both move the draw; zero probabilities are never chosen
    draws = {O.sample_gumbel(p, 1.0, 5, pos) for pos in range(64)}
    assert len(draws) > 8
    q = np.zeros(1003, np.uint16)
    assert O.sample_gumbel(q, 1.0, 1, 0) == 0                      # nothing eligible -> token 0
    q[777] = O.f16_bits(np.array([0.5], np.float32))[0]
    assert all(O.sample_gumbel(q, 0.7, s, s) == 777 for s in range(20))


def test_gumbel_max_samples_p_to_the_one_over_t():
    # Gumbel-max over log(p)/T is a categorical draw with weights p^(1/T)
    rng = np.random.default_rng(0)
    p = O.softmax_f16(rng.standard_normal(600).astype(np.float32) * 2.5)
    pf = O.f16_to_float(p).astype(np.float64)
    for T in (1.0, 0.6):
        w = np.where(pf > 0, pf ** (1.0 / T), 0.0)
        w /= w.sum()
        n = 6000
        cnt = np.bincount([O.sample_gumbel(p, T, 1000 + s, s % 5) for s in range(n)], minlength=600)
        top = np.argsort(-w)[:6]
        sigma = np.sqrt(w[top] * (1 - w[top]) / n)
        assert np.all(np.abs(cnt[top] / n - w[top]) <= 5 * sigma + 1e-3)


def test_repetition_penalty_and_sampler_policy():
    # Sampler.applyRepetitionPenaltyInPlace (Sampler.swift:259-293), HF convention: a positive logit
    # is divided, a negative one multiplied, once per DISTINCT history id, ids outside the
    # vocabulary ignored.  Exactly representable values pin the arithmetic.
    lg = np.array([2.0, -2.0, 0.0, 4.0, -1.0, 8.0], np.float32)
    out = O.repetition_penalty(lg, 1, [0, 1, 1, 2, 0, 99, -3], 1.25)
    assert list(out) == [1.599609375, -2.5, 0.0, 4.0, -1.0, 8.0]     # 2 / 1.25 = 1.6 -> fp16 1638 / 1024
    assert np.array_equal(O.repetition_penalty(lg, 0, [3, 5], 2.0), [2.0, -2.0, 0.0, 2.0, -1.0, 4.0])
    # with a softcap the PENALIZED CAPPED logit is what the downstream softcap reproduces
    cap, pen = 30.0, 1.1
    z = np.array([50.0, -50.0, 3.0, 200.0], np.float32)
    got = O.repetition_penalty(z, 1, [0, 1, 2, 3], pen, cap).astype(np.float64)
    capped = cap * np.tanh(z.astype(np.float64) / cap)
    want_capped = np.where(capped > 0, capped / pen, capped * pen)
    want_capped = np.clip(want_capped, -cap * 0.9999, cap * 0.9999)
    # fp16 rounding of the stored logit moves the capped value by at most ulp * (1 - tanh^2)
    assert np.abs(cap * np.tanh(got / cap) - want_capped).max() < 0.05
    assert np.all(np.isfinite(got))                                 # the clamp keeps atanh finite (:283-286)
    # path choice (Sampler.swift:196-231): tiled for k in 1...64 at T > 0, generic otherwise
    assert [O.sampler_route(True, 0.6, k) for k in (1, 20, 64, 65, 256, None)] == [2, 2, 2, 1, 1, 1]
    assert O.sampler_route(True, 0.0, 20) == 0 and O.sampler_route(False, 0.6, 20) == 1
    # the whole call equals its parts
    rng = np.random.default_rng(8)
    logits = O.round_bf16((rng.standard_normal(5000) * 3).astype(np.float32))
    tok, probs = O.sampler_sample(logits, 30.0, 0.6, 20, 0.95, 1234, 7)
    assert np.array_equal(probs, O.softmax_f16(logits, softcap=30.0, tiled=True))
    assert tok == O.sample_topk64(probs, 0.6, 0.95, O.seed_for(1234, 7), top_k=20)
    tok, probs = O.sampler_sample(logits, 0.0, 0.0, None, None, 1234, 7)
    assert tok == int(np.argmax(logits))                            # greedy
    tok, probs = O.sampler_sample(logits, 0.0, 0.8, None, None, 5, 3)
    assert tok == O.sample_gumbel(probs, 0.8, O.seed_for(5, 3), 3)  # neither top-k nor top-p: Gumbel-max
    tok, probs = O.sampler_sample(logits, 0.0, 0.8, 100, 0.9, 5, 3)
    assert tok == O.sample_generic(probs, 0.8, 100, 0.9, O.seed_for(5, 3))
