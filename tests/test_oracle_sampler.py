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
    assert O.sample_topk64(pb, 1.0, 0.4, 77, 20) == 10           # nucleus cut at the first entry
