"""GPU parity: tiled softmax and the top-64 / generic samplers through the C ABI.

Token ids are integer-class given identical fp16 probabilities: the GPU samplers read the same
probability buffer as the oracle and must return the same token."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import act_np, act_tensor, dev, gauss, round_act, say, u16, u32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nv():
    import nvmai_amd
    return nvmai_amd


@pytest.fixture(scope="module", params=[0, 1], ids=["bf16", "fp16"])
def ctx(request, nv):
    c = nv.Context(0, request.param)
    yield c
    torch.cuda.synchronize()
    c.close()


def _probs_dev(p_bits):
    return dev(np.ascontiguousarray(p_bits).view(np.float16))


@pytest.mark.parametrize("v", [1003, 4096, 248320])
def test_softmax_tiled_matches_oracle(nv, ctx, v):
    say("softmax", ctx.act, v)
    rng = np.random.default_rng(v)
    logits = round_act(gauss(rng, (3, v), 4.0), ctx.act)
    sm = nv.LogitSoftcapSoftmaxTiled(ctx, v)
    for softcap in (0.0, 30.0):
        got = u16(sm.encode(act_tensor(logits, ctx), softcap=softcap))
        torch.cuda.synchronize()
        for r in range(3):
            want = O.softmax_f16(logits[r], softcap)
            assert np.abs(got[r].astype(np.int32) - want.astype(np.int32)).max() <= 2       # fp16 ulps
            p = O.f16_to_float(got[r]).astype(np.float64)
            assert abs(p.sum() - 1.0) < 2e-3
    with pytest.raises(nv.NvmaiError):                       # "vocab mismatch: built for ..."
        sm.encode(act_tensor(logits[:, :v - 1], ctx))


def _lcg_probs(v):
    i = np.arange(v, dtype=np.uint64)
    mixed = i * np.uint64(6364136223846793005) + np.uint64(1442695040888963407)
    p = ((mixed >> np.uint64(40)).astype(np.uint32).astype(np.float32) + np.float32(1)) * np.float32(1.0 / 16777217.0)
    return O.f16_bits(p)


def test_top64_candidates_and_tokens_on_reference_input(nv, ctx):
    # SampleTopK64Tests.swift:115-130, 168-187: production vocabulary, LCG probabilities
    say("sampler lcg", ctx.act)
    v = 262144
    probs = _lcg_probs(v)
    pd = _probs_dev(probs)
    tk = nv.SampleTopK64(ctx, v)
    assert tk.scratch_bytes == 139264                        # SampleTopK64Tests.swift:117
    gen = nv.Sample(ctx)
    tok, top = tk.encode(pd, 1.0, 0.95, 1, 64, want_top64=True)
    torch.cuda.synchronize()
    _, idx, val = O.sample_topk64(probs, 1.0, 0.95, 1, 64, want_top64=True)
    top = top.cpu().numpy().view(np.uint32)[0]
    assert np.array_equal(top[:, 1], idx) and np.array_equal(top[:, 0], val.view(np.uint32))
    for k in (1, 2, 7, 20, 33, 63, 64):
        for t in (0.6, 0.7, 1.0):
            for seed in (1, 42, 0x123456789ABCDEF0, 2 ** 64 - 1):
                want = O.sample_topk64(probs, t, 0.95, seed, k)
                a = int(tk.encode(pd, t, 0.95, seed, k)[0]) & 0xFFFFFFFF
                assert a == want, (k, t, seed)
    for k, t, seed in [(1, 0.6, 1), (20, 0.6, 42), (64, 1.0, 7)]:        # generic == tiled, token for token
        b = int(gen.encode(pd, t, k, 0.95, seed)[0]) & 0xFFFFFFFF
        assert b == O.sample_generic(probs, t, k, 0.95, seed) == O.sample_topk64(probs, t, 0.95, seed, k)


def test_sampler_ties_flat_geometric_and_greedy(nv, ctx):
    say("sampler small cases", ctx.act)
    v = 1003
    tk, gen = nv.SampleTopK64(ctx, v), nv.Sample(ctx)
    ones = O.f16_bits(np.ones(v, np.float32))
    flat = O.f16_bits(np.full(v, 1.0 / v, np.float32))
    geo = np.zeros(v, np.float32)
    geo[:128] = (0.85 ** np.arange(128)).astype(np.float32)
    geo = O.f16_bits(geo)
    for name, probs, ks in (("ones", ones, (64,)), ("flat", flat, (64,)), ("geo", geo, (3, 8, 20, 64))):
        pd = _probs_dev(probs)
        for k in ks:
            rows = 16
            seeds = [s * 7919 + 1 for s in range(rows)]
            batch = tk.encode(pd.expand(rows, -1).contiguous(), 1.0, 0.95, seeds, k).cpu().numpy().view(np.uint32)
            gbatch = gen.encode(pd.expand(rows, -1).contiguous(), 1.0, k, 0.95, seeds).cpu().numpy().view(np.uint32)
            for r, seed in enumerate(seeds):
                want = O.sample_topk64(probs, 1.0, 0.95, seed, k)
                assert batch[r] == want == gbatch[r], (name, k, seed)
                assert want < 64 and (name != "geo" or want < k)
    p = np.zeros(512, np.float32)
    p[[10, 20, 30]] = [0.5, 0.25, 0.25]
    pd = _probs_dev(O.f16_bits(p))
    assert int(gen.encode(pd, 0.0, 20, 0.95, 1)[0]) == 10                  # greedy argmax
    tie = np.zeros(512, np.float32)
    tie[[40, 7, 300]] = 0.3
    assert int(gen.encode(_probs_dev(O.f16_bits(tie)), 0.0)[0]) == 7       # lowest index wins a tie
    # greedy with nothing above -inf (all NaN, all -inf): token 0 as the reference's reduction gives
    # (logit.metal:340-382), never an out-of-range id
    assert int(gen.encode(_probs_dev(np.full(512, 0x7E00, np.uint16)), 0.0)[0]) == 0
    assert int(gen.encode(_probs_dev(np.full(512, 0xFC00, np.uint16)), 0.0)[0]) == 0
    with pytest.raises(nv.NvmaiError):                                     # temperature must be > 0
        nv.SampleTopK64(ctx, 512).encode(pd, 0.0, 0.95, 1, 20)
    with pytest.raises(nv.NvmaiError):                                     # k in 1...64
        nv.SampleTopK64(ctx, 512).encode(pd, 1.0, 0.95, 1, 65)
    with pytest.raises(nv.NvmaiError):                                     # unsupportedVocabulary
        nv.SampleTopK64(ctx, 262145)


def test_softmax_then_sampler_pipeline(nv, ctx):
    # configs[4] tail: logits over 248,320 entries -> softmax -> top-k 20, top-p 0.95, T 0.6, fixed seed
    say("softmax+sampler pipeline", ctx.act)
    v = 248320
    rng = np.random.default_rng(5)
    logits = round_act(gauss(rng, (2, v), 3.0), ctx.act)
    probs = nv.LogitSoftcapSoftmaxTiled(ctx, v).encode(act_tensor(logits, ctx), softcap=0.0)
    seeds = [nv.sampler_seed_for(1234, pos) for pos in (0, 1)]
    assert seeds == [O.seed_for(1234, 0), O.seed_for(1234, 1)]
    tok = nv.SampleTopK64(ctx, v).encode(probs, 0.6, 0.95, seeds, 20).cpu().numpy().view(np.uint32)
    torch.cuda.synchronize()
    ph = u16(probs)
    for r in range(2):
        assert tok[r] == O.sample_topk64(ph[r], 0.6, 0.95, seeds[r], 20)


def test_gumbel_max_path_matches_oracle(nv, ctx):
    say("gumbel sampler", ctx.act)
    # top_k == 0 and top_p outside (0, 1): logit.metal:391-429; scores must be the same bits
    gen = nv.Sample(ctx)
    rng = np.random.default_rng(17)
    for v in (1003, 248320):
        p = O.softmax_f16(gauss(rng, (v,), 3.0))
        p[5] = 0                                                   # an ineligible entry
        pd = _probs_dev(p)
        for t, top_p in ((1.0, 1.0), (0.6, 0.0), (2.5, 1.5)):
            for seed, pos in ((1, 0), (42, 17), (0x123456789ABCDEF0, 4095)):
                got = int(gen.encode(pd, t, 0, top_p, seed, pos)[0]) & 0xFFFFFFFF
                assert got == O.sample(p, t, 0, top_p, seed, pos), (v, t, seed, pos)
    # rows with their own seed and position
    rows = 7
    seeds, poss = [100 + r for r in range(rows)], [3 * r for r in range(rows)]
    batch = gen.encode(pd.expand(rows, -1).contiguous(), 0.8, 0, 1.0, seeds, poss).cpu().numpy().view(np.uint32)
    assert [int(x) for x in batch] == [O.sample_gumbel(p, 0.8, seeds[r], poss[r]) for r in range(rows)]
    # a second call right after (the per-row block counters must have been reset)
    again = gen.encode(pd.expand(rows, -1).contiguous(), 0.8, 0, 1.0, seeds, poss).cpu().numpy().view(np.uint32)
    assert np.array_equal(batch, again)
    z = np.zeros(512, np.uint16)
    assert int(gen.encode(_probs_dev(z), 1.0, 0, 1.0, 1, 0)[0]) == 0   # nothing eligible -> token 0


def test_sampler_sample_front_end(nv, ctx):
    # Sampler.sample (Sampler.swift:171-234): penalty over the history, softcap + softmax, then the
    # tiled sampler for k in 1...64 at T > 0 and the generic kernel otherwise.  Tokens must equal the
    # oracle's samplers run on the probabilities the GPU produced; the path names are the reference's.
    say("Sampler.sample", ctx.act)
    v = 248320
    rng = np.random.default_rng(31)
    base = (rng.standard_normal(v) * 2.5).astype(np.float32)
    base[[17, 4000, 99999]] += 9.0
    base = round_act(base, ctx.act)
    history = [17, 4000, 17, 5, v + 3, -1, 4000]
    for softcap in (0.0, 30.0):
        for cfg, path_name, tiled in [
                (nv.GenerationConfig(seed=1234), "gpuSampled", True),                       # production default
                (nv.GenerationConfig(top_k=64, top_p=None, seed=9), "gpuSampled", True),
                (nv.GenerationConfig(top_k=100, top_p=0.9, seed=9), "gpuSampled", False),   # k > 64: generic
                (nv.GenerationConfig(temperature=0.8, top_k=None, top_p=None, seed=5), "gpuSampled", False),   # Gumbel
                (nv.GenerationConfig(temperature=0.0, seed=1), "greedyGPU", False),
                (nv.GenerationConfig(repetition_penalty=1.3, seed=77), "hostPenalty", True),
                (nv.GenerationConfig(temperature=0.0, repetition_penalty=4.0, seed=1), "hostPenalty", False)]:
            for which in ("tiled", "generic"):
                sampler = nv.Sampler(ctx, v, softcap, which)
                logits = act_tensor(base, ctx)
                position = 41
                tok, path = sampler.sample(logits, history, cfg, position)
                torch.cuda.synchronize()
                assert path == path_name
                want_logits = base
                if cfg.repetition_penalty != 1.0:
                    want_logits = O.repetition_penalty(base, ctx.act, history, cfg.repetition_penalty, softcap)
                    got_logits = act_np(logits)
                    if softcap == 0.0:
                        assert np.array_equal(got_logits, want_logits)         # one IEEE operation per id
                    else:
                        assert np.abs(got_logits - want_logits).max() <= 2 ** -5   # tanh / atanh from two libraries
                    assert np.array_equal(np.delete(got_logits, [17, 4000, 5]), np.delete(base, [17, 4000, 5]))
                probs = sampler.probs.cpu().numpy().view(np.uint16)
                ref = O.f16_to_float(O.softmax_f16(act_np(logits), softcap=softcap, tiled=True))
                assert np.abs(O.f16_to_float(probs) - ref).max() <= 2e-3 * ref.max() + 1e-7
                seed = O.seed_for(cfg.seed, position)
                k = 0 if cfg.top_k is None else cfg.top_k
                p = 1.0 if cfg.top_p is None else cfg.top_p
                if which == "tiled" and tiled and cfg.temperature > 0:
                    want = O.sample_topk64(probs, cfg.temperature, p, seed, top_k=k)
                else:
                    want = O.sample(probs, cfg.temperature, k, p, seed, position)
                assert int(tok[0]) == want, (softcap, which, cfg.__dict__)
                if cfg.temperature == 0.0 and cfg.repetition_penalty == 4.0 and softcap == 0.0:
                    assert want not in (17, 4000, 99999) or want == 99999       # the penalized peaks lost
    # the incremental history of the reference: the first call folds the whole history, later calls
    # only the last id (Sampler.swift:262-270)
    sampler = nv.Sampler(ctx, v, 0.0)
    cfg = nv.GenerationConfig(temperature=0.0, repetition_penalty=2.0, seed=1)
    logits = act_tensor(base, ctx)
    sampler.sample(logits, [17], cfg, 0)
    logits2 = act_tensor(base, ctx)
    sampler.sample(logits2, [99999, 4000], cfg, 1)          # only 4000 joins the table
    torch.cuda.synchronize()
    want = O.repetition_penalty(base, ctx.act, [17, 4000], 2.0)
    assert np.array_equal(act_np(logits2), want)
    with pytest.raises(nv.NvmaiError) as e:                 # top-p below one without top-k is not implemented
        nv.Sampler(ctx, v, 0.0).sample(logits, [], nv.GenerationConfig(top_k=None, top_p=0.5), 0)
    assert e.value.name == "unsupported"
    with pytest.raises(nv.NvmaiError):
        nv.Sampler(ctx, v, 0.0).sample(logits, [], nv.GenerationConfig(top_k=300), 0)


def test_repetition_penalty_long_history_with_repeats(nv, ctx):
    # a history of 131,072 ids drawn from 5,000 distinct ones (every id about 26 times, plus ids out of range):
    # every distinct id is penalised exactly once, whatever the number and the order of its occurrences --
    # the oracle walks the distinct ids as the reference's dictionary does (Sampler.swift:259-293)
    say("repetition penalty, long history", ctx.act)
    rng = np.random.default_rng(131072)
    v = 248320
    base = round_act(gauss(rng, (v,), 3.0), ctx.act)
    pool_ids = rng.choice(v, 5000, replace=False)
    history = rng.choice(pool_ids, 131072).astype(np.int32)
    history[::1000] = -1
    history[500::1000] = v + 7
    for softcap in (0.0, 30.0):
        logits = act_tensor(base, ctx)
        nv.ops.repetition_penalty(ctx, logits, dev(history), 1.3, softcap)
        torch.cuda.synchronize()
        distinct = [int(i) for i in dict.fromkeys(history.tolist()) if 0 <= i < v]
        want = O.repetition_penalty(base, ctx.act, distinct, 1.3, softcap)
        if softcap == 0.0:
            assert np.array_equal(act_np(logits), want)                     # one IEEE operation per id
        else:
            assert np.abs(act_np(logits) - want).max() <= 2 ** -5           # tanh / atanh from two libraries
        untouched = np.ones(v, bool)
        untouched[distinct] = False
        assert np.array_equal(act_np(logits)[untouched], base[untouched])


def test_sampler_sample_reference_properties(nv, ctx):
    # The reference's own Sampler tests (tests/NVMAI/Core/Runtime/Generation/SamplerTests.swift:68-197)
    # through the C ABI, default softcap 30 as there.
    say("Sampler.sample reference properties", ctx.act)

    def draw(sampler, values, cfg, position=0, history=()):
        tok, path = sampler.sample(act_tensor(np.asarray(values, np.float32), ctx), list(history), cfg, position)
        torch.cuda.synchronize()
        return int(tok[0]), path

    # degenerateDistributionStillReturnsAnInRangeToken (:68-80)
    s = nv.Sampler(ctx, 64)
    for fill in (-np.inf, np.nan):
        for seed in range(1, 9):
            tok, _ = draw(s, np.full(64, fill, np.float32), nv.GenerationConfig(1.0, 64, 0.95, seed=seed), seed)
            assert tok < 64
    # greedy_picksArgmax (:82-91)
    lg = np.full(2048, 0.1, np.float32)
    lg[1337] = 9.0
    assert draw(nv.Sampler(ctx, 2048), lg, nv.GenerationConfig(temperature=0.0)) == (1337, "greedyGPU")
    # seeded_isDeterministicAtPosition / reproducibleAcrossPositions (:93-121)
    g = O.seed_tree(0x51A71006, "sampler-position-replay")
    lg = g.uniform_array(1024, -2.0, 2.0)
    s = nv.Sampler(ctx, 1024)
    cfg = nv.GenerationConfig(temperature=1.0, seed=42)
    run1 = [draw(s, lg, cfg, p)[0] for p in range(5)]
    run2 = [draw(s, lg, cfg, p)[0] for p in range(5)]
    assert run1 == run2 and draw(s, lg, cfg, 0)[1] == "gpuSampled"
    assert [draw(s, lg, nv.GenerationConfig(temperature=1.0, seed=43), p)[0] for p in range(5)] != run1
    # topK_restrictsToTop (:123-135)
    lg = np.full(1024, -8.0, np.float32)
    lg[[10, 200, 500, 900]] = [4.0, 3.0, 2.0, 1.0]
    for t in range(32):
        assert draw(s, lg, nv.GenerationConfig(1.0, 4, 0.95, seed=t + 1), t)[0] in (10, 200, 500, 900)
    # topP_restrictsToNucleus (:137-147)
    lg = np.full(512, -10.0, np.float32)
    lg[7], lg[42] = 6.0, 5.6
    s = nv.Sampler(ctx, 512)
    for t in range(32):
        assert draw(s, lg, nv.GenerationConfig(1.0, 20, 0.9, seed=t + 1), t)[0] in (7, 42)
    # repetitionPenalty_suppressesHistory (:149-169)
    s = nv.Sampler(ctx, 64)
    count5 = 0
    for t in range(200):
        tok, path = draw(s, np.full(64, 8.0, np.float32), nv.GenerationConfig(1.0, 20, 0.95, 2.0, seed=t + 1), t, [5, 5, 5])
        assert path == "hostPenalty"
        count5 += tok == 5
    assert count5 < 0.5 * 200 / 64
    # repetitionPenalty_bitesOnSaturatedLogits (:177-197)
    s = nv.Sampler(ctx, 64)
    lg = np.full(64, 300.0, np.float32)
    lg[5] = 400.0
    count5 = sum(draw(s, lg, nv.GenerationConfig(1.0, 20, 0.95, 1.3, seed=t + 1), t, [5])[0] == 5 for t in range(64))
    assert count5 < 64 // 8
