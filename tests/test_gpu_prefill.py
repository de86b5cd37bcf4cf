"""GPU parity for the prefill side: pair records, permutation / histogram by expert, grouped
expert GEMMs and the rank-order reduce, called through the C ABI and compared with the CPU
oracle.

Bars: every grouping array bit-exact (integers); 16-bit outputs within 1e-2 of the oracle as
max|diff| / max|ref| (RelError.swift:5-16)."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import act_np, act_tensor, dev, gauss, say, u32

pytestmark = pytest.mark.gpu

TOL_ACT = 1e-2


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


@pytest.fixture(scope="module")
def ctx_bf16(nv):
    c = nv.Context(0, 0)
    yield c
    torch.cuda.synchronize()
    c.close()


def _pairs(rows):
    a = np.zeros(len(rows), O.PAIR_DTYPE)
    for i, (t, e, r, w) in enumerate(rows):
        a[i] = (t, e, r, w)
    return a


def _pairs_dev(p):
    return dev(p.view(np.uint32).reshape(-1, 4).view(np.int32))


def _check_routes(routes, want):
    """Every array of the device grouping against the oracle's dict."""
    torch.cuda.synchronize()
    info = routes.validate()
    got_sorted = u32(routes.sorted_pairs).reshape(-1).view(O.PAIR_DTYPE)
    assert np.array_equal(got_sorted, want["sorted"])
    assert np.array_equal(u32(routes.per_expert_offsets), want["offsets"])
    assert np.array_equal(u32(routes.per_expert_counts), want["counts"])
    assert info[0] == want["groups"].size and info[1] == want["tiles"].size
    assert np.array_equal(u32(routes.groups).reshape(-1).view(O.GROUP_DTYPE), want["groups"])
    assert np.array_equal(u32(routes.tiles).reshape(-1).view(O.TILE_DTYPE), want["tiles"])
    assert info[4] == (want["counts"].max() if want["counts"].size else 0)


# ------------------------------------------------------------------ pairs + grouping
def test_make_pairs_token_major(nv, ctx_bf16):
    say("prefill make_pairs")
    # PrefillRouterTests.swift:12-31
    w = O.f16_bits(np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6], np.float32)).reshape(2, 3)
    idx = np.array([[3, 1, 2], [4, 0, 5]], np.uint32)
    got = nv.PrefillRouter(ctx_bf16).make_token_expert_pairs(dev(idx.view(np.int32)), dev(w.view(np.int16)))
    torch.cuda.synchronize()
    assert np.array_equal(u32(got).reshape(-1).view(O.PAIR_DTYPE), O.make_pairs(idx, w))


def test_grouping_reference_known_answers(nv, ctx_bf16):
    say("prefill grouping known answers")
    g = nv.PrefillMoEGrouping(ctx_bf16)
    # PrefillMoEGroupingTests.swift:5-53, input reversed
    rows = [(0, 3, 0, 10), (0, 1, 1, 11), (0, 4, 2, 12), (1, 1, 0, 13), (1, 3, 1, 14),
            (1, 2, 2, 15), (2, 4, 0, 16), (2, 3, 1, 17), (2, 1, 2, 18), (3, 5, 0, 19),
            (3, 1, 1, 20), (3, 4, 2, 21)]
    p = _pairs(rows[::-1])
    r = g.group_token_expert_pairs(_pairs_dev(p), 4, 3, 6, tile_expert_count=2)
    _check_routes(r, O.group_pairs(p, 4, 3, 6, 2))
    assert u32(r.per_expert_offsets).tolist() == [0xFFFFFFFF, 0, 4, 5, 8, 11]
    assert u32(r.tiles).tolist() == [[0, 2, 0, 5], [2, 2, 5, 6], [4, 1, 11, 1]]
    # :55-82 shuffled input, weight bits travel with their pair
    tm = [(0, 2, 0, 101), (0, 1, 1, 102), (1, 2, 0, 103), (1, 0, 1, 104), (2, 1, 0, 105), (2, 2, 1, 106)]
    sh = _pairs([tm[5], tm[1], tm[3], tm[0], tm[4], tm[2]])
    r = g.group_token_expert_pairs(_pairs_dev(sh), 3, 2, 3, 2)
    _check_routes(r, O.group_pairs(sh, 3, 2, 3, 2))
    assert u32(r.sorted_pairs)[:, 3].tolist() == [104, 102, 105, 101, 103, 106]
    # :84-115 expert sort keys
    rows = _pairs([(0, 1, 0, 10), (0, 2, 1, 20), (1, 3, 0, 30), (1, 1, 1, 11), (2, 2, 0, 21), (2, 3, 1, 31)])
    keys = np.array([0, 30, 10, 20], np.uint64)
    r = g.group_token_expert_pairs(_pairs_dev(rows), 3, 2, 4, 2, expert_sort_keys=dev(keys.view(np.int64)))
    _check_routes(r, O.group_pairs(rows, 3, 2, 4, 2, sort_keys=keys))
    assert u32(r.groups)[:, 0].tolist() == [2, 3, 1]
    # :175-203 pressure case
    rows = _pairs([(t, (t + r_ * 7) % 74, r_, t * 8 + r_) for t in range(32) for r_ in range(8)])
    r = g.group_token_expert_pairs(_pairs_dev(rows), 32, 8, 128, 16)
    _check_routes(r, O.group_pairs(rows, 32, 8, 128, 16))


def test_grouping_rejects_invalid_metadata(nv, ctx_bf16):
    say("prefill grouping errors")
    # PrefillMoEGroupingTests.swift:117-173
    g = nv.PrefillMoEGrouping(ctx_bf16)
    one = _pairs_dev(_pairs([(0, 0, 0, 1)]))
    cases = [((one, 1, 1, 1, 17), {}, "invalidTileExpertCount"),
             ((_pairs_dev(_pairs([(0, 2, 0, 1)])), 1, 1, 2, 1), {}, "expertOutOfRange"),
             ((_pairs_dev(_pairs([(0, 0, 0, 1), (0, 1, 0, 2)])), 1, 2, 2, 1), {}, "duplicateTokenRank"),
             ((one, 1, 1, 2, 1), dict(expert_sort_keys=dev(np.zeros(1, np.int64))), "expertSortKeyCountMismatch"),
             ((one, 2, 1, 1, 1), {}, "pairCountMismatch"),
             ((one, -1, 1, 1, 1), {}, "invalidQueryCount"),
             ((one, 1, 0, 1, 1), {}, "invalidTopK"),
             ((one, 1, 1, 0, 1), {}, "invalidNumExperts"),
             ((_pairs_dev(_pairs([(1, 0, 0, 1)])), 1, 1, 1, 1), {}, "tokenOutOfRange"),
             ((_pairs_dev(_pairs([(0, 0, 1, 1)])), 1, 1, 1, 1), {}, "rankOutOfRange")]
    for args, kw, name in cases:
        with pytest.raises(nv.PrefillMoEGroupingError) as e:
            g.group_token_expert_pairs(*args, **kw)
        assert e.value.name == name, name
    # the first failing pair in input order decides, as in the reference's loop
    p = _pairs([(0, 0, 0, 1), (0, 1, 1, 2), (1, 9, 0, 3), (0, 1, 1, 4), (7, 0, 1, 5)])
    with pytest.raises(O.GroupingError) as want:
        O.group_pairs(np.concatenate([p, p[:1]]), 3, 2, 4, 1)
    with pytest.raises(nv.PrefillMoEGroupingError) as e:
        g.group_token_expert_pairs(_pairs_dev(np.concatenate([p, p[:1]])), 3, 2, 4, 1)
    assert e.value.name == want.value.name == "expertOutOfRange" and e.value.pair_index == 2
    # empty input is valid and yields nothing
    r = g.group_token_expert_pairs(torch.empty((0, 4), dtype=torch.int32, device="cuda"), 0, 8, 4, 16)
    _check_routes(r, O.group_pairs(_pairs([]), 0, 8, 4, 16))
    # the C ABI itself refuses what the host check refuses
    st = nv.lib.nvmai_hip_prefill_group_pairs(ctx_bf16.handle, None, one.data_ptr(), 1, 1, 1, 1, 17, None, 0,
                                              r.desc)
    assert st == -1


def _zipf_routes(rng, tokens, E, k, s=1.1):
    """k distinct experts per token, expert popularity ~ 1 / rank^s."""
    p = 1.0 / np.arange(1, E + 1) ** s
    p /= p.sum()
    perm = rng.permutation(E)
    keys = rng.random((tokens, E)) ** (1.0 / p[None, :])      # weighted sampling without replacement
    idx = perm[np.argsort(-keys, axis=1)[:, :k]].astype(np.uint32)
    w = rng.random((tokens, k)).astype(np.float32) + 0.05
    w /= w.sum(axis=1, keepdims=True)
    return idx, O.f16_bits(w)


# (300, 600, ..) and (9000, 64, ..) take the three-launch path (more than 512 experts, more than 64
# histogram blocks), the others the fused scan + scatter launch
@pytest.mark.parametrize("tokens,E,k,tile", [(1, 8, 2, 16), (37, 20, 3, 4), (1000, 256, 8, 16), (4096, 256, 8, 16),
                                             (300, 600, 4, 7), (9000, 64, 8, 16), (8100, 512, 8, 16)])
def test_grouping_random_routes_bit_exact(nv, ctx_bf16, tokens, E, k, tile):
    say("prefill grouping random", tokens, E, k, tile)
    rng = np.random.default_rng(tokens * 31 + E)
    idx, w = _zipf_routes(rng, tokens, E, k)
    pairs = O.make_pairs(idx, w)
    g = nv.PrefillMoEGrouping(ctx_bf16)
    want = O.group_pairs(pairs, tokens, k, E, tile)
    # straight from the router's outputs
    _check_routes(g.group_routes(dev(idx.view(np.int32)), dev(w.view(np.int16)), E, tile), want)
    # pair records in shuffled order, with and without sort keys
    shuffled = pairs[rng.permutation(pairs.size)]
    _check_routes(g.group_token_expert_pairs(_pairs_dev(shuffled), tokens, k, E, tile), want)
    keys = rng.integers(0, 5, E).astype(np.uint64)
    _check_routes(g.group_token_expert_pairs(_pairs_dev(shuffled), tokens, k, E, tile,
                                             expert_sort_keys=dev(keys.view(np.int64))),
                  O.group_pairs(pairs, tokens, k, E, tile, sort_keys=keys))
    # histogram / permutation invariants at any size
    sp = want["sorted"]
    assert np.array_equal(want["counts"], np.bincount(idx.reshape(-1), minlength=E))
    assert np.all(np.diff(sp["expert"].astype(np.int64) * 2**40 + sp["token"].astype(np.int64) * 64 + sp["rank"]) > 0)


# ------------------------------------------------------------------ grouped GEMM + reduce
def _prefill_case(nv, ctx, rng, d, f, E, k, bits, tokens, std=0.05, check_tokens=None):
    mats = [(gauss(rng, (f, d), std), gauss(rng, (f, d), std), gauss(rng, (d, f), std)) for _ in range(E)]
    blobs = np.stack([O.pack_expert(*m, bits) for m in mats])
    x = O.round_bf16(gauss(rng, (tokens, d))) if ctx.act == 0 else O.f16_to_float(O.f16_bits(gauss(rng, (tokens, d))))
    idx, w = _zipf_routes(rng, tokens, E, k)
    off, stride = nv.expert_offsets(d, f, bits)
    assert stride == blobs.shape[1]
    routes = nv.PrefillMoEGrouping(ctx).group_routes(dev(idx.view(np.int32)), dev(w.view(np.int16)), E)
    partials, act = nv.PrefillGroupedRoutedMoE(ctx, bits).encode(dev(blobs), off, act_tensor(x, ctx), d, f, routes)
    h2 = nv.PrefillMoE(ctx).encode_reduce_token_major(partials, dev(w.view(np.int16)), tokens, k, d)
    torch.cuda.synchronize()
    routes.validate()
    sel = np.arange(tokens) if check_tokens is None else check_tokens
    want = O.prefill_moe(blobs, bits, x[sel], d, f, idx[sel], w[sel])
    err = O.rel_error(act_np(h2)[sel], want)
    assert err <= TOL_ACT, err
    return err


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("d,f,E,k,tokens", [(128, 64, 4, 2, 3), (256, 192, 6, 3, 150), (192, 64, 5, 2, 131)])
def test_grouped_moe_toy_shapes(nv, ctx, bits, d, f, E, k, tokens):
    say("prefill grouped moe toy", ctx.act, bits, d, f, E, k, tokens)
    _prefill_case(nv, ctx, np.random.default_rng(d + f + bits), d, f, E, k, bits, tokens)


def test_grouped_moe_synthetic_pool_known_answer(nv, ctx_bf16):
    say("prefill grouped moe synthetic pool")
    # PrefillGroupedRoutedMoETests.swift:271-280 closed-form weights (silu activation)
    d, f, E, T = 128, 64, 4, 3

    def rows(expert, role, r, c):
        i, j = np.meshgrid(np.arange(r), np.arange(c), indexing="ij")
        return ((expert + 1) * 1e-3 + (role + 1) * 3e-3 + ((i % 7) - 3) * 4e-4 + ((j % 11) - 5) * 2e-4).astype(np.float32)
    blobs = np.stack([O.pack_expert(rows(e, 0, f, d), rows(e, 1, f, d), rows(e, 2, d, f), 4) for e in range(E)])
    hidden = np.array([[(i % 17) - 8 for i in range(d)]] * T, np.float32) * np.float32(0.125)
    hidden += np.arange(T, dtype=np.float32)[:, None] * np.float32(0.25)
    idx = np.array([[0, 2], [1, 2], [3, 0]], np.uint32)
    w = O.f16_bits(np.array([[0.75, 0.25], [0.5, 0.5], [0.625, 0.375]], np.float32))
    off, _ = nv.expert_offsets(d, f, 4)
    routes = nv.PrefillMoEGrouping(ctx_bf16).group_routes(dev(idx.view(np.int32)), dev(w.view(np.int16)), E)
    partials, _ = nv.PrefillGroupedRoutedMoE(ctx_bf16, 4).encode(dev(blobs), off, act_tensor(hidden, ctx_bf16), d, f, routes)
    h2 = nv.PrefillMoE(ctx_bf16).encode_reduce_token_major(partials, dev(w.view(np.int16)), T, 2, d)
    torch.cuda.synchronize()
    assert O.rel_error(act_np(h2), O.prefill_moe(blobs, 4, hidden, d, f, idx, w)) <= TOL_ACT


def test_reduce_token_major_rank_order(nv, ctx):
    say("prefill reduce", ctx.act)
    rng = np.random.default_rng(5)
    T, k, d = 33, 8, 130
    part = act_tensor(gauss(rng, (T * k, d)), ctx)
    w = O.f16_bits(rng.random((T, k)).astype(np.float32))
    h2 = nv.PrefillMoE(ctx).encode_reduce_token_major(part, dev(w.view(np.int16)), T, k, d)
    torch.cuda.synchronize()
    pf, wf = act_np(part).reshape(T, k, d), O.f16_to_float(w)
    acc = np.zeros((T, d), np.float32)
    for r in range(k):                                   # prefill.metal:450-457: fma chain in rank order
        acc = (wf[:, r, None].astype(np.float64) * pf[:, r].astype(np.float64) + acc.astype(np.float64)).astype(np.float32)
    want = act_tensor(acc, ctx)
    assert torch.equal(h2.cpu(), want.cpu())


@pytest.mark.parametrize("bits", [4, 8])
def test_grouped_moe_production_shape(nv, ctx_bf16, bits):
    say("prefill grouped moe production", bits)
    # 4096 tokens x top-8 of 256 experts, D 2048, F 512, Zipf routing; the oracle checks a
    # sample of tokens, the rest is covered by linearity below.
    d, f, E, k, tokens = 2048, 512, 256, 8, 4096
    rng = np.random.default_rng(77 + bits)
    off, stride = nv.expert_offsets(d, f, bits)
    gen = torch.Generator(device="cuda").manual_seed(5 + bits)
    pool = torch.empty((E, stride), dtype=torch.uint8, device="cuda")
    for rows_, n, wo, so, bo in ((f, d, off.gate_w, off.gate_s, off.gate_b), (f, d, off.up_w, off.up_s, off.up_b),
                                 (d, f, off.down_w, off.down_s, off.down_b)):
        wmat = torch.empty((E * rows_, n), dtype=torch.bfloat16, device="cuda").normal_(0.0, 0.03, generator=gen)
        p, s, b = nv.quantize_affine(ctx_bf16, wmat, bits)
        wb, mb = rows_ * n * bits // 8, rows_ * n // 32
        pool[:, wo:wo + wb] = p.view(E, wb)
        pool[:, so:so + mb] = s.view(torch.uint8).view(E, mb)
        pool[:, bo:bo + mb] = b.view(torch.uint8).view(E, mb)
        del wmat, p, s, b
    x = O.round_bf16(gauss(rng, (tokens, d)))
    idx, w = _zipf_routes(rng, tokens, E, k)
    xd, idxd, wd = act_tensor(x, ctx_bf16), dev(idx.view(np.int32)), dev(w.view(np.int16))
    grouping, moe, red = nv.PrefillMoEGrouping(ctx_bf16), nv.PrefillGroupedRoutedMoE(ctx_bf16, bits), nv.PrefillMoE(ctx_bf16)
    routes = grouping.group_routes(idxd, wd, E)
    partials, _ = moe.encode(pool, off, xd, d, f, routes)
    h2 = red.encode_reduce_token_major(partials, wd, tokens, k, d)
    torch.cuda.synchronize()
    _check_routes(routes, O.group_pairs(O.make_pairs(idx, w), tokens, k, E, 16))
    sel = np.sort(rng.choice(tokens, 24, replace=False))
    blobs = pool.cpu().numpy()
    want = O.prefill_moe(blobs, bits, x[sel], d, f, idx[sel], w[sel])
    got = act_np(h2)
    assert O.rel_error(got[sel], want) <= TOL_ACT
    assert np.isfinite(got).all()
    # a token's row does not depend on what else is in the batch: the first 512 tokens alone
    r2 = grouping.group_routes(idxd[:512].contiguous(), wd[:512].contiguous(), E)
    p2, _ = moe.encode(pool, off, xd[:512].contiguous(), d, f, r2)
    h2b = red.encode_reduce_token_major(p2, wd[:512].contiguous(), 512, k, d)
    torch.cuda.synchronize()
    assert torch.equal(h2b, h2[:512])


# ------------------------------------------------------------------ dense QMM
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (16, 1000, 2048), (130, 384, 192), (300, 2048, 512)])
def test_dense_qmm_matches_oracle(nv, ctx, bits, m, n, k):
    say("dense qmm", ctx.act, bits, m, n, k)
    # MPPPrefillInt4QMMTests.swift:190-201 bars: max-abs <= 0.03, relative <= 1e-3 of an fp16 path
    # against its own fp16 oracle; here the bar is the 16-bit class, 1e-2 of max|ref|.
    rng = np.random.default_rng(m * 7 + n + k + bits)
    w = gauss(rng, (n, k), 0.05)
    p, s, b = O.quantize_affine(w, bits)
    xs = gauss(rng, (m, k))
    x = O.round_bf16(xs) if ctx.act == 0 else O.f16_to_float(O.f16_bits(xs))
    y = nv.MPPPrefillInt4QMM(ctx, bits).encode(dev(p), dev(s.view(np.int16)), dev(b.view(np.int16)),
                                               act_tensor(x, ctx), n, k)
    torch.cuda.synchronize()
    want = np.stack([O.affine_gemv(p, s, b, x[t], bits) for t in range(m)])
    assert O.rel_error(act_np(y), want) <= TOL_ACT


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m", [16, 17, 33, 48, 65, 128, 129])
@pytest.mark.parametrize("n,k", [(200, 320), (264, 256)])
def test_dense_qmm_every_row_tile_count(nv, ctx_bf16, bits, m, n, k):
    """One, two, three..four and five..eight 16-row tiles take different loop bodies; k = 320 has
    an odd number of groups (scale rows on 2-byte boundaries, half a super-step at the end) and
    n = 200 / 264 leave a last column block that sticks out."""
    say("dense qmm row tiles", bits, m, n, k)
    rng = np.random.default_rng(m * 13 + n + k + bits)
    w = gauss(rng, (n, k), 0.05)
    p, s, b = O.quantize_affine(w, bits)
    x = O.round_bf16(gauss(rng, (m, k)))
    y = nv.MPPPrefillInt4QMM(ctx_bf16, bits).encode(dev(p), dev(s.view(np.int16)), dev(b.view(np.int16)),
                                                    act_tensor(x, ctx_bf16), n, k)
    torch.cuda.synchronize()
    want = np.stack([O.affine_gemv(p, s, b, x[t], bits) for t in range(m)])
    assert O.rel_error(act_np(y), want) <= TOL_ACT


@pytest.mark.parametrize("bits,m", [(4, 1056), (4, 1280 + 64), (8, 1024 + 40), (4, 1024 + 96)])
def test_projection_with_a_sliver_of_rows_at_the_end(nv, ctx, bits, m):
    """A projection over many input rows whose matrix ends in a few rows past the last full block of the
    matrix-core product (the concatenated input projections of a gated-DeltaNet layer end in 2 x 32 rows):
    every column against the oracle, and the last partial block's columns on their own."""
    say("projection with sliver", ctx.act, bits, m)
    n, tokens = 512, 300
    rng = np.random.default_rng(m + bits)
    w = gauss(rng, (m, n), 0.05)
    p, s, b = O.quantize_affine(w, bits)
    xs = gauss(rng, (tokens, n))
    x = O.round_bf16(xs) if ctx.act == 0 else O.f16_to_float(O.f16_bits(xs))
    y = nv.affine_gemv(ctx, dev(p), dev(s.view(np.int16)), dev(b.view(np.int16)), bits, act_tensor(x, ctx), m, n)
    torch.cuda.synchronize()
    got = act_np(y)
    want = np.stack([O.affine_gemv(p, s, b, x[t], bits) for t in range(0, tokens, 7)])
    assert O.rel_error(got[::7], want) <= TOL_ACT
    tail = m % (256 if bits == 4 else 128)
    assert O.rel_error(got[::7, m - tail:], want[:, m - tail:]) <= TOL_ACT        # the sliver on its own


def test_gemm_refuses_operands_beyond_32_bit_offsets(nv, ctx_bf16):
    say("gemm 4 GiB limits")
    q = nv.MPPPrefillInt4QMM(ctx_bf16, 4)
    p = torch.zeros((64, 32), dtype=torch.uint8, device="cuda")
    s = torch.zeros((64, 1), dtype=torch.int16, device="cuda")
    x = torch.zeros((4, 64), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((4, 64), dtype=torch.bfloat16, device="cuda")
    # 2^26 rows at a stride of 64 elements would put the last row past 4 GiB: refused before any launch
    rc = nv.lib.nvmai_hip_affine_qmm(ctx_bf16.handle, None, p.data_ptr(), s.data_ptr(), s.data_ptr(), 4,
                                     x.data_ptr(), 64, y.data_ptr(), 64, 1 << 26, 64, 64)
    assert rc == -2                                              # NVMAI_ERR_UNSUPPORTED


def test_dense_qmm_rejects_bad_arguments(nv, ctx_bf16):
    say("dense qmm errors")
    q = nv.MPPPrefillInt4QMM(ctx_bf16, 4)
    p = torch.zeros((64, 48), dtype=torch.uint8, device="cuda")
    s = torch.zeros((64, 1), dtype=torch.int16, device="cuda")
    x = torch.zeros((4, 96), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(nv.NvmaiError) as e:                       # k not a multiple of 64
        q.encode(p, s, s, x, 64, 96)
    assert e.value.name == "invalid_arg"
    with pytest.raises(nv.NvmaiError):
        nv.MPPPrefillInt4QMM(ctx_bf16, 3)


def test_grouped_moe_on_a_failed_grouping_returns_zeros_and_the_error(nv, ctx_bf16):
    # An expert id out of range: the reference throws expertOutOfRange before any compute
    # (PrefillMoEGrouping.swift:121-138).  Here the failure is found on the device: the products do
    # not run, the route partials (handed in full of junk) come back as zeros, so the reduce gives
    # zeros, and validate() raises the reference's error with the first failing pair.
    say("prefill grouped moe on a failed grouping")
    ctx, d, f, E, k, tokens, bits = ctx_bf16, 128, 64, 4, 2, 40, 4
    rng = np.random.default_rng(11)
    blobs = np.stack([O.pack_expert(gauss(rng, (f, d), .05), gauss(rng, (f, d), .05), gauss(rng, (d, f), .05), bits)
                      for _ in range(E)])
    idx, w = _zipf_routes(rng, tokens, E, k)
    idx[17, 1] = E + 3
    off, _ = nv.expert_offsets(d, f, bits)
    routes = nv.PrefillMoEGrouping(ctx).group_routes(dev(idx.view(np.int32)), dev(w.view(np.int16)), E)
    junk = torch.full((tokens * k, d), 7.0, dtype=ctx.dtype, device="cuda")
    partials, _ = nv.PrefillGroupedRoutedMoE(ctx, bits).encode(dev(blobs), off, act_tensor(gauss(rng, (tokens, d)), ctx),
                                                               d, f, routes, route_partials=junk)
    h2 = nv.PrefillMoE(ctx).encode_reduce_token_major(partials, dev(w.view(np.int16)), tokens, k, d)
    torch.cuda.synchronize()
    assert not act_np(partials).any() and not act_np(h2).any()
    with pytest.raises(nv.PrefillMoEGroupingError) as e:
        routes.validate()
    assert e.value.name == "expertOutOfRange" and e.value.pair_index == 17 * k + 1


# ------------------------------------------------------------------ streamed tiles (experts bound one by one)
def _scattered_views(blobs, expert_ids, gap=4096, first=256):
    """Each expert's blob copied to its own place inside one big device buffer, at a nonzero
    16-byte-aligned offset (streamedViewsWithNonzeroOffsets)."""
    stride = blobs.shape[1]
    pitch = (stride + gap + 15) // 16 * 16
    buf = torch.zeros(first + pitch * len(expert_ids), dtype=torch.uint8, device="cuda")
    views = []
    for i, e in enumerate(expert_ids):
        off = first + i * pitch
        buf[off:off + stride] = dev(blobs[e])
        views.append((buf, off))
    return buf, views


def _route_partials_oracle(blobs, bits, x, d, f, idx, act):
    """cpuSyntheticRoutePartials (PrefillGroupedRoutedMoETests.swift:293-378): per (token, rank) the
    expert's FFN of the token's row, through the oracle's single-route call."""
    tokens, k = idx.shape
    one = O.f16_bits(np.ones((1, 1), np.float32))
    out = np.zeros((tokens * k, d), np.float32)
    for t in range(tokens):
        for r in range(k):
            out[t * k + r] = O.prefill_moe(blobs, bits, x[t:t + 1], d, f, idx[t:t + 1, r:r + 1], one)[0]
    return out


@pytest.mark.parametrize("bits", [4, 8])
def test_streamed_tile_matches_reference_case(nv, ctx, bits):
    # streamedBatchedMatchesReferenceAcrossPartialMicrobatch (PrefillGroupedRoutedMoETests+Execution.swift:8-110):
    # d = f = 64, three rows, top-2 of 16 experts, every expert bound through a view at a nonzero offset
    say("prefill streamed tile, reference case", ctx.act, bits)
    d = f = 64
    rows, k, E = 3, 2, 16
    idx = np.array([[2, 0], [1, 2], [0, 1]], np.uint32)
    w = O.f16_bits(np.ones((rows, k), np.float32))

    def mat(expert, role, r, c):                     # makeSyntheticExpertPool's closed form
        i, j = np.meshgrid(np.arange(r), np.arange(c), indexing="ij")
        return ((expert + 1) * 1e-3 + (role + 1) * 3e-3 + ((i % 7) - 3) * 4e-4 + ((j % 11) - 5) * 2e-4).astype(np.float32)
    blobs = np.stack([O.pack_expert(mat(e, 0, f, d), mat(e, 1, f, d), mat(e, 2, d, f), bits) for e in range(E)])
    hidden = np.array([(i % 17) - 8 for i in range(rows * d)], np.float32).reshape(rows, d)
    off, _ = nv.expert_offsets(d, f, bits)
    routes = nv.PrefillMoEGrouping(ctx).group_routes(dev(idx.view(np.int32)), dev(w.view(np.int16)), E)
    torch.cuda.synchronize()
    routes.validate()
    expert_ids = list(range(E))
    buf, views = _scattered_views(blobs, expert_ids)
    binding = nv.PrefillStreamedTileBinding(expert_ids, views)
    n = rows * k
    params = nv.prefill_streamed_params(0, n, d, f, k, d, binding, off)
    partials = torch.full((n, d), -77.0, dtype=ctx.dtype, device="cuda")
    act = torch.zeros((n, f), dtype=ctx.dtype, device="cuda")
    err = torch.full((2,), 9, dtype=torch.int32, device="cuda")
    nv.PrefillGroupedRoutedMoE(ctx, bits).encode_streamed_batched(act_tensor(hidden, ctx), routes.sorted_pairs, partials,
                                                                 act, binding, params, err=err)
    torch.cuda.synchronize()
    assert err.tolist() == [0, 0]
    want = _route_partials_oracle(blobs, bits, hidden, d, f, idx, ctx.act)
    assert O.rel_error(act_np(partials), want) <= TOL_ACT
    assert all(o > 0 for _, o in views)
    binding.validate_covers_pairs(u32(routes.sorted_pairs).reshape(-1, 4)[:, 1].tolist(), 0, n)


@pytest.mark.parametrize("bits", [4, 8])
def test_streamed_tiles_equal_the_resident_pool_call(nv, ctx_bf16, bits):
    # tile after tile (at most 16 experts each, bound from scattered copies, only the tile's pair
    # range computed) gives the bits of the one call over the resident pool; a tile that leaves an
    # expert of its range unbound computes nothing and reports the first such pair
    say("prefill streamed tiles vs pool", bits)
    ctx = ctx_bf16
    rng = np.random.default_rng(31 + bits)
    d, f, E, k, tokens = 256, 128, 40, 4, 700
    mats = [(gauss(rng, (f, d), 0.05), gauss(rng, (f, d), 0.05), gauss(rng, (d, f), 0.05)) for _ in range(E)]
    blobs = np.stack([O.pack_expert(*m, bits) for m in mats])
    x = O.round_bf16(gauss(rng, (tokens, d)))
    idx, w = _zipf_routes(rng, tokens, E, k)
    off, stride = nv.expert_offsets(d, f, bits)
    routes = nv.PrefillMoEGrouping(ctx).group_routes(dev(idx.view(np.int32)), dev(w.view(np.int16)), E)
    moe = nv.PrefillGroupedRoutedMoE(ctx, bits)
    xd = act_tensor(x, ctx)
    want, want_act = moe.encode(dev(blobs), off, xd, d, f, routes)
    torch.cuda.synchronize()
    info = routes.validate()
    groups = u32(routes.groups).reshape(-1, 3)[:info[0]].tolist()
    tiles = u32(routes.tiles).reshape(-1, 4)[:info[1]].tolist()
    assert len(tiles) == 3                                     # 40 experts in tiles of 16
    n = tokens * k
    got = torch.zeros((n, d), dtype=ctx.dtype, device="cuda")
    act = torch.zeros((n, f), dtype=ctx.dtype, device="cuda")
    err = torch.zeros(2, dtype=torch.int32, device="cuda")
    lifetime = nv.PrefillStreamedTileSlotLifetime()
    keep = []
    for t, tile in enumerate(tiles):
        ids = nv.PrefillStreamedTileBinding.expert_ids_for_tile(t, groups, tiles)
        lifetime.begin(t, list(range(len(ids))))
        buf, views = _scattered_views(blobs, ids, gap=16 * (t + 1))
        keep.append(buf)
        binding = nv.PrefillStreamedTileBinding(ids, views)
        params = nv.prefill_streamed_params(tile[2], tile[3], d, f, k, xd.stride(0), binding, off)
        moe.encode_streamed_batched(xd, routes.sorted_pairs, got, act, binding, params, err=err)
        torch.cuda.synchronize()
        assert err.tolist() == [0, 0]
        lifetime.complete(t)
    assert torch.equal(got, want) and torch.equal(act, want_act)
    # the second tile with its last expert left out
    ids = nv.PrefillStreamedTileBinding.expert_ids_for_tile(1, groups, tiles)
    buf, views = _scattered_views(blobs, ids[:-1])
    binding = nv.PrefillStreamedTileBinding(ids[:-1], views)
    params = nv.prefill_streamed_params(tiles[1][2], tiles[1][3], d, f, k, xd.stride(0), binding, off)
    before = got.clone()
    moe.encode_streamed_batched(xd, routes.sorted_pairs, got, act, binding, params, err=err)
    torch.cuda.synchronize()
    first_unbound = groups[tiles[1][0] + tiles[1][1] - 1][1]
    assert err.tolist() == [1, first_unbound] and torch.equal(got, before)
    with pytest.raises(nv.PrefillGroupedRoutedMoEError):
        binding.validate_covers_pairs(u32(routes.sorted_pairs).reshape(-1, 4)[:, 1].tolist(), tiles[1][2], tiles[1][3])
    # argument checks of the entry point: a pair range past the end, a misaligned blob
    bad = nv.prefill_streamed_params(n - 4, 8, d, f, k, xd.stride(0), binding, off)
    with pytest.raises(nv.NvmaiError):
        moe.encode_streamed_batched(xd, routes.sorted_pairs, got, act, binding, bad)
    crooked = nv.PrefillStreamedTileBinding(ids[:1], [(buf, 257)])
    with pytest.raises(nv.NvmaiError):
        moe.encode_streamed_batched(xd, routes.sorted_pairs, got, act, crooked,
                                    nv.prefill_streamed_params(0, 4, d, f, k, xd.stride(0), crooked, off))
