"""GPU parity: quantizer, affine GEMV, router, routed phases, shared expert and the fused
decode layer, each called through the C ABI and compared with the CPU oracle.

Bars: codes / scale bits / routing indices / router logits bit-exact; fp32 outputs within
2e-3 and 16-bit outputs within 1e-2 of the oracle, both as max|diff| / max|ref|
(RelError.swift:5-16)."""
import math

import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import act_np, act_tensor, dev, gauss, round_act, say, u16, u32

pytestmark = pytest.mark.gpu

TOL_F32 = 2e-3
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


# ------------------------------------------------------------------ quantizer
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(64, 128), (512, 2048), (2048, 512), (3, 2816)])
def test_quantizer_codes_bit_exact(nv, ctx_bf16, bits, shape):
    say("quantizer", bits, shape)
    rng = np.random.default_rng(100 + bits)
    w = gauss(rng, shape, 0.02)
    w[0, :64] = 0.42                       # flat group
    w[1, 64:128] = np.linspace(1, 2, 64)   # positive-only group
    for as_bf16 in (False, True):
        wh = O.round_bf16(w) if as_bf16 else w
        wd = dev(wh).to(torch.bfloat16) if as_bf16 else dev(wh)
        p, s, b = nv.quantize_affine(ctx_bf16, wd, bits)
        torch.cuda.synchronize()
        po, so, bo = O.quantize_affine(wh, bits)
        assert np.array_equal(p.cpu().numpy(), po)
        assert np.array_equal(u16(s), so) and np.array_equal(u16(b), bo)
        codes, vals = nv.dequantize_affine(ctx_bf16, p, s, b, bits)
        torch.cuda.synchronize()
        assert np.array_equal(codes.cpu().numpy(), O.unpack_codes(po, bits))
        want = O.round_bf16(O.dequantize_affine(po, so, bo, shape[1], bits)).reshape(-1)
        assert np.array_equal(act_np(vals), want)


# ------------------------------------------------------------------ GEMV
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,n,tokens", [(64, 128, 1), (512, 2048, 1), (2048, 512, 1), (100, 2816, 3),
                                        (512, 2048, 7), (2048, 512, 5), (37, 1024, 2), (64, 192, 1)])
def test_affine_gemv_matches_oracle(nv, ctx, bits, m, n, tokens):
    say("gemv", ctx.act, bits, m, n, tokens)
    rng = np.random.default_rng(m * 7 + n + bits)
    p, s, b = O.quantize_affine(gauss(rng, (m, n), 0.05), bits)
    x = round_act(gauss(rng, (tokens, n)), ctx.act)
    want = np.stack([O.affine_gemv(p, s, b, x[t], bits) for t in range(tokens)])
    pd, sd, bd = dev(p), dev(s.view(np.int16)), dev(b.view(np.int16))
    y32 = nv.affine_gemv(ctx, pd, sd, bd, bits, act_tensor(x, ctx), m, n, out_f32=True)
    y16 = nv.affine_gemv(ctx, pd, sd, bd, bits, act_tensor(x, ctx), m, n)
    torch.cuda.synchronize()
    assert O.rel_error(y32.cpu().numpy(), want) < TOL_F32
    assert O.rel_error(act_np(y16), want) < TOL_ACT


@pytest.mark.parametrize("bits", [4, 8])
def test_affine_gemv_small_batch_on_the_matrix_cores(nv, ctx, bits):
    # 5 .. 32 input rows against rows of whole 512-code stages: the matrix is read once for all of
    # them.  Ragged row counts (last block, last wave, last four rows), one and two token tiles,
    # one and two input panels, padded output rows, an all-zero input row and one with a huge entry
    rng = np.random.default_rng(300 + bits)
    for m, n, tokens in [(64, 512, 5), (100, 1024, 16), (203, 2048, 17), (2048, 4096, 9), (1001, 2048, 32),
                         (130, 4096, 31), (12352, 2048, 16)]:
        say("gemv mfma", ctx.act, bits, m, n, tokens)
        p, s, b = O.quantize_affine(gauss(rng, (m, n), 0.05), bits)
        x = gauss(rng, (tokens, n))
        x[1] = 0.0
        x[2, 7] = 3.0e4 if ctx.act == 1 else 1.0e30
        x[3] *= 1e-3
        x = round_act(x, ctx.act)
        want = np.stack([O.affine_gemv(p, s, b, x[t], bits) for t in range(tokens)])
        stride = m + 12
        y = torch.full((tokens, stride), 7.0, dtype=ctx.dtype, device="cuda")
        yf = torch.full((tokens, stride), 7.0, dtype=torch.float32, device="cuda")
        pd, sd, bd = dev(p), dev(s.view(np.int16)), dev(b.view(np.int16))
        nv.affine_gemv(ctx, pd, sd, bd, bits, act_tensor(x, ctx), m, n, y=y, y_f32=yf)
        torch.cuda.synchronize()
        got32, got16 = yf[:, :m].cpu().numpy(), act_np(y[:, :m])
        for t in range(tokens):                         # per input row: a small row must not hide behind a large one
            assert O.rel_error(got32[t], want[t]) < TOL_F32, (m, n, tokens, t)
            if np.isfinite(round_act(want[t], ctx.act)).all():
                assert O.rel_error(got16[t], want[t]) < TOL_ACT, (m, n, tokens, t)
        assert not got32[1].any()
        assert (yf[:, m:] == 7.0).all() and (y[:, m:].float() == 7.0).all()     # padding untouched
        # the same product through the row engine (four rows at a time): both paths within the bar of each other
        y4 = torch.cat([nv.affine_gemv(ctx, pd, sd, bd, bits, act_tensor(x[t0:t0 + 4], ctx), m, n, out_f32=True)
                        for t0 in range(0, tokens, 4)])
        torch.cuda.synchronize()
        assert O.rel_error(got32, y4.cpu().numpy()) < TOL_F32


@pytest.mark.parametrize("bits", [4, 8])
def test_affine_gemv_both_outputs_padded_stride(nv, ctx, bits):
    # 16-bit and fp32 results in one call, rows of the outputs further apart than m; shapes with a
    # single-launch instantiation (any chunk count 16 / 32 / 64 / 128) and one without (n = 192)
    rng = np.random.default_rng(90 + bits)
    per = 128 // bits
    for m, n, tokens in [(70, 16 * per, 1), (130, 32 * per, 3), (64, 64 * per, 4), (33, 128 * per, 9), (40, 192, 2)]:
        say("gemv padded", ctx.act, bits, m, n, tokens)
        p, s, b = O.quantize_affine(gauss(rng, (m, n), 0.05), bits)
        x = round_act(gauss(rng, (tokens, n)), ctx.act)
        want = np.stack([O.affine_gemv(p, s, b, x[t], bits) for t in range(tokens)])
        stride = m + 24
        y = torch.full((tokens, stride), 7.0, dtype=ctx.dtype, device="cuda")
        yf = torch.full((tokens, stride), 7.0, dtype=torch.float32, device="cuda")
        nv.affine_gemv(ctx, dev(p), dev(s.view(np.int16)), dev(b.view(np.int16)), bits, act_tensor(x, ctx), m, n,
                       y=y, y_f32=yf)
        torch.cuda.synchronize()
        assert O.rel_error(yf[:, :m].cpu().numpy(), want) < TOL_F32
        assert O.rel_error(act_np(y[:, :m]), want) < TOL_ACT
        assert (yf[:, m:] == 7.0).all() and (y[:, m:].float() == 7.0).all()     # padding untouched


def test_gemv_bitstream_known_answer(nv, ctx_bf16):
    # AffineQuantTests.swift:35-56: value=(row*11+col*3)&mask, scale 1, bias 0, x=1 => sum(values)
    for bits in (4, 8):
        say("gemv-bitstream", bits)
        rows, cols = 3, 128
        mask = (1 << bits) - 1
        values = np.array([[(r * 11 + c * 3) & mask for c in range(cols)] for r in range(rows)])
        packed = np.zeros((rows, cols * bits // 8), np.uint8)
        for r in range(rows):
            for c in range(cols):
                packed[r, c * bits // 8] |= (int(values[r, c]) << ((c * bits) % 8)) & 0xFF
        one = np.full((rows, 2), 0x3F80, np.uint16).view(np.int16)
        zero = np.zeros((rows, 2), np.int16)
        x = torch.ones((1, cols), dtype=torch.bfloat16, device="cuda")
        y = nv.affine_gemv(ctx_bf16, dev(packed), dev(one), dev(zero), bits, x, rows, cols, out_f32=True)
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy()[0], values.sum(1).astype(np.float32))


def test_reference_signature_host_gemv(nv, ctx_bf16):
    say("nvmai_int4_affine_gemv host signature")
    rng = np.random.default_rng(11)
    for rows, n in [(512, 2048), (2048, 512), (5, 192)]:
        w = gauss(rng, (rows, n), 0.02)
        p, s, b = O.quantize_affine(w, 4)
        x = gauss(rng, (n,))
        got = nv.int4_affine_gemv(p, s, b, x, rows, n)
        want = O.affine_gemv(p, s, b, x, 4)
        assert O.rel_error(got, want) <= TOL_F32
    # a contract violation cannot be returned: it must not look like a result
    bad = nv.int4_affine_gemv(p, s, b, x[:100], 5, 100)
    assert np.isnan(bad).all()


def test_read_probe_runs_and_checks_its_arguments(nv, ctx_bf16):
    # the measuring stick of bench.py: reads a buffer and writes nothing; sizes with a ragged end, the empty
    # buffer, and the refusals (misaligned start, a size that is no multiple of 16)
    say("read probe")
    buf = torch.full(((1 << 20) + 48,), 7, dtype=torch.uint8, device="cuda")
    for n in (0, 16, 1008, 8192, 65536 + 16, 1 << 20, (1 << 20) + 48):
        ctx_bf16.read_probe(buf[:n])
    torch.cuda.synchronize()
    assert bool((buf == 7).all())
    with pytest.raises(nv.NvmaiError) as e:
        ctx_bf16.read_probe(buf[8:8 + 64])
    assert e.value.name == "alignment"
    with pytest.raises(nv.NvmaiError) as e:
        ctx_bf16.read_probe(buf[:40])
    assert e.value.name == "alignment"


def test_gemv_rejects_bad_arguments(nv, ctx_bf16):
    say("gemv-errors")
    w = torch.zeros(64 * 128, dtype=torch.uint8, device="cuda")
    s = torch.zeros(64 * 2, dtype=torch.int16, device="cuda")
    x = torch.zeros((1, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(nv.NvmaiError) as e:
        nv.affine_gemv(ctx_bf16, w, s, s, 6, x, 64, 128)
    assert e.value.name == "unsupported"
    with pytest.raises(nv.NvmaiError) as e:
        nv.affine_gemv(ctx_bf16, w, s, s, 4, x[:, :100], 64, 100)       # n % 64 != 0
    assert e.value.name == "invalid_arg"
    with pytest.raises(nv.NvmaiError) as e:
        nv.affine_gemv(ctx_bf16, w[1:], s, s, 8, x, 8, 128)             # misaligned weights
    assert e.value.name == "alignment"


# ------------------------------------------------------------------ router
def _router_case(nv, ctx, kind, E, D, tokens, k, rng, eff=None, pes=None, w=None, x=None):
    if w is None:
        w = O.round_bf16(gauss(rng, (E, D), 0.02))
    if x is None:
        x = round_act(gauss(rng, (tokens, D)), ctx.act)
    if kind == 16:
        host = (O.bf16_bits(w), None, None)
        desc = nv.rows_desc(16, dev(host[0].view(np.int16)))
    else:
        host = O.quantize_affine(w, kind)
        desc = nv.rows_desc(kind, dev(host[0]), dev(host[1].view(np.int16)), dev(host[2].view(np.int16)))
    effd = None if eff is None else dev(eff.view(np.int16))
    pesd = None if pes is None else dev(pes.view(np.int16))
    moe = nv.MoE(ctx)
    idx, wt, logits = moe.encode_router(desc, act_tensor(x, ctx), E, D, k, effd, pesd, want_logits=True)
    torch.cuda.synchronize()
    for t in range(x.shape[0]):
        lo = O.router_logits(kind, host[0], host[1], host[2], x[t], eff)
        assert np.array_equal(logits[t].cpu().numpy().view(np.uint32), lo.view(np.uint32)), "logits bits"
        io, wo = O.router_topk(lo, k, pes)
        assert np.array_equal(u32(idx[t]), io)
        assert np.abs(act_np(wt[t]) - O.f16_to_float(wo)).max() < 5e-3     # RouterTopKTests.swift:43
        assert np.abs(u16(wt[t]).astype(np.int32) - wo.astype(np.int32)).max() <= 1   # fp16 ulp
    return idx, wt


@pytest.mark.parametrize("kind", [16, 8, 4])
def test_router_indices_and_logits_bit_exact(nv, ctx, kind):
    rng = np.random.default_rng(kind)
    for E, D, tokens, k in [(256, 2048, 9, 8), (16, 128, 3, 8), (100, 512, 2, 4), (256, 2048, 1, 8)]:
        say("router", ctx.act, kind, E, D, tokens, k)
        _router_case(nv, ctx, kind, E, D, tokens, k, rng)
    say("router scales", kind)
    eff = O.bf16_bits(rng.uniform(0.5, 1.5, 128).astype(np.float32) / np.float32(math.sqrt(128)))
    pes = O.bf16_bits(rng.uniform(0.6, 1.4, 16).astype(np.float32))
    _router_case(nv, ctx, kind, 16, 128, 4, 8, rng, eff, pes)


@pytest.mark.parametrize("kind", [16, 8, 4])
def test_router_many_tokens_same_bits(nv, ctx, kind):
    # 64 tokens and more take the register-tiled kernel: same sums in the same order, so the same bits
    rng = np.random.default_rng(100 + kind)
    # (one row: the form the shared expert's gate row takes, a half-wave per token)
    for E, D, tokens, k in [(256, 2048, 150, 8), (100, 512, 70, 4), (20, 192, 64, 8), (33, 2048, 97, 2),
                            (1, 2048, 131, 1), (1, 512, 64, 1), (1, 4096, 70, 1)]:
        say("router tiled", ctx.act, kind, E, D, tokens, k)
        _router_case(nv, ctx, kind, E, D, tokens, k, rng)
    say("router tiled scales", kind)
    eff = O.bf16_bits(rng.uniform(0.5, 1.5, 256).astype(np.float32) / np.float32(math.sqrt(256)))
    pes = O.bf16_bits(rng.uniform(0.6, 1.4, 40).astype(np.float32))
    _router_case(nv, ctx, kind, 40, 256, 81, 8, rng, eff, pes)


def test_router_many_tokens_padded_stride(nv, ctx_bf16):
    say("router tiled padded stride")
    E, D, T, k = 48, 256, 75, 8
    rng = np.random.default_rng(78)
    stride = D + 13                                   # rows not 16-byte aligned: element loads into LDS
    w = O.round_bf16(gauss(rng, (E, D), 0.04))
    host = O.quantize_affine(w, 8)
    desc = nv.rows_desc(8, dev(host[0]), dev(host[1].view(np.int16)), dev(host[2].view(np.int16)))
    block = np.full((T, stride), -31.0, np.float32)
    block[:, :D] = O.round_bf16(rng.uniform(-1, 1, (T, D)).astype(np.float32))
    hd = dev(block).to(torch.bfloat16)
    idx, wt, logits = nv.MoE(ctx_bf16).encode_router(desc, hd[:, :D], E, D, k, want_logits=True)
    torch.cuda.synchronize()
    for t in range(T):
        lo = O.router_logits(8, host[0], host[1], host[2], block[t, :D])
        assert np.array_equal(logits[t].cpu().numpy().view(np.uint32), lo.view(np.uint32))
        assert np.array_equal(u32(idx[t]), O.router_topk(lo, k)[0])


def test_router_padded_hidden_stride(nv, ctx_bf16):
    # PrefillRouterTests.swift:33-95: rows of `hidden` are d + 13 apart and the padding is left alone
    say("router padded stride")
    E, D, T, k = 16, 128, 3, 8
    rng = np.random.default_rng(77)
    stride = D + 13
    w = O.round_bf16(gauss(rng, (E, D), 0.04) + np.arange(E, dtype=np.float32)[:, None] * np.float32(0.015))
    host = O.quantize_affine(w, 8)
    desc = nv.rows_desc(8, dev(host[0]), dev(host[1].view(np.int16)), dev(host[2].view(np.int16)))
    block = np.full((T, stride), -31.0, np.float32)
    block[:, :D] = O.round_bf16(rng.uniform(-1, 1, (T, D)).astype(np.float32))
    hd = dev(block).to(torch.bfloat16)
    idx, wt = nv.MoE(ctx_bf16).encode_router(desc, hd[:, :D], E, D, k)
    torch.cuda.synchronize()
    for t in range(T):
        io, wo = O.router_topk(O.router_logits(8, host[0], host[1], host[2], block[t, :D]), k)
        assert np.array_equal(u32(idx[t]), io)
        assert np.abs(act_np(wt[t]) - O.f16_to_float(wo)).max() < 5e-3
    assert np.array_equal(act_np(hd)[:, D:], block[:, D:])


def test_router_near_tie_and_exact_ties(nv, ctx_bf16):
    # RouterTopKTests.swift:46-70: gains 0.5 and 0.5*(1+1e-4) must order like the reference
    say("router near tie")
    E, D = 16, 128
    g = O.SplitMix64(0x71E0F4A)
    pattern = g.uniform_array(D, 0.2, 1.0)
    hidden = O.round_bf16(g.uniform_array(D, 0.5, 1.5))[None, :]
    gains = np.array([1.0 - e * 0.05 for e in range(7)] + [0.5, 0.5 * (1 + 1e-4)] +
                     [0.4 - (e - 9) * 0.02 for e in range(9, E)], np.float32)
    w = np.stack([pattern * gn for gn in gains]).astype(np.float32)
    idx, _ = _router_case(nv, ctx_bf16, 8, E, D, 1, 8, None, w=w, x=hidden)
    assert list(u32(idx[0])[:7]) == list(range(7))
    say("router exact ties")
    w = np.tile(O.round_bf16(gauss(np.random.default_rng(1), (1, 256), 0.05)), (64, 1))  # identical rows
    idx, wt = _router_case(nv, ctx_bf16, 16, 64, 256, 2, 8, np.random.default_rng(2), w=w)
    assert list(u32(idx[0])) == list(range(8)) and np.all(act_np(wt) == 0.125)


# ------------------------------------------------------------------ routed phases
def _constant_blob(d, f, bits):
    off = O.expert_offsets(d, f, bits)
    blob = np.zeros(int(off[9]), np.uint8)
    bf = lambda v: int(np.float32(v).view(np.uint32)) >> 16
    for o, count, v in ((off[2], f * d // 64, 1 / 64), (off[5], f * d // 64, 0.5 / 64),
                        (off[8], d * f // 64, 1 / 64)):
        blob[int(o):int(o) + 2 * count].view(np.uint16)[:] = bf(v)
    return blob


@pytest.mark.parametrize("bits", [4, 8])
def test_routed_pipeline_constant_blob_known_answer(nv, ctx, bits):
    # MoEFusedFFNTests.swift:17-54: x=1, eight experts at weight 0.125 => silu(2) everywhere
    say("constant blob", ctx.act, bits)
    d, f, k = 128, 64, 8
    blobs = [dev(_constant_blob(d, f, bits)) for _ in range(k)]
    off, _ = nv.expert_offsets(d, f, bits)
    moe = nv.MoE(ctx, bits)
    x = torch.ones(d, dtype=ctx.dtype, device="cuda")
    acts = torch.zeros((k, f), dtype=torch.float32, device="cuda")
    w = torch.full((k,), 0.125, dtype=torch.float16, device="cuda")
    res = torch.zeros(d, dtype=ctx.dtype, device="cuda")
    y = torch.empty(d, dtype=ctx.dtype, device="cuda")
    moe.encode_routed_phase1(blobs, off, x, acts, d, f, k)
    moe.encode_routed_phase2_reduce(blobs, off, acts, w, res, y, d, f, k)
    torch.cuda.synchronize()
    assert np.abs(act_np(y) - 2.0 / (1.0 + math.exp(-2.0))).max() < 0.01


def _random_blobs(rng, d, f, bits, count, std=0.05):
    mk = lambda r, c: O.round_bf16(gauss(rng, (r, c), std))
    return np.stack([O.pack_expert(mk(f, d), mk(f, d), mk(d, f), bits) for _ in range(count)])


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("d,f", [(128, 64), (2048, 512), (1024, 256), (192, 128)])
def test_routed_phases_match_oracle_and_split_equals_full(nv, ctx, bits, d, f):
    say("routed phases", ctx.act, bits, d, f)
    rng = np.random.default_rng(d + f + bits)
    k = 8
    host = _random_blobs(rng, d, f, bits, k, 0.05 if d < 1024 else 0.02)
    blobs = [dev(host[i]) for i in range(k)]
    off, stride = nv.expert_offsets(d, f, bits)
    assert stride == host.shape[1]
    x = round_act(gauss(rng, d), ctx.act)
    rw = O.f16_bits(rng.dirichlet(np.ones(k)).astype(np.float32))
    residual = round_act(gauss(rng, d, 0.1), ctx.act)
    want = residual.copy()
    for i in range(k):
        O.expert_ffn_accumulate(host[i], bits, x, d, f, float(O.f16_to_float(rw[i])), want)
    moe = nv.MoE(ctx, bits)
    xd = act_tensor(x, ctx)
    acts = torch.zeros((k, f), dtype=torch.float32, device="cuda")
    y = torch.empty(d, dtype=ctx.dtype, device="cuda")
    moe.encode_routed_phase1(blobs, off, xd, acts, d, f, k)
    moe.encode_routed_phase2_reduce(blobs, off, acts, dev(rw.view(np.float16)), act_tensor(residual, ctx), y, d, f, k)
    torch.cuda.synchronize()
    assert O.rel_error(act_np(y), want) < TOL_ACT
    # hit/miss split (MoEFusedFFNTests.swift:195-197): two subset launches == one full launch, bit for bit
    acts2 = torch.zeros_like(acts)
    hits = torch.tensor([0, 2, 3, 7], dtype=torch.int32, device="cuda")
    miss = torch.tensor([1, 4, 5, 6, 99], dtype=torch.int32, device="cuda")[:4]
    moe.encode_routed_phase1(blobs, off, xd, acts2, d, f, k, active_slots=hits)
    moe.encode_routed_phase1(blobs, off, xd, acts2, d, f, k, active_slots=miss)
    torch.cuda.synchronize()
    assert torch.equal(acts, acts2)
    # slots >= top_k are skipped
    acts3 = torch.full_like(acts, 7.0)
    moe.encode_routed_phase1(blobs, off, xd, acts3, d, f, k,
                             active_slots=torch.tensor([5, 8, 1000], dtype=torch.int32, device="cuda"))
    torch.cuda.synchronize()
    assert torch.equal(acts3[5], acts[5]) and bool((acts3[[0, 1, 2, 3, 4, 6, 7]] == 7.0).all())


@pytest.mark.parametrize("bits", [4, 8])
def test_shared_expert_with_scalar_gate(nv, ctx, bits):
    rng = np.random.default_rng(bits)
    # 192 tokens and more go through the grouped-GEMM kernels in their dense mode
    # (one to four tokens of a shape the row engine has short blocks for: three launches)
    for d, f, tokens in [(128, 64, 1), (2048, 512, 1), (2048, 512, 6), (256, 128, 9), (256, 128, 192), (192, 64, 250),
                         (2048, 512, 200), (512, 192, 300), (256, 128, 130), (2048, 512, 3), (1024, 1024, 4)]:
        say("shared expert", ctx.act, bits, d, f, tokens)
        host = _random_blobs(rng, d, f, bits, 1, 0.03)[0]
        gate = O.quantize_affine(O.round_bf16(gauss(rng, (1, d), 0.05)), 8)
        x = round_act(gauss(rng, (tokens, d)), ctx.act)
        off, _ = nv.expert_offsets(d, f, bits)
        se = nv.SharedExpertRuntime(ctx, bits)
        gdesc = nv.rows_desc(8, dev(gate[0]), dev(gate[1].view(np.int16)), dev(gate[2].view(np.int16)))
        y = se.encode(dev(host), off, act_tensor(x, ctx), d, f, gdesc)
        y0 = se.encode(dev(host), off, act_tensor(x, ctx), d, f, None)
        torch.cuda.synchronize()
        for t in range(tokens):
            plain = O.expert_ffn_accumulate(host, bits, x[t], d, f, 1.0, np.zeros(d, np.float32))
            g = O.router_logits(8, gate[0], gate[1], gate[2], x[t])[0]
            assert O.rel_error(act_np(y0[t]), plain) < TOL_ACT
            assert O.rel_error(act_np(y[t]), plain / (1 + np.exp(-g))) < TOL_ACT
    with pytest.raises(nv.NvmaiError) as e:                 # SharedExpertError.unsupportedWeightBits
        nv.SharedExpertRuntime(ctx, 6)
    assert e.value.name == "unsupported"


# ------------------------------------------------------------------ fused decode layer
def _layer_case(nv, ctx, rng, d, f, E, k, bits, tokens, router_kind, std, shared=True, gated=True):
    mk = lambda r, c, s_=std: O.round_bf16(gauss(rng, (r, c), s_))
    # build the pool on the GPU with the (bit-exact) device quantizer, then read it back
    off, stride = nv.expert_offsets(d, f, bits)
    pool = torch.empty((E + 1, stride), dtype=torch.uint8, device="cuda")
    for e in range(E + 1):
        gw = torch.randn((f, d), device="cuda", dtype=torch.float32).mul_(std).to(torch.bfloat16)
        uw = torch.randn((f, d), device="cuda", dtype=torch.float32).mul_(std).to(torch.bfloat16)
        dw = torch.randn((d, f), device="cuda", dtype=torch.float32).mul_(std).to(torch.bfloat16)
        nv.pack_expert(ctx, gw, uw, dw, bits, pool[e])
    torch.cuda.synchronize()
    pool_h = pool.cpu().numpy()
    rw = mk(E, d, 0.02)
    if router_kind == 16:
        rh = (O.bf16_bits(rw), None, None)
        rdesc = nv.rows_desc(16, dev(rh[0].view(np.int16)))
    else:
        rh = O.quantize_affine(rw, router_kind)
        rdesc = nv.rows_desc(router_kind, dev(rh[0]), dev(rh[1].view(np.int16)), dev(rh[2].view(np.int16)))
    gh = O.quantize_affine(mk(1, d, 0.05), 8)
    gdesc = nv.rows_desc(8, dev(gh[0]), dev(gh[1].view(np.int16)), dev(gh[2].view(np.int16)))
    x = round_act(gauss(rng, (tokens, d)), ctx.act)
    layer = nv.moe_layer_desc(d, f, E, k, bits, rdesc, pool[:E], pool[E] if shared else None,
                              gdesc if shared and gated else None)
    stats = torch.zeros(2, dtype=torch.int32, device="cuda")
    y, idx, w = nv.MoE(ctx, bits).decode_layer(layer, act_tensor(x, ctx), want_routes=True, stats=stats)
    torch.cuda.synchronize()
    io, wo, yo = O.moe_layer_forward(x, d, f, k, bits, (router_kind,) + rh, pool_h[:E],
                                     pool_h[E] if shared else None, (8,) + gh if shared and gated else None)
    assert np.array_equal(u32(idx), io), "routing indices"
    assert np.abs(u16(w).astype(np.int32) - wo.astype(np.int32)).max() <= 1
    assert O.rel_error(act_np(y), yo) < TOL_ACT
    assert int(stats[1]) == len(np.unique(io))


@pytest.mark.parametrize("bits", [8, 4])
def test_decode_layer_toy_shapes(nv, ctx, bits):
    rng = np.random.default_rng(40 + bits)
    for d, f, E, k, tokens, kind in [(128, 64, 16, 8, 1, 8), (128, 64, 16, 8, 5, 16), (256, 128, 32, 4, 11, 4),
                                     (192, 64, 8, 2, 3, 16)]:
        say("decode layer toy", ctx.act, bits, d, f, E, k, tokens, kind)
        _layer_case(nv, ctx, rng, d, f, E, k, bits, tokens, kind, 0.05)


def test_decode_layer_many_tokens_gate_row(nv, ctx_bf16):
    # 64 tokens and more: router rows and the shared expert's gate row through the tiled router kernel
    say("decode layer many tokens")
    _layer_case(nv, ctx_bf16, np.random.default_rng(5), 256, 128, 32, 4, 8, 90, 16, 0.05)
    _layer_case(nv, ctx_bf16, np.random.default_rng(6), 128, 64, 16, 8, 4, 70, 8, 0.05)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("tokens", [1, 4, 32])
def test_decode_layer_production_shape(nv, ctx_bf16, bits, tokens):
    # configs[1]: hidden 2048, 256 experts top-8, intermediate 512, shared expert with sigmoid gate
    say("decode layer production", bits, tokens)
    _layer_case(nv, ctx_bf16, np.random.default_rng(tokens + bits), 2048, 512, 256, 8, bits, tokens, 16, 0.02)


@pytest.mark.parametrize("bits", [8, 4])
def test_decode_layer_few_tokens_three_launches(nv, ctx, bits):
    # one to four tokens: gate/up selects for itself, down projection and combine are one launch;
    # every row-chunk count both kernels are built for, with and without shared expert and gate,
    # tokens that share experts (few experts), and one shape outside them (the five-launch path)
    rng = np.random.default_rng(70 + bits)
    per = 128 // bits                                  # codes per 16-byte chunk
    for c1, c2, E, k, tokens, shared, gated in [(64, 16, 16, 8, 1, True, True), (128, 32, 12, 11, 4, True, False),
                                                (64, 64, 8, 2, 3, False, False), (64, 32, 300, 8, 1, True, True),
                                                (128, 16, 10, 8, 2, True, True), (64, 8, 8, 4, 2, True, True)]:
        d, f = c1 * per, c2 * per
        say("decode layer few tokens", ctx.act, bits, d, f, E, k, tokens, shared, gated)
        _layer_case(nv, ctx, rng, d, f, E, k, bits, tokens, 16 if d <= 2048 else 8, 0.03, shared, gated)


@pytest.mark.parametrize("tokens", [1, 12])
def test_decode_layer_replays_from_a_captured_graph(nv, ctx_bf16, tokens):
    # The calls only enqueue kernels (no allocation after warm-up, no memset nodes), so a caller may
    # capture a decode step in a HIP graph: every replay, with new inputs in the same buffers and
    # eager work in between, must equal the eager result bit for bit (three launches at one token,
    # five with the work list at twelve).
    say("decode layer graph replay", tokens)
    ctx, d, f, E, k, bits = ctx_bf16, 1024, 256, 24, 8, 8
    gen = torch.Generator(device="cuda").manual_seed(5 + tokens)
    off, stride = nv.expert_offsets(d, f, bits)
    pool = torch.empty((E + 1, stride), dtype=torch.uint8, device="cuda")
    for e in range(E + 1):
        mk = lambda r, c: torch.empty((r, c), device="cuda").normal_(0.0, 0.03, generator=gen).to(torch.bfloat16)
        nv.pack_expert(ctx, mk(f, d), mk(f, d), mk(d, f), bits, pool[e])
    router = torch.empty((E, d), device="cuda").normal_(0.0, 0.05, generator=gen).to(torch.bfloat16)
    layer = nv.moe_layer_desc(d, f, E, k, bits, nv.rows_desc(16, router.view(torch.int16)), pool[:E], pool[E])
    moe = nv.MoE(ctx, bits)
    xs = [torch.empty((tokens, d), device="cuda").normal_(0.0, 1.0, generator=gen).to(torch.bfloat16) for _ in range(4)]
    x_static = xs[0].clone()
    y_static = torch.empty((tokens, d), dtype=torch.bfloat16, device="cuda")
    moe.decode_layer(layer, x_static, y_static)                      # warm-up: the workspace is sized here
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            moe.decode_layer(layer, x_static, y_static)
    torch.cuda.synchronize()
    for x in xs:
        want = moe.decode_layer(layer, x).clone()                    # eager, its own output buffer
        torch.cuda.synchronize()
        x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_static, want)


def test_captured_graph_survives_workspace_growth(nv):
    # A captured step keeps the workspace addresses it was recorded with.  A later, larger call on the
    # same context moves the workspace to a new block; the old block must stay allocated, so that a
    # replay after the growth still equals the eager result bit for bit.  A call that would have to
    # grow the workspace while its stream is being captured reports "scratch" and launches nothing.
    say("graph replay after workspace growth")
    ctx = nv.Context(0, nv.ACT_BF16)
    d, f, E, k, bits, tokens = 1024, 256, 24, 8, 8, 12
    gen = torch.Generator(device="cuda").manual_seed(77)
    off, stride = nv.expert_offsets(d, f, bits)
    pool = torch.empty((E + 1, stride), dtype=torch.uint8, device="cuda")
    mk = lambda r, c, s=0.03: torch.empty((r, c), device="cuda").normal_(0.0, s, generator=gen).to(torch.bfloat16)
    for e in range(E + 1):
        nv.pack_expert(ctx, mk(f, d), mk(f, d), mk(d, f), bits, pool[e])
    router = mk(E, d, 0.05)
    layer = nv.moe_layer_desc(d, f, E, k, bits, nv.rows_desc(16, router.view(torch.int16)), pool[:E], pool[E])
    moe = nv.MoE(ctx, bits)
    x_static = mk(tokens, d, 1.0)
    y_static = torch.empty((tokens, d), dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.Stream()
    # (a) no warm-up: the workspace would have to grow inside the capture
    assert ctx.workspace_bytes == 0
    refused = torch.cuda.CUDAGraph()
    err = None
    with torch.cuda.stream(stream):
        with torch.cuda.graph(refused, stream=stream):
            y_static.zero_()
            try:
                moe.decode_layer(layer, x_static, y_static)
            except nv.NvmaiError as e:
                err = e
    torch.cuda.synchronize()
    assert err is not None and err.name == "scratch" and ctx.workspace_bytes == 0
    # (b) reserve a small workspace, capture, then grow it with a 100-token call and replay
    ctx.reserve(1 << 20)
    moe.decode_layer(layer, x_static, y_static)
    torch.cuda.synchronize()
    before = ctx.workspace_bytes
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            moe.decode_layer(layer, x_static, y_static)
    torch.cuda.synchronize()
    big = moe.decode_layer(layer, mk(100, d, 1.0))
    torch.cuda.synchronize()
    assert ctx.workspace_bytes > before and bool(torch.isfinite(big.float()).all())
    for _ in range(3):
        x = mk(tokens, d, 1.0)
        want = moe.decode_layer(layer, x).clone()
        junk = torch.full((1 << 20,), 1.0, device="cuda")          # eager work between the replays
        torch.cuda.synchronize()
        del junk
        x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_static, want)
    ctx.close()


@pytest.mark.parametrize("bits", [8, 4])
def test_decode_layer_prenorm_equals_the_separate_calls(nv, ctx, bits):
    # residual add + RMSNorm done by the router launch: the same bits as nvmai_hip_residual_add_rmsnorm
    # followed by the plain decode layer, for the three-launch path (1-4 tokens), the work-list path
    # (5-63) and the fallback (64 and more; or the residual rows updated in place)
    rng = np.random.default_rng(500 + bits)
    d, f, E, k = 256, 128, 16, 4
    off, stride = nv.expert_offsets(d, f, bits)
    pool = torch.empty((E + 1, stride), dtype=torch.uint8, device="cuda")
    for e in range(E + 1):
        mk = lambda r, c: torch.randn((r, c), device="cuda").mul_(0.05).to(torch.bfloat16)
        nv.pack_expert(ctx, mk(f, d), mk(f, d), mk(d, f), bits, pool[e])
    rdesc = nv.rows_desc(16, dev(O.bf16_bits(gauss(rng, (E, d), 0.02)).view(np.int16)))
    gh = O.quantize_affine(O.round_bf16(gauss(rng, (1, d), 0.05)), 8)
    gdesc = nv.rows_desc(8, dev(gh[0]), dev(gh[1].view(np.int16)), dev(gh[2].view(np.int16)))
    layer = nv.moe_layer_desc(d, f, E, k, bits, rdesc, pool[:E], pool[E], gdesc)
    w = dev(O.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32)).view(np.int16))
    moe = nv.MoE(ctx, bits)
    for tokens, with_delta, in_place in [(1, True, False), (3, False, False), (5, True, False), (32, True, False),
                                         (70, True, False), (4, True, True)]:
        say("decode layer prenorm", ctx.act, bits, tokens, with_delta, in_place)
        h = act_tensor(round_act(gauss(rng, (tokens, d)), ctx.act), ctx)
        delta = act_tensor(round_act(gauss(rng, (tokens, d), 0.3), ctx.act), ctx) if with_delta else None
        # reference: the separate calls
        h_ref = h.clone()
        if with_delta:
            n_ref = nv.residual_add_rmsnorm(ctx, h_ref, delta, w)
        else:
            n_ref = nv.RMSNorm(ctx).encode_bf16w(h_ref, w)
        y_ref, i_ref, w_ref = moe.decode_layer(layer, n_ref, want_routes=True)
        h_in = h.clone()
        h_out = h_in if in_place else torch.full_like(h, 9.0)
        normed, y = torch.full_like(h, 9.0), torch.full_like(h, 9.0)
        idx = torch.zeros((tokens, k), dtype=torch.int32, device="cuda")
        wt = torch.zeros((tokens, k), dtype=torch.int16, device="cuda")
        moe.decode_layer_prenorm(layer, h_in, delta, w, h_out, normed, y, idx=idx, w=wt)
        torch.cuda.synchronize()
        assert torch.equal(h_out, h_ref) and torch.equal(normed, n_ref)
        assert torch.equal(idx, i_ref.view(torch.int32).reshape(tokens, k)) and torch.equal(wt, w_ref.view(torch.int16).reshape(tokens, k))
        assert torch.equal(y, y_ref)
        if not in_place:
            assert torch.equal(h_in, h)                      # the residual rows read by the launch are untouched


@pytest.mark.parametrize("bits", [4, 8])
def test_decode_layer_with_both_norms_equals_the_separate_calls(nv, ctx, bits):
    # the block between two norms in one call: residual add + norm before it, and after it the residual
    # add that closes the layer with the norm that opens the next one -- in the combine launch from
    # five tokens on, the residual-add-norm kernel after the block below that and from 64 tokens on; the
    # next norm's rows may land in the buffer of the first norm's (dead by then)
    rng = np.random.default_rng(900 + bits)
    d, f, E, k = 256, 128, 16, 4
    off, stride = nv.expert_offsets(d, f, bits)
    pool = torch.empty((E + 1, stride), dtype=torch.uint8, device="cuda")
    for e in range(E + 1):
        mk = lambda r, c: torch.randn((r, c), device="cuda").mul_(0.05).to(torch.bfloat16)
        nv.pack_expert(ctx, mk(f, d), mk(f, d), mk(d, f), bits, pool[e])
    rdesc = nv.rows_desc(16, dev(O.bf16_bits(gauss(rng, (E, d), 0.02)).view(np.int16)))
    gh = O.quantize_affine(O.round_bf16(gauss(rng, (1, d), 0.05)), 8)
    gdesc = nv.rows_desc(8, dev(gh[0]), dev(gh[1].view(np.int16)), dev(gh[2].view(np.int16)))
    w1 = dev(O.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32)).view(np.int16))
    w2 = dev(O.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32)).view(np.int16))
    moe = nv.MoE(ctx, bits)
    for tokens, gated, alias in [(1, True, False), (4, True, True), (5, True, False), (16, True, True), (32, False, True),
                                 (63, True, False), (70, True, True)]:
        say("decode layer norms", ctx.act, bits, tokens, gated, alias)
        layer = nv.moe_layer_desc(d, f, E, k, bits, rdesc, pool[:E], pool[E], gdesc if gated else None)
        h = act_tensor(round_act(gauss(rng, (tokens, d)), ctx.act), ctx)
        delta = act_tensor(round_act(gauss(rng, (tokens, d), 0.3), ctx.act), ctx)
        # reference: the separate calls
        h_ref, n_ref, y_ref = torch.full_like(h, 9.0), torch.full_like(h, 9.0), torch.full_like(h, 9.0)
        moe.decode_layer_prenorm(layer, h.clone(), delta, w1, h_ref, n_ref, y_ref)
        next_ref = nv.residual_add_rmsnorm(ctx, h_ref, y_ref, w2)
        h_out, normed, y = torch.full_like(h, 9.0), torch.full_like(h, 9.0), torch.full_like(h, 9.0)
        nxt = normed if alias else torch.full_like(h, 9.0)
        moe.decode_layer_norms(layer, h.clone(), delta, w1, h_out, normed, y, w2, nxt)
        torch.cuda.synchronize()
        assert torch.equal(y, y_ref)
        assert torch.equal(h_out, h_ref)                      # the stream after the layer
        assert torch.equal(nxt, next_ref)
        if not alias:
            assert torch.equal(normed, n_ref)


@pytest.mark.parametrize("bits", [4, 8])
def test_affine_gemv_prenorm_equals_the_separate_calls(nv, ctx, bits):
    # a layer's input norm (with the residual add before it) done by the projection launch: the bits
    # of nvmai_hip_residual_add_rmsnorm followed by nvmai_hip_affine_gemv, for the one-launch shapes
    # (1-4 rows of 2048 against a projection of a decode step) and for the shapes that fall back to
    # the two steps through the scratch rows (more rows, short rows, a long projection)
    rng = np.random.default_rng(900 + bits)
    for tokens, m, n, with_delta in [(1, 12352, 2048, True), (4, 9216, 2048, True), (2, 2048, 2048, False), (3, 4100, 2048, True),
                                     (1, 320, 256, True), (6, 2048, 2048, True), (2, 17000, 2048, True)]:
        say("affine gemv prenorm", ctx.act, bits, tokens, m, n, with_delta)
        wmat = torch.empty((m, n), device="cuda").normal_(0.0, 0.03).to(torch.bfloat16)
        p_, s_, b_ = nv.quantize_affine(ctx, wmat, bits)
        h = act_tensor(round_act(gauss(rng, (tokens, n)), ctx.act), ctx)
        delta = act_tensor(round_act(gauss(rng, (tokens, n), 0.3), ctx.act), ctx) if with_delta else None
        w = dev(O.bf16_bits(rng.uniform(0.5, 1.5, n).astype(np.float32)).view(np.int16))
        h_ref = h.clone()
        n_ref = nv.residual_add_rmsnorm(ctx, h_ref, delta, w) if with_delta else nv.RMSNorm(ctx).encode_bf16w(h_ref, w)
        y_ref = nv.affine_gemv(ctx, p_, s_, b_, bits, n_ref, m, n)
        h_in, h_out = h.clone(), torch.full_like(h, 9.0)
        scratch = torch.full_like(h, 7.0)
        y = nv.affine_gemv_prenorm(ctx, p_, s_, b_, bits, h_in, delta, w, h_out, m, n, normed_scratch=scratch)
        torch.cuda.synchronize()
        assert torch.equal(h_out, h_ref), "residual rows"
        assert torch.equal(y.view(torch.int16), y_ref.view(torch.int16)), "projection"
        assert torch.equal(h_in, h)                          # the rows the launch reads are untouched
        fused = tokens <= 4 and n == 2048 and m <= 16384
        assert bool((scratch == 7.0).all()) == fused         # the one-launch form never touches the scratch rows
        if not fused:                                        # and without them the other shapes are refused
            with pytest.raises(nv.NvmaiError):
                nv.affine_gemv_prenorm(ctx, p_, s_, b_, bits, h_in, delta, w, h_out, m, n)
    # hidden_out must be a buffer of its own for the one-launch form; in place it takes the two steps
    h_in = h.clone()
    y2 = nv.affine_gemv_prenorm(ctx, p_, s_, b_, bits, h_in, delta, w, h_in, m, n, normed_scratch=scratch)
    torch.cuda.synchronize()
    assert torch.equal(h_in, h_ref) and torch.equal(y2.view(torch.int16), y_ref.view(torch.int16))
