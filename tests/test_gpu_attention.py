"""GPU parity: KV quantize-on-write (codes and fp16 scale/bias bits exact), partial RoPE and GQA
decode attention over quantized K/V, through the C ABI against the CPU oracle.

Attention bar: 16-bit output within 1e-2 of the oracle's attention over the SAME quantized rows
(max|diff| / max|ref|, RelError.swift:5-16); and the reference's own bar against unquantized
attention: 0.02 at 8 bits, 0.20 at 4 bits (KVCacheQuantizedAttentionTests.swift:71)."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import act_np, act_tensor, dev, gauss, round_act, say

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


def test_row_layout_and_geometry_known_answers(nv):
    # KVCacheQuantizedAttentionTests.swift:76-88, AttentionTests.swift:25-47
    assert nv.kv_row_layout(512, 16) == (1024, 1024)
    assert nv.kv_row_layout(512, 8) == (544, 512)
    assert nv.kv_row_layout(512, 4) == (288, 256)
    assert nv.Attention.split_geometry(16, 8, 1536, 512, True) == (1024, 16, 64, 128)
    assert nv.Attention.split_geometry(16, 2, 1536, 0, False) == (1536, 16, 96, 256)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("elements,tokens", [(512, 37), (100, 3), (64, 1), (2048, 5)])
def test_kv_quantize_codes_bit_exact(nv, ctx, bits, elements, tokens):
    say("kv quantize", ctx.act, bits, elements, tokens)
    rng = np.random.default_rng(elements + bits)
    v = round_act(gauss(rng, (tokens, elements)), ctx.act)
    v[0, :64] = 0.25                                   # flat group: scale 0, codes 0
    if tokens > 2:
        v[2, :] = v[2, 0]
    src_stride = elements + 24                         # a padded source row, as the QKV stage buffer has
    src = np.zeros((tokens, src_stride), np.float32)
    src[:, :elements] = v
    cache = nv.KVCache(1, tokens + 2, elements, bits)
    nv.KVCacheQuantizer(ctx).encode(act_tensor(src, ctx), src_stride, cache.view(0, 1), tokens, elements)
    torch.cuda.synchronize()
    got = cache.rows[0].cpu().numpy()
    want = O.kv_quantize(v, bits)
    assert np.array_equal(got[1:1 + tokens], want)     # codes, fp16 scale bits, fp16 bias bits
    assert not got[0].any() and not got[-1].any()      # neighbouring rows untouched


def test_kv_quantize_rejects_bad_arguments(nv, ctx):
    say("kv quantize errors")
    cache = nv.KVCache(1, 4, 512, 16)
    x = torch.zeros((1, 512), dtype=ctx.dtype, device="cuda")
    with pytest.raises(nv.NvmaiError) as e:            # "KV quantizer requires 4-bit or 8-bit destination"
        nv.KVCacheQuantizer(ctx).encode(x, 512, cache.view(), 1, 512)
    assert e.value.name == "unsupported"
    cache8 = nv.KVCache(1, 4, 512, 8)
    with pytest.raises(nv.NvmaiError) as e:            # "source token stride is too small"
        nv.KVCacheQuantizer(ctx).encode(x, 256, cache8.view(), 1, 512)
    assert e.value.name == "invalid_arg"


def test_rope_matches_oracle(nv, ctx):
    say("rope", ctx.act)
    rng = np.random.default_rng(3)
    x = round_act(gauss(rng, (6, 16, 256)), ctx.act)
    pos = np.array([0, 1, 17, 4095, 32767, 131071], np.uint32)
    want = O.rope_neox_subdim(x, 64, pos, 1e7)
    d = act_tensor(x, ctx)
    nv.rope_neox_subdim(ctx, d, 64, 1e7, positions=dev(pos.view(np.int32)))
    torch.cuda.synchronize()
    got = act_np(d)
    assert np.array_equal(got[..., 64:], x[..., 64:])                  # pass-through region untouched
    assert np.array_equal(got[0], x[0])                                # position 0 is the identity
    assert np.abs(got - round_act(want, ctx.act)).max() <= 2 ** -6     # one 16-bit ulp at |x| < 4
    assert O.rel_error(got, want) < 1e-2
    d2 = act_tensor(x[:2], ctx)
    nv.rope_neox_subdim(ctx, d2, 64, 1e7, position=17)                 # the reference's single-position call
    torch.cuda.synchronize()
    want2 = O.rope_neox_subdim(x[:2], 64, np.array([17, 17], np.uint32), 1e7)
    assert O.rel_error(act_np(d2), want2) < 1e-2


def _attention_case(nv, ctx, rng, bits, batch, nq, nkv, hd, seq, kv_start=0, std=1.0, uniform=False):
    elements = nkv * hd
    mk = (lambda s: rng.uniform(-0.5, 0.5, s).astype(np.float32)) if uniform else (lambda s: gauss(rng, s, std))
    q = round_act(mk((batch, nq, hd)), ctx.act)
    k = round_act(mk((batch, seq, elements)), ctx.act)
    v = round_act(mk((batch, seq, elements)), ctx.act)
    kc, vc = nv.KVCache(batch, seq, elements, bits), nv.KVCache(batch, seq, elements, bits)
    if bits == 16:
        kc.rows.copy_(dev(k).to(torch.float16).view(torch.uint8).view(batch, seq, -1))
        vc.rows.copy_(dev(v).to(torch.float16).view(torch.uint8).view(batch, seq, -1))
    else:
        quant = nv.KVCacheQuantizer(ctx)
        for b in range(batch):
            quant.encode(act_tensor(k[b], ctx), elements, kc.view(b), seq, elements)
            quant.encode(act_tensor(v[b], ctx), elements, vc.view(b), seq, elements)
    out = nv.Attention(ctx).encode_full(act_tensor(q, ctx), kc, vc, hd, nq, nkv, seq, scale=None, kv_start=kv_start)
    torch.cuda.synchronize()
    got = act_np(out)
    scale = 1.0 / np.sqrt(hd)
    for b in range(batch):
        if bits == 16:
            k16 = O.f16_to_float(O.f16_bits(k[b]))
            v16 = O.f16_to_float(O.f16_bits(v[b]))
            want = O.attention_decode(q[b], k16, v16, 32, nq, nkv, hd, seq, scale, kv_start)
        else:
            kq, vq = kc.rows[b].cpu().numpy(), vc.rows[b].cpu().numpy()
            assert np.array_equal(kq, O.kv_quantize(k[b], bits))       # KV codes bit-exact
            want = O.attention_decode(q[b], kq, vq, bits, nq, nkv, hd, seq, scale, kv_start)
        err = O.rel_error(got[b], want)
        assert err < 1e-2, "batch %d rel %g" % (b, err)
    return got, q, k, v


@pytest.mark.parametrize("bits", [8, 4])
def test_attention_production_shape(nv, ctx, bits):
    # configs[3]: 16 query heads, 2 KV heads, head_dim 256; ragged lengths exercise the tails
    rng = np.random.default_rng(bits)
    for batch, seq, kv_start in [(1, 8, 0), (1, 1, 0), (2, 33, 0), (1, 127, 0), (1, 128, 0), (3, 1000, 0),
                                 (1, 4096, 0), (2, 2048, 1024), (1, 300, 299)]:
        say("attention mfma", ctx.act, bits, batch, seq, kv_start)
        _attention_case(nv, ctx, rng, bits, batch, 16, 2, 256, seq, kv_start)


def test_attention_tracks_unquantized_reference(nv, ctx):
    # KVCacheQuantizedAttentionTests.swift:7-74: seq 8, uniform(-0.5, 0.5)
    for bits, tol in ((8, 0.02), (4, 0.20)):
        say("attention vs unquantized", ctx.act, bits)
        rng = np.random.default_rng(0x4B56 + bits)
        got, q, k, v = _attention_case(nv, ctx, rng, bits, 1, 16, 2, 256, 8, uniform=True)
        want = O.attention_decode(q[0], k[0], v[0], 32, 16, 2, 256, 8, 1 / 16.0)
        assert O.rel_error(got[0], want) < tol


@pytest.mark.parametrize("bits", [16, 8, 4])
def test_attention_other_shapes_generic_path(nv, ctx, bits):
    rng = np.random.default_rng(10 + bits)
    for batch, nq, nkv, hd, seq, kv_start in [(1, 4, 2, 64, 19, 0), (2, 8, 8, 128, 70, 0), (1, 16, 8, 256, 40, 8),
                                              (1, 2, 1, 512, 9, 0), (1, 4, 4, 96, 5, 0)]:
        say("attention generic", ctx.act, bits, batch, nq, nkv, hd, seq, kv_start)
        _attention_case(nv, ctx, rng, bits, batch, nq, nkv, hd, seq, kv_start)


def test_attention_empty_range_and_errors(nv, ctx):
    say("attention empty range")
    kc, vc = nv.KVCache(1, 8, 512, 8), nv.KVCache(1, 8, 512, 8)
    q = torch.ones((1, 16, 256), dtype=ctx.dtype, device="cuda")
    out = nv.Attention(ctx).encode_full(q, kc, vc, 256, 16, 2, 8, kv_start=8)       # attention.metal:410-416
    torch.cuda.synchronize()
    assert not act_np(out).any()
    with pytest.raises(nv.NvmaiError) as e:            # numQHeads must be a multiple of numKVHeads
        nv.Attention(ctx).encode_full(q, kc, vc, 256, 15, 2, 8)
    assert e.value.name == "invalid_arg"


def test_attention_long_context_properties(nv):
    # 32K context: too slow for the scalar oracle in full, so (a) one head group against the oracle
    # and (b) size-independent properties: permuting the KV positions changes nothing, and a cache
    # whose V rows are all equal returns that row.
    say("attention 32K")
    ctx = nv.Context(0, 0)
    rng = np.random.default_rng(99)
    nq, nkv, hd, seq, bits = 16, 2, 256, 32768, 8
    q = O.round_bf16(gauss(rng, (1, nq, hd)))
    k = torch.randn((seq, nkv * hd), device="cuda").to(torch.bfloat16)
    v = torch.randn((seq, nkv * hd), device="cuda").to(torch.bfloat16)
    kc, vc = nv.KVCache(1, seq, nkv * hd, bits), nv.KVCache(1, seq, nkv * hd, bits)
    quant, attn = nv.KVCacheQuantizer(ctx), nv.Attention(ctx)
    quant.encode(k, nkv * hd, kc.view(), seq, nkv * hd)
    quant.encode(v, nkv * hd, vc.view(), seq, nkv * hd)
    qd = act_tensor(q, ctx)
    out = attn.encode_full(qd, kc, vc, hd, nq, nkv, seq)
    perm = torch.randperm(seq, device="cuda")
    kc2, vc2 = nv.KVCache(1, seq, nkv * hd, bits), nv.KVCache(1, seq, nkv * hd, bits)
    kc2.rows[0] = kc.rows[0][perm]
    vc2.rows[0] = vc.rows[0][perm]
    out2 = attn.encode_full(qd, kc2, vc2, hd, nq, nkv, seq)
    vc3 = nv.KVCache(1, seq, nkv * hd, bits)
    vc3.rows[0] = vc.rows[0][:1].expand(seq, -1)
    out3 = attn.encode_full(qd, kc, vc3, hd, nq, nkv, seq)
    torch.cuda.synchronize()
    assert O.rel_error(act_np(out2), act_np(out)) < 1e-2
    row0 = O.kv_dequant(vc.rows[0][:1].cpu().numpy(), nkv * hd, bits)[0].reshape(nkv, hd)
    assert np.abs(act_np(out3)[0].reshape(nkv, 8, hd) - row0[:, None, :]).max() < 2e-2
    want = O.attention_decode(q[0], kc.rows[0].cpu().numpy(), vc.rows[0].cpu().numpy(), bits, nq, nkv, hd, seq,
                              1 / 16.0)
    assert O.rel_error(act_np(out)[0], want) < 1e-2
    torch.cuda.synchronize()
    ctx.close()


def _long_cache(nv, ctx, gen, batch, seq, elements, bits):
    """K and V caches of `batch` sequences filled by quantize-on-write from seeded bf16 rows made on
    the GPU; returns the caches and, per sequence, a few source rows for the code check."""
    kc, vc = nv.KVCache(batch, seq, elements, bits), nv.KVCache(batch, seq, elements, bits)
    quant = nv.KVCacheQuantizer(ctx)
    probes = []
    for b in range(batch):
        k = torch.empty((seq, elements), device="cuda").normal_(0.0, 1.0, generator=gen).to(torch.bfloat16)
        v = torch.empty((seq, elements), device="cuda").normal_(0.0, 1.0, generator=gen).to(torch.bfloat16)
        quant.encode(k, elements, kc.view(b), seq, elements)
        quant.encode(v, elements, vc.view(b), seq, elements)
        rows = np.r_[0:32, seq // 2 - 16:seq // 2 + 16, seq - 32:seq]
        probes.append((rows, k[torch.from_numpy(rows).cuda()].float().cpu().numpy()))
    torch.cuda.synchronize()
    return kc, vc, probes


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("batch,seq,kv_start", [(8, 32768, 0), (1, 131072, 0), (8, 131072, 0), (2, 131067, 77)],
                         ids=["32Kx8", "128Kx1", "128Kx8", "128K-ragged"])
def test_attention_configs3_long_context(nv, bits, batch, seq, kv_start):
    # configs[3] at its long contexts and at batch 8: the production kernel's size-dependent parts
    # (32-bit row offsets, buffer bounds of seq * stride bytes, up to 512 chunks) against the oracle
    # on EVERY sequence, KV codes of the quantize-on-write bit-exact on sampled rows, a start
    # offset and a length that is not a multiple of the 32-token step, and two different chunk
    # counts (a sequence alone, and inside the batch) giving the same output.
    say("attention long context", bits, batch, seq, kv_start)
    ctx = nv.Context(0, 0)
    nq, nkv, hd = 16, 2, 256
    elements = nkv * hd
    gen = torch.Generator(device="cuda").manual_seed(seq % 1000 + 10 * batch + bits)
    kc, vc, probes = _long_cache(nv, ctx, gen, batch, seq, elements, bits)
    q = O.round_bf16(gauss(np.random.default_rng(seq + bits), (batch, nq, hd)))
    attn = nv.Attention(ctx)
    out = act_np(attn.encode_full(act_tensor(q, ctx), kc, vc, hd, nq, nkv, seq, kv_start=kv_start))
    torch.cuda.synchronize()
    worst = 0.0
    for b in range(batch):
        rows, src = probes[b]
        got_rows = kc.rows[b][torch.from_numpy(rows).cuda()].cpu().numpy()
        assert np.array_equal(got_rows, O.kv_quantize(src, bits)), "KV codes, sequence %d" % b
        kq, vq = kc.rows[b].cpu().numpy(), vc.rows[b].cpu().numpy()
        want = O.attention_decode(q[b], kq, vq, bits, nq, nkv, hd, seq, 1 / 16.0, kv_start)
        err = O.rel_error(out[b], want)
        worst = max(worst, err)
        assert err < 1e-2, "sequence %d rel %g" % (b, err)
        del kq, vq
    print("worst rel", worst, flush=True)
    if batch > 1:
        # the last sequence on its own: batch 1 cuts the range into more chunks than batch 8 does
        b = batch - 1
        k1, v1 = nv.KVCache(1, 1, elements, bits), nv.KVCache(1, 1, elements, bits)
        k1.rows, v1.rows = kc.rows[b:b + 1], vc.rows[b:b + 1]
        alone = act_np(attn.encode_full(act_tensor(q[b:b + 1], ctx), k1, v1, hd, nq, nkv, seq, kv_start=kv_start))
        torch.cuda.synchronize()
        assert O.rel_error(alone[0], out[b]) < 1e-2
    torch.cuda.synchronize()
    ctx.close()


# ---------------------------------------------------------------- causal prefill attention
def _prefill_case(nv, ctx, seed, bits, start, chunk, window, hd, nq, nkv, extra_kv=0, pad=True, ring=0, lo=-0.35,
                  hi=0.35, tol=1e-2, scale=1.0):
    """One PrefillAttention.encodeCausal call against the oracle over the same rows.  pad: strided
    q / out rows and offset buffers as PrefillAttentionTests.swift:179-258 builds them."""
    rng = np.random.default_rng(seed)
    kv_valid = start + chunk + extra_kv
    elements, row = nkv * hd, nq * hd
    q = round_act(rng.uniform(lo, hi, (chunk, row)).astype(np.float32), ctx.act)
    k = round_act(rng.uniform(lo, hi, (kv_valid, elements)).astype(np.float32), ctx.act)
    v = round_act(rng.uniform(lo, hi, (kv_valid, elements)).astype(np.float32), ctx.act)
    q_stride, o_stride, q_off, o_off = (row + 3, row + 7, 17, 29) if pad else (row, row, 0, 0)
    if pad == "aligned":                                            # strided and offset, every row at a 16-byte boundary
        q_stride, o_stride, q_off, o_off = row + 8, row + 16, 24, 40
    q_buf = torch.zeros(q_off + chunk * q_stride, dtype=ctx.dtype, device="cuda")
    q_buf[q_off:].view(chunk, q_stride)[:, :row] = act_tensor(q, ctx)
    out_buf = torch.full((o_off + chunk * o_stride,), 7.0, dtype=ctx.dtype, device="cuda")
    rows = ring if ring else kv_valid
    kc, vc = nv.KVCache(1, rows, elements, bits), nv.KVCache(1, rows, elements, bits)
    if bits == 16:
        k, v = O.f16_to_float(O.f16_bits(k)), O.f16_to_float(O.f16_bits(v))
        ko, vo = k, v
        if ring:
            ko, vo = np.zeros((ring, elements), np.float32), np.zeros((ring, elements), np.float32)
            for p in range(kv_valid):
                ko[p % ring], vo[p % ring] = k[p], v[p]
        kc.rows[0].copy_(dev(ko).to(torch.float16).view(torch.uint8).view(rows, -1))
        vc.rows[0].copy_(dev(vo).to(torch.float16).view(torch.uint8).view(rows, -1))
        obits = 32
    else:
        assert not ring
        quant = nv.KVCacheQuantizer(ctx)
        quant.encode(act_tensor(k, ctx), elements, kc.view(), kv_valid, elements)
        quant.encode(act_tensor(v, ctx), elements, vc.view(), kv_valid, elements)
        ko, vo = kc.rows[0].cpu().numpy(), vc.rows[0].cpu().numpy()
        obits = bits
    nv.PrefillAttention(ctx).encode_causal(q_buf[q_off:], kc.view(), vc.view(), out_buf[o_off:], start, chunk, hd, nq, nkv,
                                           kv_valid, sliding_window=window, q_token_stride=q_stride,
                                           o_token_stride=o_stride, scale=scale, kv_ring_capacity=ring)
    torch.cuda.synchronize()
    flat = act_np(out_buf)
    got = flat[o_off:].reshape(chunk, o_stride)[:, :row]
    want = O.attention_prefill_causal(q, ko, vo, obits, nq, nkv, hd, start, kv_valid, scale, window=window, ring=ring)
    err = O.rel_error(got, want)
    assert err < tol, "rel %g" % err
    # nothing outside the output rows is written
    assert np.all(flat[:o_off] == 7.0) and np.all(flat[o_off:].reshape(chunk, o_stride)[:, row:] == 7.0)
    return got, want, (q, k, v)


def test_prefill_attention_reference_cases(nv, ctx):
    # PrefillAttentionTests.swift:10-25, 79-116: fp16 rows, strided and offset buffers
    cases = [(0, 3, 0, 8, 4, 2), (4, 3, 0, 8, 4, 2), (2, 4, 16, 8, 4, 2), (7, 4, 5, 8, 4, 2),
             (1023, 1, 1, 256, 16, 8), (1024, 1, 1, 256, 16, 8), (4095, 1, 1, 256, 16, 8), (0, 1, 0, 512, 16, 2),
             (3, 1, 0, 512, 16, 2), (1023, 4, 1024, 256, 16, 8), (31, 8, 0, 512, 16, 2)]
    for n, (start, chunk, window, hd, nq, nkv) in enumerate(cases):
        say("prefill attention fp16 rows", ctx.act, start, chunk, window, hd, nq, nkv)
        _prefill_case(nv, ctx, 0xA510 + n, 16, start, chunk, window, hd, nq, nkv)
    say("prefill attention ring", ctx.act)                         # PrefillAttentionTests.swift:27-56
    _prefill_case(nv, ctx, 0xA611, 16, 20, 4, 8, 32, 4, 2, ring=16)


@pytest.mark.parametrize("bits", [8, 4])
def test_prefill_attention_quantized_rows(nv, ctx, bits):
    # KVCacheQuantizedAttentionTests.swift:91-157 (start 4, four queries, qwen shape) and beyond it:
    # chunks that start deep in the cache, windows, kv_valid past the chunk, odd query counts, the
    # generic path (head_dim 128 and padded rows) beside the matrix-core one
    say("prefill attention vs unquantized", ctx.act, bits)
    got, want, (q, k, v) = _prefill_case(nv, ctx, 0x5052, bits, 4, 4, 0, 256, 16, 2, pad=False, lo=-0.5, hi=0.5,
                                         scale=1 / 16.0)
    dense = O.attention_prefill_causal(q, k, v, 32, 16, 2, 256, 4, 8, 1 / 16.0)
    assert O.rel_error(got, dense) < (0.025 if bits == 8 else 0.20)
    for start, chunk, window, hd, nq, nkv, extra, pad in [
            (0, 1, 0, 256, 16, 2, 0, False), (0, 67, 0, 256, 16, 2, 0, False), (130, 33, 0, 256, 16, 2, 5, False),
            (500, 40, 64, 256, 16, 2, 0, False), (100, 9, 7, 256, 16, 8, 0, False), (64, 5, 0, 256, 16, 16, 0, False),
            (31, 6, 0, 256, 6, 2, 0, False), (40, 7, 16, 256, 16, 2, 0, True), (9, 5, 0, 128, 8, 2, 3, False)]:
        say("prefill attention quantized", ctx.act, bits, start, chunk, window, hd, nq, nkv, extra, pad)
        _prefill_case(nv, ctx, start + chunk, bits, start, chunk, window, hd, nq, nkv, extra_kv=extra, pad=pad,
                      lo=-1.0, hi=1.0, scale=1.0 / np.sqrt(hd))


def test_prefill_attention_long_chunks(nv):
    # chunks whose queries give every compute unit a block (queries x q heads >= 16,384) take the two-launch form
    # -- the key range dequantized once into fp16 scratch, then flash attention on that: every row against the
    # oracle over the same cache rows -- quantized and fp16 rows, a chunk deep in the cache, a window, keys past
    # the chunk, odd query counts (a last block with dead waves and dead columns), every group size, a ring,
    # strided and offset rows at 16-byte boundaries, and rows that are not (those keep the one-launch kernels,
    # which need no scratch: the context's workspace tells which form ran)
    for act in (0, 1):
        for bits, start, chunk, window, nq, nkv, extra, pad, ring in [
                (8, 0, 258, 0, 64, 8, 0, False, 0), (4, 37, 261, 0, 64, 8, 5, False, 0), (8, 300, 257, 64, 64, 8, 0, False, 0),
                (8, 0, 260, 0, 64, 64, 0, False, 0), (16, 5, 256, 0, 64, 16, 0, False, 0), (4, 64, 259, 0, 64, 32, 3, "aligned", 0),
                (16, 200, 256, 64, 64, 8, 0, False, 320), (8, 0, 300, 0, 64, 4, 0, "aligned", 0), (8, 11, 270, 0, 64, 8, 0, True, 0),
                # enough queries for blocks of eight waves (sixteen queries per block at this group size)
                (8, 100, 523, 64, 64, 8, 0, False, 0), (4, 0, 513, 0, 64, 8, 0, False, 0)]:
            if act == 1 and (bits == 4 or chunk > 512):
                continue                                            # the fp16 context repeats the 8- and 16-bit cases only
            ctx = nv.Context(0, act)
            say("prefill attention long chunk", act, bits, start, chunk, window, nq, nkv, extra, pad, ring)
            _prefill_case(nv, ctx, 0xFA00 + start + chunk, bits, start, chunk, window, 256, nq, nkv, extra_kv=extra, pad=pad,
                          ring=ring, lo=-1.0, hi=1.0, scale=1.0 / 16.0)
            keys = min(start + chunk, window + chunk) if window else start + chunk
            scratch = 2 * (keys // 32 * 32) * nkv * 256 * 2          # at least: K rows and V^T rows of the key range
            assert (ctx.workspace_bytes >= scratch) == (pad is not True), ctx.workspace_bytes
            ctx.close()


def _two_forms_cases():
    cases = [(8, 777, 1500, 0), (4, 1000, 4100, 2000), (8, 0, 4096, 0), (4, 2049, 1100, 333)]
    rng = np.random.default_rng(20240521)
    for _ in range(10):                                             # seeded draws: starts, counts and windows off every grid
        chunk = int(rng.integers(1024, 2300))
        start = int(rng.integers(0, 3000))
        window = int(rng.choice([0, 0, int(rng.integers(1, 64)), int(rng.integers(64, 2500))]))
        cases.append((int(rng.choice([4, 8])), start, chunk, window))
    return cases


@pytest.mark.parametrize("bits,start,chunk,window", _two_forms_cases())
def test_prefill_attention_two_forms_agree(nv, bits, start, chunk, window):
    # size-independent property at sizes the scalar oracle cannot walk: the same chunk through the two-launch
    # form (fp16 scratch + flash attention, four- and eight-wave blocks) and through the one-launch kernels that
    # multiply the codes -- reached by giving q and out rows that do not start at 16-byte boundaries -- agree
    # to the bar both are held to against the oracle; starts and windows that are no multiples of the 32-key
    # tile, query counts that leave dead waves and dead columns in the last block
    say("prefill attention two forms", bits, start, chunk, window)
    ctx = nv.Context(0, 0)
    gen = torch.Generator(device="cuda").manual_seed(300 + bits + chunk)
    nq, nkv, hd = 16, 2, 256
    kv_valid, row = start + chunk, nq * hd
    kc, vc, _ = _long_cache(nv, ctx, gen, 1, kv_valid, nkv * hd, bits)
    q = torch.randn((chunk, row), generator=gen, device="cuda", dtype=torch.float32).to(ctx.dtype)
    pa = nv.PrefillAttention(ctx)
    out_a = torch.empty_like(q)
    pa.encode_causal(q, kc.view(), vc.view(), out_a, start, chunk, hd, nq, nkv, kv_valid, sliding_window=window)
    assert ctx.workspace_bytes >= 2 * (min(kv_valid, window + chunk) if window else kv_valid) // 32 * 32 * nkv * hd * 2
    other = nv.Context(0, 0)                                        # a context of its own: its workspace stays empty
    q_buf = torch.zeros(1 + chunk * row, dtype=ctx.dtype, device="cuda")
    q_buf[1:].view(chunk, row).copy_(q)
    out_buf = torch.zeros(1 + chunk * row, dtype=ctx.dtype, device="cuda")
    nv.PrefillAttention(other).encode_causal(q_buf[1:], kc.view(), vc.view(), out_buf[1:], start, chunk, hd, nq, nkv, kv_valid,
                                             sliding_window=window)
    torch.cuda.synchronize()
    assert other.workspace_bytes < 1 << 20
    a, b = act_np(out_a), act_np(out_buf[1:].view(chunk, row))
    assert np.isfinite(a).all()
    assert O.rel_error(a, b) < 1e-2
    # row by row as well: no query may be off while the whole chunk looks right
    worst = max(O.rel_error(a[t], b[t]) for t in range(0, chunk, 37))
    assert worst < 2e-2, worst
    ctx.close()
    other.close()


@pytest.mark.parametrize("bits", [8, 4])
def test_prefill_attention_chunk_equals_decode_steps(nv, bits):
    # size-independent property at a prefill size the scalar oracle cannot walk: query t of a
    # 512-token chunk at the end of an 8K context is the decode call with seq_len = start + t + 1
    # (the same kernels, a different packing of queries into blocks), and the oracle agrees on a few rows
    say("prefill chunk vs decode", bits)
    ctx = nv.Context(0, 0)
    gen = torch.Generator(device="cuda").manual_seed(11 + bits)
    nq, nkv, hd, start, chunk = 16, 2, 256, 7680, 512
    kv_valid, elements = start + chunk, nkv * hd
    kc, vc, _ = _long_cache(nv, ctx, gen, 1, kv_valid, elements, bits)
    q = torch.randn((chunk, nq, hd), generator=gen, device="cuda", dtype=torch.float32).to(ctx.dtype)
    out = torch.empty_like(q)
    nv.PrefillAttention(ctx).encode_causal(q, kc.view(), vc.view(), out, start, chunk, hd, nq, nkv, kv_valid)
    att = nv.Attention(ctx)
    kq, vq = kc.rows[0].cpu().numpy(), vc.rows[0].cpu().numpy()
    for t in (0, 1, 255, 510, 511):
        one = att.encode_full(q[t:t + 1], kc, vc, hd, nq, nkv, start + t + 1)
        torch.cuda.synchronize()
        assert O.rel_error(act_np(out[t]), act_np(one[0])) < 1e-2       # two bf16 roundings of differently ordered sums
    for t in (0, 511):
        want = O.attention_decode(act_np(q[t]), kq, vq, bits, nq, nkv, hd, start + t + 1, 1 / 16.0)
        assert O.rel_error(act_np(out[t]), want) < 1e-2
    # ragged decode: the same rows again, every query as its own "sequence" of the one cache
    lens = torch.arange(start + 1, start + chunk + 1, device="cuda", dtype=torch.int32)
    ragged = att.encode_ragged(q, _Shared(kc), _Shared(vc), hd, nq, nkv, lens, kv_valid)
    torch.cuda.synchronize()
    assert O.rel_error(act_np(ragged), act_np(out)) < 1e-2
    ctx.close()


class _Shared:
    """A cache whose every sequence is sequence 0 (batch stride 0)."""

    def __init__(self, cache):
        self.cache, self.batch_stride = cache, 0

    def view(self):
        return self.cache.view()


def test_attention_ragged_batch(nv, ctx):
    # sequences of different lengths and starts in one call, an empty one included
    say("attention ragged", ctx.act)
    rng = np.random.default_rng(41)
    nq, nkv, hd, batch, cap = 16, 2, 256, 5, 700
    for bits in (8, 4, 16):
        elements = nkv * hd
        q = round_act(gauss(rng, (batch, nq, hd)), ctx.act)
        k = round_act(gauss(rng, (batch, cap, elements)), ctx.act)
        v = round_act(gauss(rng, (batch, cap, elements)), ctx.act)
        kc, vc = nv.KVCache(batch, cap, elements, bits), nv.KVCache(batch, cap, elements, bits)
        if bits == 16:
            kc.rows.copy_(dev(k).to(torch.float16).view(torch.uint8).view(batch, cap, -1))
            vc.rows.copy_(dev(v).to(torch.float16).view(torch.uint8).view(batch, cap, -1))
        else:
            quant = nv.KVCacheQuantizer(ctx)
            for b in range(batch):
                quant.encode(act_tensor(k[b], ctx), elements, kc.view(b), cap, elements)
                quant.encode(act_tensor(v[b], ctx), elements, vc.view(b), cap, elements)
        lens = np.array([700, 1, 333, 64, 0], np.uint32)
        starts = np.array([0, 0, 300, 63, 0], np.uint32)
        for use_starts in (False, True):
            out = nv.Attention(ctx).encode_ragged(act_tensor(q, ctx), kc, vc, hd, nq, nkv,
                                                  dev(lens.view(np.int32)), cap,
                                                  kv_starts=dev(starts.view(np.int32)) if use_starts else None)
            torch.cuda.synchronize()
            got = act_np(out)
            for b in range(batch):
                s0 = int(starts[b]) if use_starts else 0
                if bits == 16:
                    want = O.attention_decode(q[b], O.f16_to_float(O.f16_bits(k[b])), O.f16_to_float(O.f16_bits(v[b])),
                                              32, nq, nkv, hd, int(lens[b]), 1 / 16.0, s0)
                else:
                    want = O.attention_decode(q[b], kc.rows[b].cpu().numpy(), vc.rows[b].cpu().numpy(), bits, nq, nkv,
                                              hd, int(lens[b]), 1 / 16.0, s0)
                if lens[b] == 0:
                    assert not got[b].any() and not want.any()
                else:
                    assert O.rel_error(got[b], want) < 1e-2, (bits, b)


def test_prefill_attention_rejects_what_validate_rejects(nv, ctx):
    say("prefill attention errors")
    kc, vc = nv.KVCache(1, 16, 512, 8), nv.KVCache(1, 16, 512, 8)
    q = torch.zeros((4, 16 * 256), dtype=ctx.dtype, device="cuda")
    out = torch.zeros_like(q)
    pa = nv.PrefillAttention(ctx)
    for kwargs in (dict(q_token_stride=100), dict(o_token_stride=100)):       # PrefillAttention.swift:176-179
        with pytest.raises(nv.NvmaiError) as e:
            pa.encode_causal(q, kc.view(), vc.view(), out, 0, 4, 256, 16, 2, 4, **kwargs)
        assert e.value.name == "invalid_arg"
    with pytest.raises(nv.NvmaiError) as e:                                      # :189-190
        pa.encode_causal(q, kc.view(), vc.view(), out, 2, 4, 256, 16, 2, 5)
    assert e.value.name == "invalid_arg"
    with pytest.raises(nv.NvmaiError) as e:                                      # queryCount must be positive
        pa.encode_causal(q, kc.view(), vc.view(), out, 0, 0, 256, 16, 2, 4)
    assert e.value.name == "invalid_arg"
    with pytest.raises(nv.NvmaiError) as e:                                      # :174-175
        pa.encode_causal(q, kc.view(), vc.view(), out, 0, 4, 256, 15, 2, 4)
    assert e.value.name == "invalid_arg"


@pytest.mark.parametrize("bits", [8, 4])
def test_attention_with_output_gate_equals_the_two_calls(nv, ctx, bits):
    # attention + sigmoid output gate in the same launches: the bits of encode_full followed by
    # encode_sigmoid_gate_mul, at a context with many chunks and at one that fits one chunk
    # (where the ungated call writes its rows from the partial kernel), and against the oracle
    say("attention with output gate", ctx.act, bits)
    rng = np.random.default_rng(77 + bits)
    nq, nkv, hd = 16, 2, 256
    attn, ew, quant = nv.Attention(ctx), nv.Elementwise(ctx), nv.KVCacheQuantizer(ctx)
    for batch, seq in ((3, 1500), (2, 96), (1, 1)):
        elements = nkv * hd
        q = round_act(gauss(rng, (batch, nq, hd)), ctx.act)
        gate = round_act(gauss(rng, (batch, nq, hd)) * 2.0, ctx.act)
        kc, vc = nv.KVCache(batch, seq, elements, bits), nv.KVCache(batch, seq, elements, bits)
        ks, vs = [], []
        for b in range(batch):
            k = round_act(gauss(rng, (seq, elements)), ctx.act)
            v = round_act(gauss(rng, (seq, elements)), ctx.act)
            quant.encode(act_tensor(k, ctx), elements, kc.view(b), seq, elements)
            quant.encode(act_tensor(v, ctx), elements, vc.view(b), seq, elements)
            ks.append(k); vs.append(v)
        qd, gd = act_tensor(q, ctx), act_tensor(gate, ctx)
        two = attn.encode_full(qd, kc, vc, hd, nq, nkv, seq)
        ew.encode_sigmoid_gate_mul(two, gd)
        one = attn.encode_full_gated(qd, kc, vc, gd, hd, nq, nkv, seq)
        torch.cuda.synchronize()
        assert torch.equal(one.view(torch.int16), two.view(torch.int16))
        for b in range(batch):
            want = O.attention_decode(q[b], O.kv_quantize(ks[b], bits), O.kv_quantize(vs[b], bits), bits, nq, nkv, hd,
                                      seq, 1.0 / np.sqrt(hd))
            want = O.elementwise(O.EW_SIGMOID_MUL, round_act(want, ctx.act), gate[b])
            assert O.rel_error(act_np(one[b]), want) < 1e-2
    # the gate is required and must cover a row
    import ctypes as C
    qd = act_tensor(round_act(gauss(rng, (1, nq, hd)), ctx.act), ctx)
    kc = nv.KVCache(1, 8, nkv * hd, bits)
    kview = kc.view()
    for gate_ptr, gate_stride in ((None, nq * hd), (qd.data_ptr(), 16)):
        rc = nv.lib.nvmai_hip_attention_decode_gated(ctx.handle, None, qd.data_ptr(), C.byref(kview), C.byref(kview), 0,
                                                     qd.data_ptr(), gate_ptr, gate_stride, 1, hd, nq, nkv, 8, 0, 0.0)
        assert rc != 0
