"""GPU parity: RMSNorm, affine embedding lookup and the fused greedy LM head through the C ABI.

All three are compared bit for bit: the oracle states the summation order the kernels use, every
other step is one IEEE operation, and the greedy token is an index."""
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


def _act_bits(a, act):
    return O.bf16_bits(a) if act == 0 else O.f16_bits(a)


def _bits(t):
    """The 16-bit patterns of an activation tensor."""
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("rows,d", [(1, 256), (1, 2048), (16, 2048), (300, 2048), (3, 2816), (16, 256), (5, 100), (9, 64)])
def test_rmsnorm_bit_exact(nv, ctx, rows, d):
    say("rmsnorm", ctx.act, rows, d)
    rng = np.random.default_rng(rows * 31 + d)
    x = round_act(rng.uniform(-1, 1, (rows, d)).astype(np.float32), ctx.act)
    w = O.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32))
    rms = nv.RMSNorm(ctx)
    got_w = _bits(rms.encode_bf16w(act_tensor(x, ctx), dev(w.view(np.int16))))
    got_n = _bits(rms.encode_no_scale(act_tensor(x, ctx)))
    torch.cuda.synchronize()
    assert np.array_equal(got_w, _act_bits(O.rmsnorm(x, w, 1e-6), ctx.act))
    assert np.array_equal(got_n, _act_bits(O.rmsnorm(x, None, 1e-6), ctx.act))
    # the reference's bar against an independent formulation (Tolerance.fp16Reduction, RMSNormTests.swift:53)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-6) * O.bf16_to_float(w).astype(np.float64)
    got_f = act_np(rms.encode_bf16w(act_tensor(x, ctx), dev(w.view(np.int16))))
    assert np.abs(got_f - want).max() / np.abs(want).max() < 5e-3


def test_rmsnorm_per_head_in_place_known_answer(nv, ctx):
    # RMSNormTests.swift:119-165: head h is the constant h + 1, unit weights, in place -> all ones;
    # rows further apart than head_dim (a padded stride) leave the padding alone
    say("rmsnorm per head", ctx.act)
    heads, hd, stride = 16, 256, 256 + 8
    buf = torch.full((heads, stride), 5.0, dtype=ctx.dtype, device="cuda")
    buf[:, :hd] = torch.arange(1, heads + 1, dtype=torch.float32, device="cuda")[:, None].to(ctx.dtype)
    view = buf[:, :hd]
    unit = dev(O.bf16_bits(np.ones(hd, np.float32)).view(np.int16))
    nv.RMSNorm(ctx).encode_bf16w_per_head(view, unit, out=view)
    torch.cuda.synchronize()
    out = buf.float().cpu().numpy()
    assert np.abs(out[:, :hd] - 1.0).max() < 1e-2
    assert (out[:, hd:] == 5.0).all()
    assert nv.lib.nvmai_hip_rmsnorm(ctx.handle, None, None, 8, None, None, 8, 1, 8, 1e-6) == -1    # no buffers


# ------------------------------------------------------------------ embedding lookup
@pytest.mark.parametrize("bits", [4, 8])
def test_embed_lookup_bit_exact_and_known_answer(nv, ctx, bits):
    say("embed", ctx.act, bits)
    # AffineQuantTests.swift:58-79: bit-stream table, scale 1, bias 0 -> the values themselves
    rows, cols = 3, 128
    mask = (1 << bits) - 1
    values = np.array([[(r * 11 + c * 3) & mask for c in range(cols)] for r in range(rows)], np.float32)
    packed = np.zeros((rows, cols * bits // 8), np.uint8)
    for r in range(rows):
        for c in range(cols):
            packed[r, c * bits // 8] |= (int(values[r, c]) << ((c * bits) % 8)) & 0xFF
    one = dev(np.full((rows, 2), 0x3F80, np.uint16).view(np.int16))
    zero = dev(np.zeros((rows, 2), np.int16))
    emb = nv.AffineQuantEmbeddingLookup(ctx, bits)
    got = act_np(emb.encode(dev(packed), one, zero, 1, cols, rows))
    torch.cuda.synchronize()
    assert np.array_equal(got[0], values[1])
    # random table, a block of token ids with one out of range, output scale, padded rows
    rng = np.random.default_rng(50 + bits)
    vocab, d = 37, 2048 + 64
    p, s, b = O.quantize_affine(gauss(rng, (vocab, d), 0.05), bits)
    ids = np.array([0, 36, 5, 37, 12, 0xFFFFFFFF, 5], np.uint32)
    out = torch.full((len(ids), d + 16), 3.0, dtype=ctx.dtype, device="cuda")
    emb.encode(dev(p), dev(s.view(np.int16)), dev(b.view(np.int16)), dev(ids.view(np.int32)), d, vocab, 45.25, out)
    torch.cuda.synchronize()
    got = _bits(out)
    for t, tok in enumerate(ids):
        assert np.array_equal(got[t, :d], _act_bits(O.embed_lookup(p, s, b, bits, int(tok), 45.25), ctx.act))
    assert (out[:, d:].float() == 3.0).all()
    assert not got[3, :d].any() and not got[5, :d].any()
    with pytest.raises(nv.NvmaiError) as e:
        nv.AffineQuantEmbeddingLookup(ctx, 6)
    assert e.value.name == "unsupported"


# ------------------------------------------------------------------ greedy LM head
def _const_rows(v, d, special, hi, lo, bits=4):
    w = np.full((v, d), lo, np.float32)
    for r in special:
        w[r] = hi
    return O.quantize_affine(w, bits)


def _head_dev(p, s, b):
    return dev(p), dev(s.view(np.int16)), dev(b.view(np.int16))


def test_greedy_head_reference_known_answers(nv, ctx):
    # LMHeadChainInt4Tests.swift:136-224
    say("greedy head known answers", ctx.act)
    d = 64
    unit = dev(O.bf16_bits(np.ones(d, np.float32)).view(np.int16))
    chain = nv.LMHeadChain(ctx, 4)
    hidden = round_act((0.25 + (np.arange(d) % 7) * 0.01).astype(np.float32), ctx.act)
    for v in (1024, 2048, 4096):
        p, s, b = _const_rows(v, d, [v - 3], 1.0, -0.5)
        tok = chain.encode_greedy_decode(act_tensor(hidden[None], ctx), unit, *_head_dev(p, s, b), d, v)
        assert int(tok[0]) == v - 3
    hidden = round_act((0.2 + (np.arange(d) % 5) * 0.02).astype(np.float32), ctx.act)
    p, s, b = _const_rows(1024, d, [17, 311], 1.0, -0.25)
    tok = chain.encode_greedy_decode(act_tensor(hidden[None], ctx), unit, *_head_dev(p, s, b), d, 1024)
    assert int(tok[0]) == 17                                    # ties resolve to the lowest index
    p, s, b = _const_rows(1024, d, [], 0.25, 0.25)
    nan = torch.full((1, d), float("nan"), dtype=ctx.dtype, device="cuda")
    tok = chain.encode_greedy_decode(nan, unit, *_head_dev(p, s, b), d, 1024)
    assert int(tok[0]) == 0                                     # no finite candidate
    # the selected row of a strided hidden buffer (:195-224)
    rows = np.stack([(0.25 + (np.arange(d) % 7) * 0.01) if r == 3 else (-0.4 - (np.arange(d) % 5) * 0.01)
                     for r in range(5)]).astype(np.float32)
    hbuf = torch.zeros((5, d + 16), dtype=ctx.dtype, device="cuda")
    hbuf[:, :d] = act_tensor(rows, ctx)
    p, s, b = _const_rows(1024, d, [777], 1.0, -0.25)
    tok = chain.encode_greedy_decode(hbuf[3:4, :d], unit, *_head_dev(p, s, b), d, 1024)
    assert int(tok[0]) == 777


@pytest.mark.parametrize("bits,d,v,tokens", [(4, 2048, 5000, 3), (8, 2048, 3001, 2), (4, 4096, 700, 1),
                                             (8, 1024, 999, 1), (4, 192, 130, 4), (8, 64, 70, 1)])
def test_greedy_head_token_equals_oracle(nv, ctx, bits, d, v, tokens):
    # random rows, nothing separated on purpose: near-ties must fall the same way as in the oracle
    say("greedy head", ctx.act, bits, d, v, tokens)
    rng = np.random.default_rng(bits * 1000 + d + v)
    p, s, b = O.quantize_affine(gauss(rng, (v, d), 0.02), bits)
    p[v // 2] = p[v // 3]; s[v // 2] = s[v // 3]; b[v // 2] = b[v // 3]          # two identical rows
    hidden = round_act(gauss(rng, (tokens, d)), ctx.act)
    nw = O.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32))
    chain = nv.LMHeadChain(ctx, bits)
    hd = _head_dev(p, s, b)
    got = u32(chain.encode_greedy_decode(act_tensor(hidden, ctx), dev(nw.view(np.int16)), *hd, d, v))
    got_raw = u32(chain.encode_greedy_decode(act_tensor(hidden, ctx), None, *hd, d, v))
    torch.cuda.synchronize()
    for t in range(tokens):
        assert got[t] == O.lm_head_greedy(hidden[t], nw, p, s, b, bits, act=ctx.act)
        assert got_raw[t] == O.lm_head_greedy(hidden[t], None, p, s, b, bits, act=ctx.act)


def test_greedy_head_rejects_bad_arguments(nv, ctx):
    say("greedy head errors", ctx.act)
    w = torch.zeros(64 * 64, dtype=torch.uint8, device="cuda")
    s = torch.zeros(64, dtype=torch.int16, device="cuda")
    h = torch.zeros((1, 128), dtype=ctx.dtype, device="cuda")
    with pytest.raises(nv.NvmaiError) as e:
        nv.LMHeadChain(ctx, 4).encode_greedy_decode(h[:, :100], None, w, s, s, 100, 64)     # d % 64 != 0
    assert e.value.name == "invalid_arg"
    with pytest.raises(nv.NvmaiError) as e:
        nv.LMHeadChain(ctx, 8).encode_greedy_decode(h, None, w[1:], s, s, 128, 8)            # misaligned rows
    assert e.value.name == "alignment"
    with pytest.raises(nv.NvmaiError) as e:
        nv.LMHeadChain(ctx, 6)
    assert e.value.name == "unsupported"


# ------------------------------------------------------------------ elementwise helpers
def _ulp16_apart(got_bits, want_bits):
    """Largest distance in 16-bit patterns (same sign assumed where values are not tiny)."""
    return np.abs(got_bits.astype(np.int32) - want_bits.astype(np.int32)).max()


def test_elementwise_helpers_match_oracle(nv, ctx):
    say("elementwise", ctx.act)
    rng = np.random.default_rng(77)
    n = 5000
    a = round_act(gauss(rng, (n,), 3.0), ctx.act)
    b = round_act(gauss(rng, (n,), 3.0), ctx.act)
    ew = nv.Elementwise(ctx)
    got = _bits(ew.encode_silu_mul(act_tensor(a, ctx), act_tensor(b, ctx)))
    # exp comes from two different libraries: at most one 16-bit ulp apart, and within the 1e-2 bar
    want = O.elementwise(O.EW_SILU_MUL, a, b)
    assert _ulp16_apart(got, _act_bits(want, ctx.act)) <= 1
    got = ew.encode_sigmoid_gate_mul(act_tensor(a, ctx), act_tensor(b, ctx))
    assert _ulp16_apart(_bits(got), _act_bits(O.elementwise(O.EW_SIGMOID_MUL, a, b), ctx.act)) <= 1
    assert O.rel_error(act_np(got), O.elementwise(O.EW_SIGMOID_MUL, a, b)) < 1e-2
    got = ew.encode_sigmoid_scalar_mul(act_tensor(a, ctx), act_tensor(b[:1], ctx))
    assert _ulp16_apart(_bits(got), _act_bits(O.elementwise(O.EW_SIGMOID_SCALAR, a, b), ctx.act)) <= 1
    # one IEEE addition, one rounding: bit-exact
    got = ew.encode_residual_add(act_tensor(a, ctx), act_tensor(b, ctx))
    assert np.array_equal(_bits(got), _act_bits(O.elementwise(O.EW_ADD, a, b), ctx.act))
    # data movement: bit-exact
    heads, dim = 16, 256
    packed = round_act(gauss(rng, (heads, 2 * dim)), ctx.act)
    q, g = ew.encode_split_q_gate(act_tensor(packed, ctx), heads, dim)
    wq, wg = O.split_q_gate(packed, heads, dim)
    assert np.array_equal(act_np(q), wq) and np.array_equal(act_np(g), wg)
    assert np.array_equal(act_np(ew.encode_concat_rows(q, g)), packed)
    torch.cuda.synchronize()
    assert nv.lib.nvmai_hip_silu_mul(ctx.handle, None, None, None, None, 4) == -1


def test_elementwise_helpers_in_16_byte_pieces_same_bits(nv, ctx):
    # 4096 values and more in 16-byte-aligned buffers go eight per thread; the same values in buffers
    # that start two bytes later take the one-value-per-thread kernels: same bits from both
    say("elementwise pieces", ctx.act)
    rng = np.random.default_rng(78)
    n = 8192
    a = round_act(gauss(rng, (n,), 3.0), ctx.act)
    b = round_act(gauss(rng, (n,), 3.0), ctx.act)
    ew = nv.Elementwise(ctx)

    def shifted(x):                       # the same values, first element two bytes past a 16-byte boundary
        t = torch.zeros(n + 8, dtype=ctx.dtype, device="cuda")
        t[1:n + 1] = act_tensor(x, ctx)
        return t[1:n + 1]

    for op in ("silu", "gate", "scalar", "add"):
        outs = []
        for make in (lambda x: act_tensor(x, ctx).clone(), shifted):
            ta, tb = make(a), make(b)
            if op == "silu":
                outs.append(ew.encode_silu_mul(ta, tb, out=make(a)))
            elif op == "gate":
                outs.append(ew.encode_sigmoid_gate_mul(ta, tb))
            elif op == "scalar":
                outs.append(ew.encode_sigmoid_scalar_mul(ta, tb[:1]))
            else:
                outs.append(ew.encode_residual_add(ta, tb))
        torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]), op


# ------------------------------------------------------------------ q / k / v epilogue
def _qkv_epilogue_case(nv, ctx, rng, tokens, nq, nkv, hd, rot, pad):
    span = 2 * nq * hd + 2 * nkv * hd
    proj = np.zeros((tokens, span + pad), np.float32)
    proj[:, :span] = round_act(gauss(rng, (tokens, span)), ctx.act)
    qw = O.bf16_bits(1.0 + 0.1 * gauss(rng, (hd,)))
    kw = O.bf16_bits(1.0 + 0.1 * gauss(rng, (hd,)))
    positions = rng.integers(0, 5000, tokens).astype(np.uint32)
    return proj, qw, kw, positions


def _run_epilogue(nv, ctx, proj, qw, kw, positions, nq, nkv, hd, rot, kviews=None, stage=True):
    import ctypes as C
    tokens = proj.shape[0]
    pd = act_tensor(proj, ctx)
    q = torch.zeros((tokens, nq, hd), dtype=pd.dtype, device="cuda")
    gate, k, v = torch.zeros_like(q), torch.zeros((tokens, nkv * hd), dtype=pd.dtype, device="cuda"), None
    v = torch.zeros_like(k)
    ptr = lambda t: None if t is None else t.data_ptr()
    qwd, kwd, posd = dev(qw), dev(kw), dev(positions)       # held until the call has run
    args = [ctx.handle, None, pd.data_ptr(), pd.stride(0), 1, qwd.data_ptr(), kwd.data_ptr(), q.data_ptr(),
            gate.data_ptr(), ptr(k if stage else None), ptr(v if stage else None), nkv * hd]
    tail = [tokens, nq, nkv, hd, rot, 0, posd.data_ptr(), 0, 1e4, 1e-6]
    if kviews is None:
        rc = nv.lib.nvmai_hip_attn_qkv_epilogue(*args, *tail)
    else:
        rc = nv.lib.nvmai_hip_attn_qkv_epilogue_kv(*args, C.byref(kviews[0]), C.byref(kviews[1]), *tail)
    torch.cuda.synchronize()
    return rc, q, gate, k, v


@pytest.mark.parametrize("tokens,nq,nkv,hd,rot", [(1, 16, 2, 256, 64), (5, 4, 2, 64, 16), (3, 6, 3, 128, 128), (2, 3, 1, 40, 8)])
def test_qkv_epilogue_equals_the_separate_operators(nv, ctx, tokens, nq, nkv, hd, rot):
    # split + per-head RMSNorm (q, k) + partial RoPE (q, k) in one launch: the bits of the oracle's
    # operators applied one after the other with a 16-bit hand-over between them
    say("qkv epilogue", ctx.act, tokens, nq, nkv, hd, rot)
    rng = np.random.default_rng(500 + hd + tokens)
    proj, qw, kw, positions = _qkv_epilogue_case(nv, ctx, rng, tokens, nq, nkv, hd, rot, pad=8)
    rc, q, gate, k, v = _run_epilogue(nv, ctx, proj, qw, kw, positions, nq, nkv, hd, rot)
    assert rc == 0
    r = lambda a: round_act(a, ctx.act)
    for t in range(tokens):
        want_q, want_gate = O.split_q_gate(proj[t, :2 * nq * hd], nq, hd)
        want_k = proj[t, 2 * nq * hd:2 * nq * hd + nkv * hd].reshape(nkv, hd)
        want_v = proj[t, 2 * nq * hd + nkv * hd:2 * nq * hd + 2 * nkv * hd]
        want_q = r(O.rmsnorm(want_q, qw, 1e-6))
        want_k = r(O.rmsnorm(want_k, kw, 1e-6))
        want_q = O.rope_neox_subdim(want_q[None], rot, positions[t:t + 1], 1e4)[0]
        want_k = O.rope_neox_subdim(want_k[None], rot, positions[t:t + 1], 1e4)[0]
        assert np.array_equal(_bits(gate[t]).reshape(nq, hd), _act_bits(want_gate, ctx.act))
        assert np.array_equal(_bits(v[t]), _act_bits(want_v, ctx.act))
        # the rotation's sine and cosine come from two libraries: one 16-bit ulp
        assert O.rel_error(act_np(q[t]), want_q) < 1e-2 and O.rel_error(act_np(k[t]).reshape(nkv, hd), want_k) < 1e-2
        unrot = slice(rot, hd)
        assert np.array_equal(_bits(q[t])[:, unrot], _act_bits(r(want_q), ctx.act)[:, unrot])


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("tokens,nq,nkv,hd,rot", [(1, 16, 2, 256, 64), (4, 4, 2, 64, 16), (3, 6, 3, 128, 128)])
def test_qkv_epilogue_with_kv_write_equals_the_separate_calls(nv, ctx, bits, tokens, nq, nkv, hd, rot):
    # the epilogue that also quantizes the finished k and v rows into the cache: q, gate and the
    # cache rows are the bits of the epilogue followed by two KVCacheQuantizer.encode calls, with
    # and without the 16-bit stage rows; the codes also equal the oracle's for the GPU's own rows
    say("qkv epilogue + kv write", ctx.act, bits, tokens, nq, nkv, hd, rot)
    rng = np.random.default_rng(900 + hd + tokens + bits)
    proj, qw, kw, positions = _qkv_epilogue_case(nv, ctx, rng, tokens, nq, nkv, hd, rot, pad=0)
    elements = nkv * hd
    rc, q0, gate0, k0, v0 = _run_epilogue(nv, ctx, proj, qw, kw, positions, nq, nkv, hd, rot)
    assert rc == 0
    quant = nv.KVCacheQuantizer(ctx)
    ref_k, ref_v = nv.KVCache(1, tokens + 2, elements, bits), nv.KVCache(1, tokens + 2, elements, bits)
    quant.encode(k0, elements, ref_k.view(0, 1), tokens, elements)
    quant.encode(v0, elements, ref_v.view(0, 1), tokens, elements)
    for stage in (True, False):
        kc, vc = nv.KVCache(1, tokens + 2, elements, bits), nv.KVCache(1, tokens + 2, elements, bits)
        rc, q1, gate1, k1, v1 = _run_epilogue(nv, ctx, proj, qw, kw, positions, nq, nkv, hd, rot,
                                              kviews=(kc.view(0, 1), vc.view(0, 1)), stage=stage)
        assert rc == 0
        assert torch.equal(q1.view(torch.int16), q0.view(torch.int16)) and torch.equal(gate1.view(torch.int16), gate0.view(torch.int16))
        if stage:
            assert torch.equal(k1.view(torch.int16), k0.view(torch.int16)) and torch.equal(v1.view(torch.int16), v0.view(torch.int16))
        else:
            assert int(k1.view(torch.int16).abs().max()) == 0      # untouched
        assert torch.equal(kc.rows, ref_k.rows) and torch.equal(vc.rows, ref_v.rows)
        stride = kc.rows.shape[-1]
        want = O.kv_quantize(act_np(k0), bits)
        assert np.array_equal(kc.rows[0, 1:1 + tokens].cpu().numpy()[:, :want.shape[1]], want[:, :stride])


def test_qkv_epilogue_with_kv_write_rejects_bad_arguments(nv, ctx):
    rng = np.random.default_rng(5)
    tokens, nq, nkv, hd, rot = 2, 4, 2, 40, 8
    proj, qw, kw, positions = _qkv_epilogue_case(nv, ctx, rng, tokens, nq, nkv, 64, rot, pad=0)
    kc, vc = nv.KVCache(1, 4, nkv * 64, 8), nv.KVCache(1, 4, nkv * 64, 4)
    # views of two formats
    rc = _run_epilogue(nv, ctx, proj, qw, kw, positions, nq, nkv, 64, rot, kviews=(kc.view(0, 0), vc.view(0, 0)))[0]
    assert rc != 0
    # a head that is not whole groups of 64
    proj, qw, kw, positions = _qkv_epilogue_case(nv, ctx, rng, tokens, nq, nkv, hd, rot, pad=0)
    k40 = nv.KVCache(1, 4, 128, 8)
    rc = _run_epilogue(nv, ctx, proj, qw, kw, positions, nq, nkv, hd, rot, kviews=(k40.view(0, 0), k40.view(0, 0)))[0]
    assert rc != 0
