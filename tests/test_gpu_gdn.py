"""GPU parity: gated-DeltaNet linear attention (conv + q / k norm, delta rule + gated output norm), the
fused residual add + RMSNorm, the fused input projections and the dense BF16 GEMV, through the C ABI
against the CPU oracle.

GDN bars, both asserted for every comparison of outputs:
 * max|got - want| / max|want| < 1e-2 (the measure and the 16-bit bar of this build, RelError.swift:5-16);
   measured: fp16 activations <= 5e-4, bf16 activations <= 3.2e-3, bf16 activations with the BF16 state
   <= 5.9e-3 (the oracle then rounds its own state to BF16 after every token, as the kernels store it);
 * the reference's own per-element bar for its kernels against its CPU model (GDNKernelTests.swift:170-185),
   |got - want| <= max(2e-2, 4e-2 |want|), with fp16 AND with bf16 activations (measured: no element uses
   more than a quarter of it), and 5e-2 on the fp32 recurrent state."""
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


def _fixture(cfg, rows, seed, act):
    kh, vh, dk, dv, taps = cfg
    C = 2 * kh * dk + vh * dv
    rng = np.random.default_rng(seed)
    u = lambda lo, hi, n: rng.uniform(lo, hi, n).astype(np.float32)
    r = lambda a: round_act(a, act)
    return dict(conv_w=O.bf16_bits(u(-0.4, 0.4, C * taps)), a_log=O.bf16_bits(u(-1.0, 1.5, vh)),
                dt_bias=O.bf16_bits(u(-0.5, 0.5, vh)), norm_w=O.bf16_bits(u(0.5, 1.5, dv)),
                qkv=r(u(-1, 1, rows * C)).reshape(rows, C), a=r(u(-1, 1, rows * vh)).reshape(rows, vh),
                b=r(u(-1, 1, rows * vh)).reshape(rows, vh), z=r(u(-1, 1, rows * vh * dv)).reshape(rows, vh * dv))


def _bits(a):
    return dev(np.ascontiguousarray(a).view(np.int16))


MEASURED = []          # (label, max|diff| / max|ref|, worst element as a fraction of its bar)


def _rel(got, want):
    """The measure the tolerances of this build are stated in: max|got - want| / max|want| (RelError.swift:5-16)."""
    return float(np.abs(got - want).max() / max(float(np.abs(want).max()), 1e-30))


def _close(got, want, act, label=""):
    lo, rel = 2e-2, 4e-2                                   # GDNKernelTests.swift:170-185, for both activation types
    use = float((np.abs(got - want) / np.maximum(lo, np.abs(want) * rel)).max())
    MEASURED.append((label, _rel(got, want), use))
    print("[measure] gdn %-28s act=%d max|d|/max|ref| %.3e  worst element at %.2f of its bar" % (label, act, MEASURED[-1][1], use),
          flush=True)
    return use <= 1.0 and MEASURED[-1][1] < 1e-2


def _gpu_rows(nv, ctx, gdn, fx, tail, state, t0, rows, batch_rows=None):
    """rows tokens of one sequence (or of each sequence when batch_rows is given) in one call."""
    sl = slice(t0, t0 + rows)
    conv = gdn.encode_conv_norm(act_tensor(fx["qkv"][sl], ctx), tail, _bits(fx["conv_w"]), rows=rows)
    return gdn.encode_delta_gated_norm(conv, act_tensor(fx["a"][sl], ctx), act_tensor(fx["b"][sl], ctx),
                                       _bits(fx["a_log"]), _bits(fx["dt_bias"]), state, act_tensor(fx["z"][sl], ctx),
                                       _bits(fx["norm_w"]), rows=rows)


@pytest.mark.parametrize("cfg", [(2, 4, 32, 32, 4), (16, 32, 128, 128, 4), (2, 2, 64, 64, 2), (1, 2, 64, 128, 3)],
                         ids=["reference-toy", "production", "dk64", "dk64-dv128"])
def test_gdn_decode_chain_matches_oracle(nv, ctx, cfg):
    # decodeChainMatchesReference (GDNKernelTests.swift:130-187): six tokens, outputs, tail and state
    say("gdn decode chain", ctx.act, cfg)
    rows = 6
    fx = _fixture(cfg, rows, 0x51D, ctx.act)
    gdn = nv.GDN(ctx, *cfg)
    tail, state = gdn.new_state()
    ref = O.GdnLayerState(*cfg)
    for t in range(rows):
        got = act_np(_gpu_rows(nv, ctx, gdn, fx, tail, state, t, 1))[0]
        want = O.gdn_step(ref, fx["qkv"][t], fx["a"][t], fx["b"][t], fx["z"][t], fx["conv_w"], fx["a_log"],
                          fx["dt_bias"], fx["norm_w"], ctx.act)
        torch.cuda.synchronize()
        assert _close(got, want, ctx.act, "decode chain"), "token %d" % t
    assert np.array_equal(act_np(tail[0]), ref.tail)               # raw rows, copied
    assert np.abs(state[0].cpu().numpy() - ref.state).max() <= 5e-2


def test_gdn_prefill_chunk_equals_sequential_decode(nv, ctx):
    # prefillChunkMatchesSequentialDecode (GDNKernelTests.swift:189-290): seven rows in one call against seven
    # calls; and a chunk shorter than the conv history (the ordered tail shift, gdn.metal:337-366)
    # (from 8 rows on the call runs the conv and the output norm spread over the device and only the
    # recurrence in sequence: 19, 33 and 12 rows, and 300 rows across two sets of precomputed gates)
    for cfg, rows in (((2, 4, 32, 32, 4), 7), ((16, 32, 128, 128, 4), 5), ((2, 4, 32, 32, 4), 2), ((2, 4, 32, 32, 4), 19),
                      ((16, 32, 128, 128, 4), 33), ((2, 2, 64, 64, 2), 12), ((1, 2, 64, 128, 3), 300),
                      # from 64 rows on a 128 x 128 head takes sixteen rows at a time on the matrix cores:
                      # whole chunks, a ragged last chunk, a single chunk plus one row
                      ((2, 4, 128, 128, 4), 64), ((16, 32, 128, 128, 4), 100), ((1, 2, 128, 128, 3), 177), ((2, 2, 128, 128, 2), 65)):
        say("gdn prefill chunk", ctx.act, cfg, rows)
        fx = _fixture(cfg, rows + 3, 0xBEEF, ctx.act)
        gdn = nv.GDN(ctx, *cfg)
        tail_a, state_a = gdn.new_state()
        tail_b, state_b = gdn.new_state()
        seq = []
        for t in range(3):                                        # a common prefix, so that the tail is not zero
            _gpu_rows(nv, ctx, gdn, fx, tail_a, state_a, t, 1)
            _gpu_rows(nv, ctx, gdn, fx, tail_b, state_b, t, 1)
        for t in range(3, 3 + rows):
            seq.append(act_np(_gpu_rows(nv, ctx, gdn, fx, tail_a, state_a, t, 1))[0])
        chunk = act_np(_gpu_rows(nv, ctx, gdn, fx, tail_b, state_b, 3, rows))
        torch.cuda.synchronize()
        assert _close(chunk, np.array(seq), ctx.act, "chunk vs sequential %d" % rows)
        assert torch.equal(tail_a, tail_b)
        assert (state_a - state_b).abs().max().item() <= 5e-2


@pytest.mark.parametrize("bf16_state", [False, True])
def test_gdn_batch_of_sequences_and_bf16_state(nv, ctx, bf16_state):
    # three sequences with their own tails and states in one call per token; the BF16 state is the
    # measured variant (half the state bytes per token) and tracks the fp32 oracle more loosely
    say("gdn batch", ctx.act, bf16_state)
    cfg, batch, steps = (16, 32, 128, 128, 4), 3, 4
    kh, vh, dk, dv, taps = cfg
    fxs = [_fixture(cfg, steps, 100 + b, ctx.act) for b in range(batch)]
    gdn = nv.GDN(ctx, *cfg)
    tail, state = gdn.new_state(batch, bf16=bf16_state)
    refs = [O.GdnLayerState(*cfg) for _ in range(batch)]
    w = fxs[0]
    for t in range(steps):
        stack = lambda key: act_tensor(np.stack([fx[key][t] for fx in fxs]), ctx)
        conv = gdn.encode_conv_norm(stack("qkv"), tail, _bits(w["conv_w"]))
        out = act_np(gdn.encode_delta_gated_norm(conv, stack("a"), stack("b"), _bits(w["a_log"]), _bits(w["dt_bias"]),
                                                 state, stack("z"), _bits(w["norm_w"])))
        torch.cuda.synchronize()
        for b in range(batch):
            want = O.gdn_step(refs[b], fxs[b]["qkv"][t], fxs[b]["a"][t], fxs[b]["b"][t], fxs[b]["z"][t], w["conv_w"],
                              w["a_log"], w["dt_bias"], w["norm_w"], ctx.act)
            if bf16_state:                              # the kernels store the state as BF16 after every token
                refs[b].state[...] = O.round_bf16(refs[b].state)
            assert _close(out[b], want, ctx.act, "batch, bf16 state" if bf16_state else "batch, fp32 state"), (t, b)
    got_state = state.float().cpu().numpy()
    for b in range(batch):
        assert np.abs(got_state[b] - refs[b].state).max() <= 5e-2


@pytest.mark.parametrize("bf16_state", [False, True])
def test_gdn_long_call_on_the_matrix_cores_batch_and_state_types(nv, ctx, bf16_state):
    # two sequences of 83 rows each in one call (five chunks of sixteen and a ragged sixth, the
    # chunked form of the recurrence) against 83 calls of one row per sequence: outputs, tails, states
    say("gdn chunked batch", ctx.act, bf16_state)
    cfg, batch, rows = (2, 4, 128, 128, 4), 2, 83
    fxs = [_fixture(cfg, rows, 700 + b, ctx.act) for b in range(batch)]
    w = fxs[0]
    gdn = nv.GDN(ctx, *cfg)
    tail_a, state_a = gdn.new_state(batch, bf16=bf16_state)
    tail_b, state_b = gdn.new_state(batch, bf16=bf16_state)
    args = (_bits(w["a_log"]), _bits(w["dt_bias"]))
    seq = []
    for t in range(rows):
        stack = lambda key: act_tensor(np.stack([fx[key][t] for fx in fxs]), ctx)
        conv = gdn.encode_conv_norm(stack("qkv"), tail_a, _bits(w["conv_w"]))
        seq.append(act_np(gdn.encode_delta_gated_norm(conv, stack("a"), stack("b"), *args, state_a, stack("z"), _bits(w["norm_w"]))))
    cat = lambda key: act_tensor(np.concatenate([fx[key] for fx in fxs]), ctx)
    conv = gdn.encode_conv_norm(cat("qkv"), tail_b, _bits(w["conv_w"]), rows=rows)
    chunk = act_np(gdn.encode_delta_gated_norm(conv, cat("a"), cat("b"), *args, state_b, cat("z"), _bits(w["norm_w"]), rows=rows))
    torch.cuda.synchronize()
    want = np.stack(seq, axis=1).reshape(batch * rows, -1)            # [batch, rows, :] like the call's rows
    # (with the BF16 state the row-by-row calls round the state after every row, the long call once per call)
    assert _close(chunk, want, ctx.act, "chunked, bf16 state" if bf16_state else "chunked, fp32 state")
    assert torch.equal(tail_a, tail_b)
    assert (state_a.float() - state_b.float()).abs().max().item() <= 5e-2


@pytest.mark.parametrize("rows", [64, 113])
def test_gdn_long_call_matches_the_oracle_row_by_row(nv, ctx, rows):
    # the chunked forms of the recurrence (fp32 matrix products with fp16 activations; split-BF16 operands and
    # precomputed chunk operands with BF16 activations) against the oracle's row-by-row fp32 rule: outputs of
    # every row, the conv tail and the recurrent state after the last one; 113 rows end in a ragged chunk
    say("gdn long call vs oracle", ctx.act, rows)
    cfg = (2, 4, 128, 128, 4)
    fx = _fixture(cfg, rows, 0xC0 + rows, ctx.act)
    gdn = nv.GDN(ctx, *cfg)
    tail, state = gdn.new_state()
    got = act_np(_gpu_rows(nv, ctx, gdn, fx, tail, state, 0, rows))
    torch.cuda.synchronize()
    ref = O.GdnLayerState(*cfg)
    want = np.stack([O.gdn_step(ref, fx["qkv"][t], fx["a"][t], fx["b"][t], fx["z"][t], fx["conv_w"], fx["a_log"],
                                fx["dt_bias"], fx["norm_w"], ctx.act) for t in range(rows)])
    assert _close(got, want, ctx.act, "long call vs oracle, %d rows" % rows)
    assert np.array_equal(act_np(tail[0]), ref.tail)
    d_state = np.abs(state[0].cpu().numpy() - ref.state).max()
    print("[measure] gdn long call state: max|d| %.3e of max|ref| %.3e" % (d_state, np.abs(ref.state).max()), flush=True)
    assert d_state <= 1e-4 * float(np.abs(ref.state).max())      # the split operands keep sixteen bits: measured 7e-6


def test_gdn_long_call_captured_in_a_graph_equals_the_eager_call(nv):
    # 100 rows of a 128 x 128 head take the chunked form, which carves 10,496 bytes per (sequence, head, chunk) out of
    # the context's workspace: a fresh context reserves them, captures the call, and every replay gives the bits of
    # the eager call (outputs, tail, state) -- a capture may not fall back to the row-by-row kernels
    say("gdn chunked call under a graph")
    cfg, rows = (2, 4, 128, 128, 4), 100
    eager_ctx = nv.Context(0, 0)
    fx = _fixture(cfg, rows, 0x6A, 0)
    gdn_e = nv.GDN(eager_ctx, *cfg)
    tail_e, state_e = gdn_e.new_state()
    want = _gpu_rows(nv, eager_ctx, gdn_e, fx, tail_e, state_e, 0, rows).clone()
    torch.cuda.synchronize()
    ctx = nv.Context(0, 0)
    ctx.reserve(1 << 20)                                # 4 value heads x 7 chunks x 10,496 bytes + 2 key heads x 7 x 4,096, and room to spare
    gdn = nv.GDN(ctx, *cfg)
    tail, state = gdn.new_state()
    ins = [act_tensor(fx[k][:rows], ctx) for k in ("qkv", "a", "b", "z")]
    w = [_bits(fx[k]) for k in ("conv_w", "a_log", "dt_bias", "norm_w")]
    conv = torch.empty_like(ins[0])
    out = torch.empty((rows, gdn.value_dim), dtype=ctx.dtype, device="cuda")
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            gdn.encode_conv_norm(ins[0], tail, w[0], conv_out=conv, rows=rows)
            gdn.encode_delta_gated_norm(conv, ins[1], ins[2], w[1], w[2], state, ins[3], w[3], out=out, rows=rows)
    torch.cuda.synchronize()
    for trial in range(3):
        tail.zero_(); state.zero_(); out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), trial
        assert torch.equal(tail, tail_e) and torch.equal(state, state_e), trial
    ctx.close()
    eager_ctx.close()


@pytest.mark.parametrize("rows", [8, 37, 133])
def test_gdn_conv_rows_in_16_byte_pieces_same_bits(nv, ctx, rows):
    # a chunk of rows with four taps and rows at 16-byte boundaries takes the conv + norm eight channels per
    # lane; input rows at a stride that is not a multiple of 16 bytes take the two-channels-per-lane kernel:
    # the same rows through both must give the same bits, the tail too (run boundaries at 8 and 128 rows)
    say("gdn conv rows pieces", ctx.act, rows)
    cfg, batch = (2, 4, 128, 128, 4), 2
    fxs = [_fixture(cfg, rows, 940 + b, ctx.act) for b in range(batch)]
    w = fxs[0]
    gdn = nv.GDN(ctx, *cfg)
    qkv = act_tensor(np.concatenate([fx["qkv"] for fx in fxs]), ctx)
    outs, tails = [], []
    for pad in (0, 4):
        tail, _ = gdn.new_state(batch)
        tail.copy_(torch.randn(tail.shape, generator=torch.Generator().manual_seed(7)).to(tail.dtype))
        x = qkv
        if pad:
            wide = torch.zeros((qkv.shape[0], qkv.shape[1] + pad), dtype=qkv.dtype, device=qkv.device)
            wide[:, :qkv.shape[1]] = qkv
            x = wide[:, :qkv.shape[1]]
            assert x.stride(0) % 8 != 0
        outs.append(gdn.encode_conv_norm(x, tail, _bits(w["conv_w"]), rows=rows))
        tails.append(tail)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(tails[0], tails[1])


@pytest.mark.parametrize("rows", [8, 37, 80])
def test_gdn_gated_norm_in_16_byte_pieces_same_bits(nv, ctx, rows):
    # heads of 128 values take the gated output norm in 16-byte pieces, sixteen lanes per (row, head);
    # z rows at a stride that is not a multiple of 16 bytes take the one-value-per-thread kernel:
    # the same rows through both must give the same bits (rows below and above the chunked form)
    say("gdn gated norm pieces", ctx.act, rows)
    cfg, batch = (2, 4, 128, 128, 4), 2
    fxs = [_fixture(cfg, rows, 900 + b, ctx.act) for b in range(batch)]
    w = fxs[0]
    gdn = nv.GDN(ctx, *cfg)
    cat = lambda key: act_tensor(np.concatenate([fx[key] for fx in fxs]), ctx)
    outs = []
    for pad in (0, 4):
        tail, state = gdn.new_state(batch)
        conv = gdn.encode_conv_norm(cat("qkv"), tail, _bits(w["conv_w"]), rows=rows)
        z = cat("z")
        if pad:
            wide = torch.zeros((z.shape[0], z.shape[1] + pad), dtype=z.dtype, device=z.device)
            wide[:, :z.shape[1]] = z
            z = wide[:, :z.shape[1]]
            assert z.stride(0) % 8 != 0
        outs.append(gdn.encode_delta_gated_norm(conv, cat("a"), cat("b"), _bits(w["a_log"]), _bits(w["dt_bias"]), state, z,
                                                _bits(w["norm_w"]), rows=rows))
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])


def test_gdn_full_size_prompt_is_the_same_in_one_call_or_in_pieces(nv, ctx):
    # the production layer (16 key / 32 value heads of 128 x 128, four taps) over 4096 rows, the size of a
    # configs[4] prompt chunk: one call against calls of 1000 rows (ragged pieces, a last one of 96) and
    # against calls of 48 rows (below the chunked form: the row-by-row recurrence) -- outputs, conv tails
    # and states of the three must agree, whatever route the rows take through the kernels
    say("gdn full size", ctx.act)
    cfg, rows = (16, 32, 128, 128, 4), 4096
    fx = _fixture(cfg, rows, 0x4096, ctx.act)
    gdn = nv.GDN(ctx, *cfg)
    outs, tails, states = [], [], []
    for piece in (rows, 1000, 48):
        tail, state = gdn.new_state()
        got = [act_np(_gpu_rows(nv, ctx, gdn, fx, tail, state, t0, min(piece, rows - t0))) for t0 in range(0, rows, piece)]
        torch.cuda.synchronize()
        outs.append(np.concatenate(got)); tails.append(tail); states.append(state)
    assert np.isfinite(outs[0]).all()
    for k in (1, 2):
        assert _close(outs[k], outs[0], ctx.act, "full size, pieces %d" % k), k
        assert torch.equal(tails[k], tails[0])
        assert (states[k] - states[0]).abs().max().item() <= 5e-2


@pytest.mark.parametrize("bf16_state", [False, True])
@pytest.mark.parametrize("cfg", [(2, 4, 32, 32, 4), (16, 32, 128, 128, 4), (4, 4, 32, 32, 2), (2, 2, 64, 64, 2), (2, 8, 32, 32, 4)],
                         ids=["toy", "production", "ratio1-taps2", "two-kernel-shape", "two-kernel-ratio"])
def test_gdn_decode_step_in_one_launch_equals_the_two_calls(nv, ctx, cfg, bf16_state):
    # conv + q / k norm + tail update + delta rule + gated norm of one token per sequence in one launch:
    # outputs, recurrent state and conv tail are the bits of the two calls, token after token, for a
    # batch of three sequences; the fused shapes and the shapes that go through the scratch rows
    say("gdn decode step, one launch", ctx.act, cfg, bf16_state)
    batch, steps = 3, 5
    fxs = [_fixture(cfg, steps, 300 + b, ctx.act) for b in range(batch)]
    gdn = nv.GDN(ctx, *cfg)
    tail_a, state_a = gdn.new_state(batch, bf16=bf16_state)
    tail_b, state_b = gdn.new_state(batch, bf16=bf16_state)
    w = fxs[0]
    ref = O.GdnLayerState(*cfg)
    scratch = torch.empty((batch, gdn.qkv_dim), dtype=ctx.dtype, device="cuda")
    for t in range(steps):
        stack = lambda key: act_tensor(np.stack([fx[key][t] for fx in fxs]), ctx)
        qkv, a, b, z = stack("qkv"), stack("a"), stack("b"), stack("z")
        weights = (_bits(w["a_log"]), _bits(w["dt_bias"]))
        conv = gdn.encode_conv_norm(qkv, tail_a, _bits(w["conv_w"]))
        two = gdn.encode_delta_gated_norm(conv, a, b, weights[0], weights[1], state_a, z, _bits(w["norm_w"]))
        one = gdn.encode_decode_step(qkv, tail_b, _bits(w["conv_w"]), a, b, weights[0], weights[1], state_b, z,
                                     _bits(w["norm_w"]), conv_scratch=scratch)
        torch.cuda.synchronize()
        assert torch.equal(one.view(torch.int16), two.view(torch.int16)), "token %d" % t
        assert torch.equal(tail_a.view(torch.int16), tail_b.view(torch.int16))
        assert torch.equal(state_a.view(torch.int32 if not bf16_state else torch.int16),
                           state_b.view(torch.int32 if not bf16_state else torch.int16))
        if not bf16_state:
            want = O.gdn_step(ref, fxs[0]["qkv"][t], fxs[0]["a"][t], fxs[0]["b"][t], fxs[0]["z"][t], w["conv_w"],
                              w["a_log"], w["dt_bias"], w["norm_w"], ctx.act)
            assert _close(act_np(one)[0], want, ctx.act, "one launch")
    # a shape without a fused kernel and no scratch rows
    if cfg == (2, 2, 64, 64, 2):
        with pytest.raises(nv.NvmaiError):
            gdn.encode_decode_step(qkv, tail_b, _bits(w["conv_w"]), a, b, weights[0], weights[1], state_b, z, _bits(w["norm_w"]))


def test_gdn_rejects_bad_shapes(nv, ctx):
    say("gdn errors")
    with pytest.raises(nv.NvmaiError) as e:            # numVHeads must be a multiple of numKHeads (GDN.swift:44-45)
        g = nv.GDN(ctx, 3, 4, 32, 32, 4)
        tail, state = g.new_state()
        g.encode_conv_norm(torch.zeros((1, g.qkv_dim), dtype=ctx.dtype, device="cuda"), tail,
                           torch.zeros(g.qkv_dim * 4, dtype=torch.int16, device="cuda"))
    assert e.value.name == "invalid_arg"
    with pytest.raises(nv.NvmaiError) as e:            # keyHeadDim must be a positive multiple of 32 (GDN.swift:38-39)
        g = nv.GDN(ctx, 2, 4, 48, 32, 4)
        tail, state = g.new_state()
        g.encode_conv_norm(torch.zeros((1, g.qkv_dim), dtype=ctx.dtype, device="cuda"), tail,
                           torch.zeros(g.qkv_dim * 4, dtype=torch.int16, device="cuda"))
    assert e.value.name == "invalid_arg"


def test_residual_add_rmsnorm_equals_the_two_calls(nv, ctx):
    say("residual add + rmsnorm", ctx.act)
    rng = np.random.default_rng(5)
    for rows, d in ((1, 2048), (5, 2048), (300, 2048), (3, 192), (16, 4096)):
        h = round_act(gauss(rng, (rows, d)), ctx.act)
        delta = round_act(gauss(rng, (rows, d), 0.3), ctx.act)
        w = _bits(O.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32)))
        h1, h2 = act_tensor(h, ctx), act_tensor(h, ctx)
        out = nv.residual_add_rmsnorm(ctx, h1, act_tensor(delta, ctx), w)
        nv.Elementwise(ctx).encode_residual_add(h2, act_tensor(delta, ctx))
        want = nv.RMSNorm(ctx).encode_bf16w(h2, w)
        torch.cuda.synchronize()
        assert torch.equal(h1, h2) and torch.equal(out, want)
        # and against the oracle: the sum rounded to the activation type, then the norm (bit-exact)
        hs = round_act(h + delta, ctx.act)
        assert np.array_equal(act_np(out), round_act(O.rmsnorm(hs, w.cpu().numpy().view(np.uint16), 1e-6), ctx.act))


@pytest.mark.parametrize("bits", [4, 8])
def test_fused_projections_equal_separate_gemvs(nv, ctx, bits):
    # GDN.encodeInputProjections (qkv, z, a, b) and FusedQKVGEMV: bit-identical to the separate GEMVs,
    # whether the parts lie back to back (one launch) or not
    say("fused projections", ctx.act, bits)
    rng = np.random.default_rng(bits)
    n, rows_list = 2048, [1024, 512, 32, 32]
    total = sum(rows_list)
    wq = O.quantize_affine(O.round_bf16(gauss(rng, (total, n), 0.02)), bits)
    W, S, B = dev(wq[0]), dev(wq[1].view(np.int16)), dev(wq[2].view(np.int16))
    x = act_tensor(round_act(gauss(rng, (1, n)), ctx.act), ctx)
    want = nv.affine_gemv(ctx, W, S, B, bits, x, total, n)
    y = torch.zeros((1, total), dtype=ctx.dtype, device="cuda")
    parts, at = [], 0
    for r in rows_list:
        parts.append((W[at:at + r], S[at:at + r], B[at:at + r], r, y[0, at:at + r]))
        at += r
    nv.affine_gemv_fused(ctx, parts, bits, x, n)
    torch.cuda.synchronize()
    assert torch.equal(y, want)
    # scattered outputs: one launch per part, same bits
    outs = [torch.zeros(r + 8, dtype=ctx.dtype, device="cuda") for r in rows_list]
    parts = [(p[0], p[1], p[2], p[3], o[:p[3]]) for p, o in zip(parts, outs)]
    nv.affine_gemv_fused(ctx, parts, bits, x, n)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([o[:r] for o, r in zip(outs, rows_list)]), want[0])


def test_dense_bf16_gemv(nv):
    # bits == 16: dense BF16 rows (the BF16 LM head), 1..16 inputs per pass and more than 16; against
    # a float64 product of the same BF16 values (fp32 accumulate: 2e-3 on the fp32 output, 1e-2 on BF16)
    say("dense bf16 gemv")
    ctx = nv.Context(0, 0)
    rng = np.random.default_rng(9)
    # (70001 rows at 16 inputs: more 64-row passes than resident blocks, so blocks walk several passes)
    for m, n, tokens in ((1000, 2048, 1), (70, 256, 3), (4096, 2048, 16), (515, 1024, 21), (64, 64, 2),
                         (70001, 2048, 16), (40000, 2048, 1)):
        w = O.round_bf16(gauss(rng, (m, n), 0.02))
        x = O.round_bf16(gauss(rng, (tokens, n)))
        wd = dev(O.bf16_bits(w).view(np.int16))
        y = nv.affine_gemv(ctx, wd, None, None, 16, act_tensor(x, ctx), m, n)
        yf = nv.affine_gemv(ctx, wd, None, None, 16, act_tensor(x, ctx), m, n, out_f32=True)
        torch.cuda.synchronize()
        want = x.astype(np.float64) @ w.astype(np.float64).T
        assert O.rel_error(yf.cpu().numpy(), want.astype(np.float32)) < 2e-3
        assert O.rel_error(act_np(y), want.astype(np.float32)) < 1e-2
    c16 = nv.Context(0, 1)
    with pytest.raises(nv.NvmaiError) as e:            # dense BF16 rows need BF16 activations
        nv.affine_gemv(c16, wd, None, None, 16, torch.zeros((1, 64), dtype=torch.float16, device="cuda"), 64, 64)
    assert e.value.name == "unsupported"
    torch.cuda.synchronize()
    ctx.close()
    c16.close()


@pytest.mark.parametrize("tokens", [1, 16])
def test_dense_bf16_gemv_at_the_lm_head_size(nv, tokens):
    # the BF16 LM head of configs[4]: 248,320 x 2048, one and sixteen input rows (the launch's grid policy
    # follows the row count and the resident blocks), every logit against a float64 product
    say("dense bf16 gemv, LM head size", tokens)
    ctx = nv.Context(0, 0)
    m, n = 248320, 2048
    gen = torch.Generator(device="cuda").manual_seed(2048 + tokens)
    wd = torch.empty((m, n), dtype=torch.float32, device="cuda").normal_(0.0, 0.02, generator=gen).to(torch.bfloat16)
    x = torch.empty((tokens, n), dtype=torch.float32, device="cuda").normal_(0.0, 1.0, generator=gen).to(torch.bfloat16)
    y = nv.affine_gemv(ctx, wd.view(torch.int16), None, None, 16, x, m, n)
    yf = nv.affine_gemv(ctx, wd.view(torch.int16), None, None, 16, x, m, n, out_f32=True)
    torch.cuda.synchronize()
    x64 = x.float().cpu().numpy().astype(np.float64)
    want = np.empty((tokens, m), np.float64)
    for r0 in range(0, m, 32768):                      # the float64 copy of the head, a slab at a time
        want[:, r0:r0 + 32768] = x64 @ wd[r0:r0 + 32768].float().cpu().numpy().astype(np.float64).T
    rel32 = O.rel_error(yf.cpu().numpy(), want.astype(np.float32))
    rel16 = O.rel_error(act_np(y), want.astype(np.float32))
    print("[measure] dense bf16 gemv 248320 x 2048, %d rows: fp32 out rel %.3e, bf16 out rel %.3e" % (tokens, rel32, rel16), flush=True)
    assert rel32 < 2e-3 and rel16 < 1e-2
    # and no row was skipped or written twice by the grid policy: the argmax agrees wherever the margin is clear
    top2 = np.sort(want, axis=1)[:, -2:]
    clear = (top2[:, 1] - top2[:, 0]) > 1e-2 * np.abs(top2[:, 1])
    assert np.array_equal(yf.cpu().numpy().argmax(axis=1)[clear], want.argmax(axis=1)[clear])
    torch.cuda.synchronize()
    ctx.close()
