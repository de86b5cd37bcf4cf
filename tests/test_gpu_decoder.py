"""GPU parity of the whole decode step on a toy hybrid model (three gated-DeltaNet layers and one
full-attention layer over a quantized KV cache, MoE block in each, BF16 LM head, tiled sampler), the
counterpart of the reference's QwenToySynthetic end-to-end check: every step of two sequences is
recomputed by the CPU oracle, operator by operator with the same 16-bit hand-over points.

Bar: final-normed rows and logits within 1e-2 (max|diff| / max|ref|) with the fp32 recurrent state
(measured: the same bits for the normed rows, 6e-8 on the logits) and 2e-2 with the BF16 state (measured
1.5e-2: the oracle rounds its state to BF16 after every token as the kernels do, but a BF16 state amplifies
every last-bit difference of the 16-bit hand-overs through the four layers), routing-independent token check: the GPU's probabilities through the oracle's sampler give
the GPU's tokens, and the recurrent state within the reference's 5e-2."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import act_np, say

pytestmark = pytest.mark.gpu


def _np16(t):
    return t.detach().cpu().numpy().view(np.uint16)


class OracleModel:
    """The decode step of nvmai_amd.decoder.HybridDecoder recomputed with oracle functions."""

    def __init__(self, cfg, w, batch):
        self.cfg, self.w, self.batch = cfg, w, batch
        kh, vh, dk, dv, taps = cfg.gdn
        self.gdn = {L: [O.GdnLayerState(kh, vh, dk, dv, taps) for _ in range(batch)]
                    for L in range(cfg.layers) if cfg.is_linear(L)}
        self.kv = {L: [([], []) for _ in range(batch)] for L in range(cfg.layers) if not cfg.is_linear(L)}
        self.r = O.round_bf16
        q3 = lambda t: (t[0].cpu().numpy(), _np16(t[1]), _np16(t[2]))
        self.embed = q3(w.embed)
        self.lm_head = O.bf16_to_float(_np16(w.lm_head[0])).astype(np.float64)
        self.layers = []
        for L, lw in enumerate(w.layers):
            d = dict(in_norm=_np16(lw["in_norm"]), post_norm=_np16(lw["post_norm"]), pool=lw["pool"].cpu().numpy(),
                     router=_np16(lw["router"]), gate=q3(lw["gate"]))
            if lw.get("shared") is not None:
                d["shared_blob"] = lw["shared"]["blob"].cpu().numpy()
            if cfg.is_linear(L):
                d.update(in_proj=q3(lw["in_proj"]), out_proj=q3(lw["out_proj"]), conv_w=_np16(lw["conv_w"]),
                         a_log=_np16(lw["a_log"]), dt_bias=_np16(lw["dt_bias"]), gdn_norm=_np16(lw["gdn_norm"]))
            else:
                d.update(qkv=q3(lw["qkv"]), o_proj=q3(lw["o_proj"]), q_norm=_np16(lw["q_norm"]), k_norm=_np16(lw["k_norm"]))
            self.layers.append(d)
        self.final_norm = _np16(w.final_norm)

    def gemv(self, m, x, bits):
        return self.r(O.affine_gemv(m[0], m[1], m[2], x, bits))

    def step(self, tokens, position):
        cfg, r = self.cfg, self.r
        D = cfg.hidden
        normed_rows, logits_rows = [], []
        for b, tok in enumerate(tokens):
            hidden = r(O.embed_lookup(*self.embed, cfg.embed_bits, int(tok)))
            normed = r(O.rmsnorm(hidden[None], self.layers[0]["in_norm"], cfg.rms_eps)[0])
            for L, lw in enumerate(self.layers):
                if cfg.is_linear(L):
                    kh, vh, dk, dv, taps = cfg.gdn
                    proj = self.gemv(lw["in_proj"], normed, cfg.attn_bits)
                    C, V = cfg.gdn_qkv_dim, cfg.gdn_value_dim
                    out = O.gdn_step(self.gdn[L][b], proj[:C], proj[C + V:C + V + vh], proj[C + V + vh:], proj[C:C + V],
                                     lw["conv_w"], lw["a_log"], lw["dt_bias"], lw["gdn_norm"], 0)
                    if cfg.gdn_state_bf16:                # the kernels store the state as BF16 after every token
                        self.gdn[L][b].state[...] = O.round_bf16(self.gdn[L][b].state)
                    branch = self.gemv(lw["out_proj"], r(out), cfg.attn_bits)
                else:
                    proj = self.gemv(lw["qkv"], normed, cfg.attn_bits)
                    hd, nh, nkv = cfg.head_dim, cfg.num_heads, cfg.num_kv_heads
                    q, gate = O.split_q_gate(proj[:2 * cfg.q_dim], nh, hd)
                    k = proj[2 * cfg.q_dim:2 * cfg.q_dim + cfg.kv_dim].reshape(nkv, hd)
                    v = proj[2 * cfg.q_dim + cfg.kv_dim:]
                    q = r(O.rmsnorm(q, lw["q_norm"], cfg.rms_eps))
                    k = r(O.rmsnorm(k, lw["k_norm"], cfg.rms_eps))
                    pos = np.array([position], np.uint32)
                    q = r(O.rope_neox_subdim(q[None], cfg.rotary_dim, pos, cfg.rope_theta)[0])
                    k = r(O.rope_neox_subdim(k[None], cfg.rotary_dim, pos, cfg.rope_theta)[0])
                    kc, vc = self.kv[L][b]
                    kc.append(O.kv_quantize(k.reshape(1, -1), cfg.kv_bits)[0])
                    vc.append(O.kv_quantize(v.reshape(1, -1), cfg.kv_bits)[0])
                    att = r(O.attention_decode(q, np.stack(kc), np.stack(vc), cfg.kv_bits, nh, nkv, hd, position + 1,
                                               1.0 / np.sqrt(hd)))
                    att = r(O.elementwise(O.EW_SIGMOID_MUL, att, gate))
                    branch = self.gemv(lw["o_proj"], att.reshape(-1), cfg.attn_bits)
                hidden = r(hidden + branch)
                routed_x = r(O.rmsnorm(hidden[None], lw["post_norm"], cfg.rms_eps)[0])
                E = cfg.num_experts
                router = (16, lw["router"].reshape(E, D), None, None)
                if "shared_blob" in lw:
                    # the routed experts alone at their width; the gated shared expert at its own: a layer whose
                    # experts all ARE the shared blob, with and without the shared slot -- the difference is the slot
                    F, sb = cfg.moe_intermediate, cfg.shared_bits
                    _, _, y_routed = O.moe_layer_forward(routed_x[None], D, F, cfg.top_k, cfg.expert_bits, router, lw["pool"][:E])
                    copies = np.stack([lw["shared_blob"]] * E)
                    _, _, y_both = O.moe_layer_forward(routed_x[None], D, F, cfg.top_k, sb, router, copies, lw["shared_blob"],
                                                       (8,) + lw["gate"])
                    _, _, y_none = O.moe_layer_forward(routed_x[None], D, F, cfg.top_k, sb, router, copies)
                    y = r(r(y_routed) + r(y_both - y_none))
                else:
                    _, _, y = O.moe_layer_forward(routed_x[None], D, cfg.moe_intermediate, cfg.top_k, cfg.expert_bits,
                                                  router, lw["pool"][:E], lw["pool"][E], (8,) + lw["gate"])
                hidden = r(hidden + r(y[0]))
                nxt = self.layers[L + 1]["in_norm"] if L + 1 < cfg.layers else self.final_norm
                normed = r(O.rmsnorm(hidden[None], nxt, cfg.rms_eps)[0])
            normed_rows.append(normed)
            logits_rows.append(r((self.lm_head @ normed.astype(np.float64)).astype(np.float32)))
        return np.stack(normed_rows), np.stack(logits_rows)


@pytest.mark.parametrize("state_bf16", [False, True], ids=["fp32-state", "bf16-state"])
def test_toy_hybrid_model_steps_match_oracle(state_bf16):
    import nvmai_amd as nv
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    say("toy hybrid decode steps", state_bf16)
    ctx = nv.Context(0, nv.ACT_BF16)
    cfg = HybridConfig(hidden=256, layers=4, full_every=4, num_heads=4, num_kv_heads=2, head_dim=64, rotary_dim=16,
                       rope_theta=1e4, gdn=(2, 4, 32, 32, 4), num_experts=16, top_k=4, moe_intermediate=128, vocab=1024,
                       expert_bits=4, attn_bits=4, kv_bits=8, head_bits=16, gdn_state_bf16=state_bf16)
    w = HybridWeights(ctx, cfg, seed=7, std=0.06)
    batch = 2
    dec = HybridDecoder(ctx, cfg, w, batch=batch, max_context=16)
    torch.cuda.synchronize()
    ref = OracleModel(cfg, w, batch)
    tokens = np.array([5, 900], np.int32)
    tol = 1e-2 if not state_bf16 else 2e-2
    for position in range(4):
        dec.tokens.copy_(torch.from_numpy(tokens).cuda())
        seeds = [nv.sampler_seed_for(42 + b, position) for b in range(batch)]
        nxt = dec.step(position, seeds)
        torch.cuda.synchronize()
        want_normed, want_logits = ref.step(tokens, position)
        err_n = O.rel_error(act_np(dec.normed), want_normed)
        err_l = O.rel_error(act_np(dec.logits), want_logits)
        print("position", position, "normed rel", err_n, "logits rel", err_l, flush=True)
        assert err_n < tol and err_l < tol
        probs = dec.probs.cpu().numpy().view(np.uint16)
        ref_probs = np.stack([O.f16_to_float(O.softmax_f16(want_logits[b], softcap=0.0, tiled=True)) for b in range(batch)])
        assert np.abs(O.f16_to_float(probs) - ref_probs).max() <= 0.05 * ref_probs.max() + 1e-4
        got = nxt.cpu().numpy()
        for b in range(batch):
            assert got[b] == O.sample_topk64(probs[b], 0.6, 0.95, seeds[b], top_k=20)
        tokens = got.astype(np.int32)
    if not state_bf16:
        for L, (tail, state) in dec.gdn_states.items():
            for b in range(batch):
                assert np.abs(state[b].cpu().numpy() - ref.gdn[L][b].state).max() <= 5e-2
    # the KV rows written by the step equal the oracle's codes where the inputs agree to the bit at position 0
    torch.cuda.synchronize()
    ctx.close()


def test_step_replays_from_a_captured_graph():
    # the whole step only enqueues kernels: captured once, replayed with new tokens in the same buffers,
    # every replay equals the eager step bit for bit (logits) when both start from the same state
    import nvmai_amd as nv
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    say("toy hybrid decode step under a graph")
    ctx = nv.Context(0, nv.ACT_BF16)
    cfg = HybridConfig(hidden=256, layers=4, full_every=2, num_heads=4, num_kv_heads=2, head_dim=64, rotary_dim=16,
                       rope_theta=1e4, gdn=(2, 4, 32, 32, 4), num_experts=16, top_k=4, moe_intermediate=128, vocab=1024)
    w = HybridWeights(ctx, cfg, seed=3, std=0.06)
    eager, graphed = HybridDecoder(ctx, cfg, w, 2, 16), HybridDecoder(ctx, cfg, w, 2, 16)
    seeds = [11, 12]
    graphed.tokens.copy_(torch.tensor([1, 2], dtype=torch.int32))
    graphed.step(0, seeds)                                  # warm-up: the workspace is sized here
    torch.cuda.synchronize()
    for buf in [graphed.gdn_states[L][i] for L in graphed.gdn_states for i in (0, 1)]:
        buf.zero_()                                         # back to the initial state
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            graphed.step(0, seeds)
    torch.cuda.synchronize()
    for buf in [graphed.gdn_states[L][i] for L in graphed.gdn_states for i in (0, 1)]:
        buf.zero_()
    for trial, toks in enumerate(([7, 300], [512, 9])):
        for d in (eager, graphed):
            for L in d.gdn_states:
                d.gdn_states[L][0].zero_(); d.gdn_states[L][1].zero_()
            d.tokens.copy_(torch.tensor(toks, dtype=torch.int32))
        want = eager.step(0, seeds).clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(graphed.logits, eager.logits) and torch.equal(graphed.next_tokens, want)
    ctx.close()


@pytest.mark.parametrize("batch", [2, 5], ids=["folded-norms", "five-sequences"])
def test_toy_hybrid_model_with_a_shared_expert_of_another_width(batch):
    # quant.sharedExpert = 8 beside quant.routedExpert = 4, the reference repacker's 4-bit profile
    # (RemoteStreamingRepacker.swift:678-683): the step runs the routed block on its own and the shared-expert operator
    # at its width beside it (RealForwardRunner.swift:3866-3912).  Two sequences take the path that folds a layer's
    # closing add and the next norm into the next projection launch, five the one with explicit launches.  Every expert
    # is selected (top_k = experts), so that no near-tie of the router can send the oracle and the GPU, whose rows
    # differ in the last bits by then, to different experts.
    import nvmai_amd as nv
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    say("toy hybrid decode steps, shared expert at 8 bits", batch)
    ctx = nv.Context(0, nv.ACT_BF16)
    cfg = HybridConfig(hidden=256, layers=4, full_every=4, num_heads=4, num_kv_heads=2, head_dim=64, rotary_dim=16,
                       rope_theta=1e4, gdn=(2, 4, 32, 32, 4), num_experts=4, top_k=4, moe_intermediate=128, vocab=1024,
                       expert_bits=4, attn_bits=4, kv_bits=8, head_bits=16, gdn_state_bf16=False, shared_bits=8)
    w = HybridWeights(ctx, cfg, seed=17, std=0.06)
    assert all(lw["shared"]["bits"] == 8 and lw["pool"].shape[0] == cfg.num_experts for lw in w.layers)
    dec = HybridDecoder(ctx, cfg, w, batch=batch, max_context=16)
    ref = OracleModel(cfg, w, batch)
    tokens = np.array([5, 900, 33, 512, 77][:batch], np.int32)
    for position in range(3):
        dec.tokens.copy_(torch.from_numpy(tokens).cuda())
        seeds = [nv.sampler_seed_for(42 + b, position) for b in range(batch)]
        nxt = dec.step(position, seeds)
        torch.cuda.synchronize()
        want_normed, want_logits = ref.step(tokens, position)
        err_n, err_l = O.rel_error(act_np(dec.normed), want_normed), O.rel_error(act_np(dec.logits), want_logits)
        print("position", position, "normed rel", err_n, "logits rel", err_l, flush=True)
        assert err_n < 1e-2 and err_l < 1e-2
        tokens = nxt.cpu().numpy().astype(np.int32)
    ctx.close()


@pytest.mark.parametrize("prompt,chunk,shared_bits", [(80, 512, None), (80, 48, None), (200, 512, None), (200, 512, 8), (80, 48, 8)],
                         ids=["one-chunk", "two-chunks", "dense-shared", "dense-shared-8bit", "two-chunks-shared-8bit"])
def test_prefill_chunks_leave_the_state_that_decode_steps_leave(prompt, chunk, shared_bits):
    # RealForwardRunner.prefillChunked against its own serial decode loop: the prompt through the prefill
    # kernels (dense matrix-core projections, recurrent kernels over the rows of a chunk, causal attention
    # over the quantized cache, tiled router + permutation + grouped GEMM + reduce, shared expert) and
    # through one decode step per token end in the same final-normed row, the same KV rows and recurrent
    # states, and the next decode step from either gives the same logits -- within the 16-bit hand-over
    # tolerance, the two paths round at different places.  Every expert is selected (top_k = experts), so
    # that no near-tie of the router can send the two paths to different experts.
    import nvmai_amd as nv
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    say("prefill chunks vs decode steps", prompt, chunk, shared_bits)
    ctx = nv.Context(0, nv.ACT_BF16)
    cfg = HybridConfig(hidden=256, layers=4, full_every=2, num_heads=4, num_kv_heads=2, head_dim=64, rotary_dim=16,
                       rope_theta=1e4, gdn=(2, 4, 32, 32, 4), num_experts=4, top_k=4, moe_intermediate=128, vocab=1024,
                       expert_bits=4, attn_bits=4, kv_bits=8, head_bits=16, gdn_state_bf16=False, shared_bits=shared_bits)
    w = HybridWeights(ctx, cfg, seed=11, std=0.06)
    serial, chunked = HybridDecoder(ctx, cfg, w, 1, 256), HybridDecoder(ctx, cfg, w, 1, 256)
    gen = torch.Generator(device="cuda").manual_seed(prompt)
    tokens = torch.randint(0, cfg.vocab, (prompt,), generator=gen, device="cuda", dtype=torch.int32)
    for position in range(prompt):
        serial.tokens.copy_(tokens[position:position + 1])
        want_last = serial.forward_hidden(position)
    got_last = chunked.prefill_chunked(tokens, sequence=0, start_position=0, chunk_tokens=chunk)
    torch.cuda.synchronize()
    err = O.rel_error(act_np(got_last), act_np(want_last))
    print("final-normed row of the last prompt token: rel", err, flush=True)
    assert err < 2e-2
    for L in serial.gdn_states:
        (tail_a, state_a), (tail_b, state_b) = serial.gdn_states[L], chunked.gdn_states[L]
        assert O.rel_error(act_np(tail_b), act_np(tail_a)) < 3e-2
        assert (state_a - state_b).abs().max().item() <= 5e-2 * max(1.0, state_a.abs().max().item())
    for L in serial.kv:
        for ca, cb in zip(serial.kv[L], chunked.kv[L]):
            ka = O.kv_dequant(ca.rows[0, :prompt].cpu().numpy(), cfg.kv_dim, cfg.kv_bits)
            kb = O.kv_dequant(cb.rows[0, :prompt].cpu().numpy(), cfg.kv_dim, cfg.kv_bits)
            assert O.rel_error(kb, ka) < 3e-2
            assert int(cb.rows[0, prompt:].abs().max()) == 0          # nothing written past the prompt
    # the next token from either state
    nxt = torch.tensor([7], dtype=torch.int32, device="cuda")
    outs = []
    for dec in (serial, chunked):
        dec.tokens.copy_(nxt)
        dec.forward_hidden(prompt)
        outs.append(act_np(dec.head()).copy())
    torch.cuda.synchronize()
    err = O.rel_error(outs[1], outs[0])
    print("logits of the next decode step: rel", err, flush=True)
    assert err < 3e-2
    ctx.close()


def test_full_size_configs4_step_properties():
    # BASELINE configs[4] at its full size: 40 layers (30 gated-DeltaNet + 10 full attention), 256 experts top-8 +
    # shared, 4-bit, BF16 recurrent state, 8-bit KV at 32K context, BF16 LM head over 248,320, sixteen sequences.
    # The CPU oracle needs minutes per token at this size, so the step is checked through what does not depend on
    # size: everything finite; the tokens are the oracle's sampler applied to the GPU's own probabilities; the
    # probabilities are the oracle's softmax of the GPU's logits; a graph replay equals the eager step bit for bit.
    import nvmai_amd as nv
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    say("configs[4] full-size step: 40 layers, 32K context, batch 16")
    ctx = nv.Context(0, nv.ACT_BF16)
    cfg = HybridConfig(layers=40, expert_bits=4, attn_bits=4, kv_bits=8, head_bits=16, gdn_state_bf16=True)
    batch, context = 16, 32768
    w = HybridWeights(ctx, cfg, seed=2024)
    dec = HybridDecoder(ctx, cfg, w, batch=batch, max_context=context)
    gen = torch.Generator(device="cuda").manual_seed(5)
    quant = nv.KVCacheQuantizer(ctx)
    for L, (kc, vc) in dec.kv.items():                      # caches full of quantized N(0, 1) rows
        for c in (kc, vc):
            for b in range(batch):
                for start in range(0, context, 8192):
                    n = min(8192, context - start)
                    src = torch.empty((n, cfg.kv_dim), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
                    quant.encode(src, cfg.kv_dim, c.view(b, start), n, cfg.kv_dim)
    tokens = torch.randint(0, cfg.vocab, (batch,), generator=gen, device="cuda", dtype=torch.int32)
    position = context - 1
    seeds = [nv.sampler_seed_for(1234, position + b) for b in range(batch)]

    def reset():
        for L in dec.gdn_states:
            for buf in dec.gdn_states[L]:
                buf.zero_()
        dec.tokens.copy_(tokens)

    reset()
    eager_tokens = dec.step(position, seeds).clone()
    torch.cuda.synchronize()
    logits, probs = dec.logits.clone(), dec.probs.clone()
    assert bool(torch.isfinite(logits.float()).all()) and bool(torch.isfinite(dec.normed.float()).all())
    assert bool(((eager_tokens >= 0) & (eager_tokens < cfg.vocab)).all())
    lg = act_np(logits)
    pr = probs.cpu().numpy().view(np.uint16)
    assert float(np.abs(lg).max()) > 0.0 and float(lg.std()) > 1e-3        # a head that really multiplied
    for b in range(batch):
        want_p = O.f16_to_float(O.softmax_f16(lg[b], softcap=0.0, tiled=True))
        assert np.abs(O.f16_to_float(pr[b]) - want_p).max() <= 2e-3 * want_p.max() + 1e-7, b
        assert int(eager_tokens[b]) == O.sample_topk64(pr[b], 0.6, 0.95, seeds[b], top_k=20), b
    # the same step from a captured graph, twice, with eager work in between
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    reset()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            dec.step(position, seeds)
    torch.cuda.synchronize()
    for trial in range(2):
        reset()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dec.logits, logits), trial
        assert torch.equal(dec.next_tokens, eager_tokens), trial
        dec.logits.zero_()                                   # eager work between the replays
    torch.cuda.synchronize()
    ctx.close()
