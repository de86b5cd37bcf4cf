"""GPU: a model directory in the reference's .gturbo format (written here from quantized random
weights, experts stored in a permuted physical order) is read into HBM by nvmai_amd.gturbo and
driven through the decode layer; the result is compared with the oracle over the arrays the
directory was written from.  No model file of the reference is available offline, so the weights are
synthetic; the format rules themselves are pinned on the CPU in tests/test_gturbo_format.py."""
import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import act_np, act_tensor, gauss, round_act, say, u16, u32

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [4, 8])
def test_model_directory_to_decode_layer(tmp_path, bits):
    import nvmai_amd as nv
    from nvmai_amd import gturbo as G
    say("gturbo directory -> decode layer", bits)
    rng = np.random.default_rng(70 + bits)
    d, f, E, k, layers = 256, 128, 16, 4, 2
    mk = lambda r, c, s=0.05: O.round_bf16(gauss(rng, (r, c), s))
    roles = ["gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases"]
    off = O.expert_offsets(d, f, bits)                     # CPUExpertFFN.Offsets: the order the repack tool writes
    sizes = [f * d * bits // 8, f * (d // 64) * 2, f * (d // 64) * 2] * 2 + [d * f * bits // 8, d * (f // 64) * 2, d * (f // 64) * 2]
    shapes = [(f, d), (f, d // 64), (f, d // 64)] * 2 + [(d, f), (d, f // 64), (d, f // 64)]
    tensors = {r: G.SubTensorEntry(int(off[i]), sizes[i], "BF16" if "_" in r else "U32", shapes[i], None if "_" in r else bits)
               for i, r in enumerate(roles)}
    used = int(off[8]) + sizes[8]
    stride = (used + G.ALIGNMENT_BYTES - 1) // G.ALIGNMENT_BYTES * G.ALIGNMENT_BYTES
    ranks = list(rng.permutation(E))
    lays, resident, truth = [], [], []
    for L in range(layers):
        blobs = np.zeros((E, stride), np.uint8)
        for e in range(E):
            blobs[e, :used] = O.pack_expert(mk(f, d), mk(f, d), mk(d, f), bits)[:used]
        lays.append({"blobs": blobs, "tensors": tensors, "ranks": [int(r) for r in ranks]})
        p = "language_model.model.layers.%d.mlp." % L
        router = O.bf16_bits(mk(E, d, 0.02))
        resident.append((p + "gate.weight", 1, (E, d), router.tobytes(), None, None))
        shared = []
        for proj, (rows, cols) in (("gate_proj", (f, d)), ("up_proj", (f, d)), ("down_proj", (d, f))):
            q = O.quantize_affine(mk(rows, cols), bits)
            shared.append(q)
            resident.append((p + "shared_expert.%s.weight" % proj, 0, (rows, cols), q[0].tobytes(), q[1].tobytes(), q[2].tobytes()))
        gate = O.quantize_affine(mk(1, d), bits)
        resident.append((p + "shared_expert_gate.weight", 0, (1, d), gate[0].tobytes(), gate[1].tobytes(), gate[2].tobytes()))
        truth.append((router, blobs, shared, gate))
    slot = lambda b: {"weightBits": b, "scheme": "affine", "scaleType": "bf16", "biasType": "bf16", "groupSize": 64}
    quant = {n: slot(bits) for n in ("embedding", "attention", "router", "sharedExpert", "routedExpert")}
    arch = {"hiddenSize": d, "ffnIntermediate": 4 * d, "moeIntermediateSize": f, "numHeads": 4, "numKVHeads": 2,
            "numFullKVHeads": 2, "headDim": 64, "fullHeadDim": 64, "vocabSize": 1000, "slidingWindow": 0,
            "finalLogitSoftcap": 0.0, "ropeTheta": 1e4, "fullRopeTheta": 1e7, "partialRotaryFactor": 0.25,
            "numLayers": layers, "numExperts": E, "topKExperts": k, "tieWordEmbeddings": False, "attentionKEqV": False,
            "hiddenActivation": "silu", "fullAttentionLayerMask": [0, 1]}
    G.write_model(str(tmp_path), arch, quant, lays, resident)

    model = G.GTurboModel(str(tmp_path))
    ctx = nv.Context(0, 0)
    x = round_act(gauss(rng, (5, d)), 0)
    for L in range(layers):
        pool = model.expert_pool(L)
        assert pool.shape == (E + 1, stride)
        assert np.array_equal(pool[:E].cpu().numpy(), lays[L]["blobs"])        # logical order in HBM
        desc, keep = model.moe_layer(L, pool)
        y, idx, w = nv.MoE(ctx, bits).decode_layer(desc, act_tensor(x, ctx), want_routes=True)
        torch.cuda.synchronize()
        router, blobs, shared, gate = truth[L]
        shared_blob = np.zeros(stride, np.uint8)
        for i, q in enumerate(shared):
            for arr, at in zip(q, (int(off[3 * i]), int(off[3 * i + 1]), int(off[3 * i + 2]))):
                raw = arr.view(np.uint8).reshape(-1)
                shared_blob[at:at + raw.size] = raw
        io, wo, yo = O.moe_layer_forward(x, d, f, k, bits, (16, router, None, None), blobs, shared_blob, (bits,) + gate)
        assert np.array_equal(u32(idx), io), "routing indices"
        assert np.abs(u16(w).astype(np.int32) - wo.astype(np.int32)).max() <= 1
        assert O.rel_error(act_np(y), yo) < 1e-2
    ctx.close()


def test_shared_expert_at_8_bits_beside_4_bit_routed_experts(tmp_path):
    # the reference's default 4-bit profile (sharedExpert = 8, routedExpert = 4, RemoteStreamingRepacker.swift:678-683):
    # the block runs the routed experts at 4 bits and the shared expert through its own operator at 8 bits
    import nvmai_amd as nv
    from nvmai_amd import gturbo as G
    say("gturbo directory, 8-bit shared expert + 4-bit routed experts")
    rng = np.random.default_rng(91)
    d, f, E, k, bits, sbits = 256, 128, 16, 4, 4, 8
    mk = lambda r, c, s=0.05: O.round_bf16(gauss(rng, (r, c), s))
    roles = ["gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases"]
    off = O.expert_offsets(d, f, bits)
    sizes = [f * d * bits // 8, f * (d // 64) * 2, f * (d // 64) * 2] * 2 + [d * f * bits // 8, d * (f // 64) * 2, d * (f // 64) * 2]
    shapes = [(f, d), (f, d // 64), (f, d // 64)] * 2 + [(d, f), (d, f // 64), (d, f // 64)]
    tensors = {r: G.SubTensorEntry(int(off[i]), sizes[i], "BF16" if "_" in r else "U32", shapes[i], None if "_" in r else bits)
               for i, r in enumerate(roles)}
    used = int(off[8]) + sizes[8]
    stride = (used + G.ALIGNMENT_BYTES - 1) // G.ALIGNMENT_BYTES * G.ALIGNMENT_BYTES
    blobs = np.zeros((E, stride), np.uint8)
    for e in range(E):
        blobs[e, :used] = O.pack_expert(mk(f, d), mk(f, d), mk(d, f), bits)[:used]
    p = "language_model.model.layers.0.mlp."
    router = O.bf16_bits(mk(E, d, 0.02))
    resident = [(p + "gate.weight", 1, (E, d), router.tobytes(), None, None)]
    shared_w = [mk(f, d), mk(f, d), mk(d, f)]
    for proj, w in zip(("gate_proj", "up_proj", "down_proj"), shared_w):
        q = O.quantize_affine(w, sbits)
        resident.append((p + "shared_expert.%s.weight" % proj, 0, w.shape, q[0].tobytes(), q[1].tobytes(), q[2].tobytes()))
    gate = O.quantize_affine(mk(1, d), bits)
    resident.append((p + "shared_expert_gate.weight", 0, (1, d), gate[0].tobytes(), gate[1].tobytes(), gate[2].tobytes()))
    slot = lambda b: {"weightBits": b, "scheme": "affine", "scaleType": "bf16", "biasType": "bf16", "groupSize": 64}
    quant = {n: slot(bits) for n in ("embedding", "attention", "router", "sharedExpert", "routedExpert")}
    quant["sharedExpert"] = slot(sbits)
    arch = {"hiddenSize": d, "ffnIntermediate": 4 * d, "moeIntermediateSize": f, "numHeads": 4, "numKVHeads": 2,
            "numFullKVHeads": 2, "headDim": 64, "fullHeadDim": 64, "vocabSize": 1000, "slidingWindow": 0,
            "finalLogitSoftcap": 0.0, "ropeTheta": 1e4, "fullRopeTheta": 1e7, "partialRotaryFactor": 0.25,
            "numLayers": 1, "numExperts": E, "topKExperts": k, "tieWordEmbeddings": False, "attentionKEqV": False,
            "hiddenActivation": "silu", "fullAttentionLayerMask": [0]}
    G.write_model(str(tmp_path), arch, quant, [{"blobs": blobs, "tensors": tensors, "ranks": None}], resident)
    model = G.GTurboModel(str(tmp_path))
    assert not model.shared_matches_routed()
    block = model.moe_block(0)
    ctx = nv.Context(0, 0)
    x = round_act(gauss(rng, (5, d)), 0)
    y, idx, w = block.decode(ctx, act_tensor(x, ctx), want_routes=True)
    torch.cuda.synchronize()
    # the oracle: routed experts alone (a zero shared expert), plus the 8-bit shared expert with its gate
    io, wo, y_routed = O.moe_layer_forward(x, d, f, k, bits, (16, router, None, None), blobs, None, None)
    shared_blob = O.pack_expert(*shared_w, sbits)
    _, _, y_both = O.moe_layer_forward(x, d, f, k, sbits, (16, router, None, None), np.stack([shared_blob] * E), shared_blob,
                                       (bits,) + gate)
    # y_both - (its routed part) = the gated shared expert at 8 bits
    _, _, y_routed8 = O.moe_layer_forward(x, d, f, k, sbits, (16, router, None, None), np.stack([shared_blob] * E), None, None)
    want = y_routed + (y_both - y_routed8)
    assert np.array_equal(u32(idx), io), "routing indices"
    assert O.rel_error(act_np(y), want) < 1e-2
    # and a model whose widths agree takes the one-call path through the same object
    ctx.close()


@pytest.mark.parametrize("head_bits,shared_bits", [(16, None), (4, None), (16, 8)], ids=["bf16-head", "4bit-head", "shared-expert-8bit"])
def test_whole_hybrid_model_from_a_directory_equals_the_model_from_arrays(tmp_path, head_bits, shared_bits):
    # every resident tensor bound by the reference's names (Model.swift:137-306): a toy hybrid model (gated-DeltaNet
    # and full-attention layers, MoE in each) written as a model directory, read back, and stepped beside the model
    # it was written from -- hidden rows, logits and sampled tokens must be the same bits, token after token.  The third
    # case keeps the shared expert at 8 bits beside 4-bit routed experts (the reference repacker's 4-bit profile).
    import nvmai_amd as nv
    from nvmai_amd import gturbo as G
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    say("gturbo directory -> HybridWeights -> decode steps", head_bits, shared_bits)
    ctx = nv.Context(0, nv.ACT_BF16)
    cfg = HybridConfig(hidden=256, layers=4, full_every=2, num_heads=4, num_kv_heads=2, head_dim=64, rotary_dim=16,
                       rope_theta=1e4, gdn=(2, 4, 32, 32, 4), num_experts=16, top_k=4, moe_intermediate=128, vocab=1024,
                       expert_bits=4, attn_bits=4, kv_bits=8, head_bits=head_bits, embed_bits=4, gdn_state_bf16=True,
                       shared_bits=shared_bits)
    w = HybridWeights(ctx, cfg, seed=21, std=0.06)
    torch.cuda.synchronize()
    G.write_hybrid_model(str(tmp_path), cfg, w)
    model = G.GTurboModel(str(tmp_path))
    for L in range(cfg.layers):                                  # every name the reference looks up is there
        for name in G.hybrid_tensor_names(L, not cfg.is_linear(L)):
            assert name in model.entries, name
    cfg2, w2 = HybridWeights.from_gturbo(ctx, model, kv_bits=8, gdn_state_bf16=True)
    assert cfg2.gdn == cfg.gdn and cfg2.head_bits == head_bits and cfg2.rotary_dim == cfg.rotary_dim
    assert cfg2.shared_bits == cfg.shared_bits and model.shared_matches_routed() == (shared_bits is None)
    assert [cfg2.is_linear(L) for L in range(4)] == [cfg.is_linear(L) for L in range(4)]
    a, b = HybridDecoder(ctx, cfg, w, 2, 16), HybridDecoder(ctx, cfg2, w2, 2, 16)
    tokens = torch.tensor([5, 900], dtype=torch.int32, device="cuda")
    for position in range(3):
        seeds = [nv.sampler_seed_for(7 + s_, position) for s_ in range(2)]
        outs = []
        for dec in (a, b):
            dec.tokens.copy_(tokens)
            outs.append(dec.step(position, seeds).clone())
        torch.cuda.synchronize()
        assert torch.equal(a.normed, b.normed) and torch.equal(a.logits, b.logits), position
        assert torch.equal(outs[0], outs[1])
        tokens = outs[0]
    ctx.close()
