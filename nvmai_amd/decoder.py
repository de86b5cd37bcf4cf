"""Decode step of the hybrid MoE model over the C ABI: the host-side counterpart of
RealForwardRunner.step (RealForwardRunner.swift:1820-2050) for experts resident in HBM.

A layer is: input RMSNorm -> attention branch (gated-DeltaNet linear attention, or full attention
with an output gate over a quantized KV cache; RealForwardRunner.swift:2066-2131, 2178-2283) ->
residual add -> post-attention RMSNorm -> MoE block (router, shared expert, routed experts) ->
residual add; then the final norm, the LM head, softmax and the sampler.  Every call only enqueues
kernels on the current stream, so a whole step can be captured into a HIP graph and replayed.

Weights are laid out for one launch per projection group: the four input projections of a linear
layer (qkv, z, a, b) and the three of a full-attention layer (packed q / gate, k, v) are rows of one
matrix each.
"""
import ctypes as C

import torch

from . import ops
from ._lib import check, lib


class HybridConfig:
    """The architecture fields the step reads (ArchConfig, ModelTypes.swift:48-204)."""

    def __init__(self, hidden=2048, layers=40, full_every=4, num_heads=16, num_kv_heads=2, head_dim=256,
                 rotary_dim=64, rope_theta=1e7, gdn=(16, 32, 128, 128, 4), num_experts=256, top_k=8,
                 moe_intermediate=512, vocab=248320, expert_bits=4, attn_bits=4, kv_bits=8, head_bits=16,
                 embed_bits=4, rms_eps=1e-6, logit_softcap=0.0, gdn_state_bf16=True, full_mask=None, shared_bits=None):
        self.hidden, self.layers, self.full_every = hidden, layers, full_every
        self.full_mask = None if full_mask is None else [bool(v) for v in full_mask]   # per layer: full attention?
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.rotary_dim, self.rope_theta, self.gdn = rotary_dim, rope_theta, gdn
        self.num_experts, self.top_k, self.moe_intermediate, self.vocab = num_experts, top_k, moe_intermediate, vocab
        self.expert_bits, self.attn_bits, self.kv_bits = expert_bits, attn_bits, kv_bits
        # quant.sharedExpert beside quant.routedExpert (Model.swift:59-60): the repacker's 4-bit profile keeps the
        # shared expert at 8 bits (RemoteStreamingRepacker.swift:678-683)
        self.shared_bits = expert_bits if shared_bits is None else shared_bits
        self.head_bits, self.embed_bits = head_bits, embed_bits
        self.rms_eps, self.logit_softcap, self.gdn_state_bf16 = rms_eps, logit_softcap, gdn_state_bf16

    def is_linear(self, layer):
        """layerIsLinear (ModelTypes.swift:288-289): by the model's layer mask when one was given, else every
        full_every-th layer is full attention and the others gated DeltaNet."""
        if self.full_mask is not None:
            return not self.full_mask[layer]
        return (layer + 1) % self.full_every != 0

    @property
    def q_dim(self):
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self):
        return self.num_kv_heads * self.head_dim

    @property
    def gdn_qkv_dim(self):
        kh, vh, dk, dv, _ = self.gdn
        return 2 * kh * dk + vh * dv

    @property
    def gdn_value_dim(self):
        return self.gdn[1] * self.gdn[3]

    def bytes_per_token(self, batch=1, context=32768):
        """Algorithmic HBM bytes of one decode step divided by the batch: every weight the step
        touches once (routed experts: the expected number of distinct ones for uniform routing), the
        recurrent states read and written, the KV rows read."""
        D, F, E, k = self.hidden, self.moe_intermediate, self.num_experts, self.top_k
        mat = lambda rows, cols, bits: rows * cols * bits / 8 + (0 if bits == 16 else 2 * rows * (cols // 64) * 2)
        expert = 2 * mat(F, D, self.expert_bits) + mat(D, F, self.expert_bits)
        distinct = E * (1.0 - (1.0 - k / E) ** batch)
        shared = 2 * mat(F, D, self.shared_bits) + mat(D, F, self.shared_bits)
        moe = distinct * expert + shared + E * D * 2 + mat(1, D, 8)
        kh, vh, dk, dv, taps = self.gdn
        lin = mat(self.gdn_qkv_dim + self.gdn_value_dim + 2 * vh, D, self.attn_bits) + mat(D, self.gdn_value_dim, self.attn_bits) \
            + self.gdn_qkv_dim * taps * 2
        lin_state = batch * 2 * vh * dv * dk * (2 if self.gdn_state_bf16 else 4)
        full = mat(2 * self.q_dim + 2 * self.kv_dim, D, self.attn_bits) + mat(D, self.q_dim, self.attn_bits)
        kv_stride = ops.kv_row_layout(self.kv_dim, self.kv_bits)[0]
        kv = batch * context * 2 * kv_stride
        n_lin = sum(self.is_linear(L) for L in range(self.layers))
        n_full = self.layers - n_lin
        total = self.layers * moe + n_lin * (lin + lin_state) + n_full * (full + kv) + mat(self.vocab, D, self.head_bits)
        return total / batch


def _randn(gen, shape, std, device):
    return torch.empty(shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen).to(torch.bfloat16)


class HybridWeights:
    """Random-init weights of the model, quantized on the device by the library's own quantizer
    (the same bits as the reference's quantizer gives for the same values)."""

    def __init__(self, ctx, cfg, seed=1234, std=0.02):
        self.ctx, self.cfg = ctx, cfg
        dev = ctx.device
        gen = torch.Generator(device=dev).manual_seed(seed)
        D = cfg.hidden
        q = lambda rows, cols, bits, s=std: ops.quantize_affine(ctx, _randn(gen, (rows, cols), s, dev), bits)
        normw = lambda n: torch.empty(n, dtype=torch.float32, device=dev).uniform_(0.8, 1.2, generator=gen) \
            .to(torch.bfloat16).view(torch.int16)
        self.embed = q(cfg.vocab, D, cfg.embed_bits, 1.0)
        self.final_norm = normw(D)
        if cfg.head_bits == 16:
            self.lm_head = (_randn(gen, (cfg.vocab, D), std, dev).view(torch.int16), None, None)
        else:
            self.lm_head = q(cfg.vocab, D, cfg.head_bits)
        off, stride = ops.expert_offsets(D, cfg.moe_intermediate, cfg.expert_bits)
        self.layers = []
        kh, vh, dk, dv, taps = cfg.gdn
        for L in range(cfg.layers):
            w = dict(in_norm=normw(D), post_norm=normw(D))
            if cfg.is_linear(L):
                rows = cfg.gdn_qkv_dim + cfg.gdn_value_dim + 2 * vh
                w["in_proj"] = q(rows, D, cfg.attn_bits)
                w["conv_w"] = torch.empty((cfg.gdn_qkv_dim, taps), dtype=torch.float32, device=dev) \
                    .uniform_(-0.4, 0.4, generator=gen).to(torch.bfloat16).view(torch.int16)
                u = lambda lo, hi, n: torch.empty(n, dtype=torch.float32, device=dev).uniform_(lo, hi, generator=gen) \
                    .to(torch.bfloat16).view(torch.int16)
                w["a_log"], w["dt_bias"], w["gdn_norm"] = u(-1.0, 1.5, vh), u(-0.5, 0.5, vh), u(0.5, 1.5, dv)
                w["out_proj"] = q(D, cfg.gdn_value_dim, cfg.attn_bits)
            else:
                w["qkv"] = q(2 * cfg.q_dim + 2 * cfg.kv_dim, D, cfg.attn_bits)
                w["q_norm"], w["k_norm"] = normw(cfg.head_dim), normw(cfg.head_dim)
                w["o_proj"] = q(D, cfg.q_dim, cfg.attn_bits)
            F = cfg.moe_intermediate
            mixed = cfg.shared_bits != cfg.expert_bits      # the shared expert then has a blob of its own width

            def fill(pool, n_blobs, o, bits):
                for (rows, n, wo, so, bo) in ((F, D, o.gate_w, o.gate_s, o.gate_b), (F, D, o.up_w, o.up_s, o.up_b),
                                              (D, F, o.down_w, o.down_s, o.down_b)):
                    p_, s_, b_ = q(n_blobs * rows, n, bits)
                    wb, mb = rows * n * bits // 8, rows * n // 32
                    pool[:, wo:wo + wb] = p_.view(n_blobs, wb)
                    pool[:, so:so + mb] = s_.view(torch.uint8).view(n_blobs, mb)
                    pool[:, bo:bo + mb] = b_.view(torch.uint8).view(n_blobs, mb)
                    del p_, s_, b_

            n_pool = cfg.num_experts + (0 if mixed else 1)
            pool = torch.empty((n_pool, stride), dtype=torch.uint8, device=dev)
            fill(pool, n_pool, off, cfg.expert_bits)
            w["pool"] = pool
            w["router"] = _randn(gen, (cfg.num_experts, D), std, dev).view(torch.int16)
            w["gate"] = q(1, D, 8)
            if mixed:
                s_off, s_stride = ops.expert_offsets(D, F, cfg.shared_bits)
                blob = torch.empty((1, s_stride), dtype=torch.uint8, device=dev)
                fill(blob, 1, s_off, cfg.shared_bits)
                w["shared"] = dict(blob=blob[0], offsets=s_off, bits=cfg.shared_bits, gate=ops.rows_desc(8, *w["gate"]))
                w["moe"] = ops.moe_layer_desc(D, F, cfg.num_experts, cfg.top_k, cfg.expert_bits,
                                              ops.rows_desc(16, w["router"]), pool)
            else:
                w["moe"] = ops.moe_layer_desc(D, F, cfg.num_experts, cfg.top_k, cfg.expert_bits,
                                              ops.rows_desc(16, w["router"]), pool[:cfg.num_experts], pool[cfg.num_experts],
                                              ops.rows_desc(8, *w["gate"]))
            self.layers.append(w)


def _from_gturbo(cls, ctx, model, gdn=None, kv_bits=8, gdn_state_bf16=True):
    """HybridWeights (and its HybridConfig) from an opened model directory (gturbo.GTurboModel): the resident
    tensors bound by the reference's names (Model.swift:137-306), the matrices of a projection group stacked
    as the rows of one matrix (one launch per group), each layer's experts in HBM with the shared expert as
    the pool's last row -- or, when quant.sharedExpert differs from quant.routedExpert, in a blob of its own
    that the step runs beside the routed block.  The manifest carries no gated-DeltaNet head shape (the reference compiles it in,
    ModelTypes.swift:162-204): value heads, value head size and conv taps are read off the tensor shapes,
    key heads assume key head size = value head size unless gdn = (Hk, Hv, Dk, Dv, taps) says otherwise.
    Returns (config, weights)."""
    import numpy as np

    from . import gturbo as G
    a, q = model.manifest.arch, model.manifest.quant
    if q is None:
        raise G.ModelError("indexCorrupt", "manifest.quant is required by the executable runtime schema")
    mixed = not model.shared_matches_routed()           # the shared expert then runs beside the routed block, at its width
    mask = a["fullAttentionLayerMask"]
    if any(v == 0 for v in mask):
        raise G.ModelError("unsupportedArch", "sliding-window layers")
    D, layers = a["hiddenSize"], a["numLayers"]
    dev = ctx.device
    keep = []

    def t3(name, bits):
        """(codes, scales, biases) device tensors of an affine matrix, or (BF16 bits, None, None) of a dense one."""
        w, s_, b_, e = model.resident(name)
        up = lambda x, dt: torch.from_numpy(np.array(x)).to(dev).view(dt)
        if e.dtype == 1:
            return (up(w, torch.int16).view(e.shape[0], -1), None, None), 16, e.shape
        rows = e.shape[0]
        return (up(w, torch.uint8).view(rows, -1), up(s_.view(np.uint8), torch.int16).view(rows, -1),
                up(b_.view(np.uint8), torch.int16).view(rows, -1)), bits, e.shape

    def bf(name):
        w, _, _, e = model.resident(name)
        if e.dtype != 1:
            raise G.ModelError("indexCorrupt", "%s must be BF16" % name)
        return torch.from_numpy(np.array(w)).to(dev).view(torch.int16)

    def stack(names, bits):
        parts = [t3(n, bits) for n in names]
        if any(p[1] != bits for p in parts):
            raise G.ModelError("indexCorrupt", "%s: the matrices of one projection group differ in format" % names[0])
        return tuple(torch.cat([p[0][j] for p in parts]).contiguous() for j in range(3)), [p[2][0] for p in parts]

    first_linear = next((L for L in range(layers) if mask[L] == 2), None)
    if gdn is None and first_linear is not None:
        p = G.LAYER_PREFIX % first_linear
        _, _, _, ea = model.resident(p + "linear_attn.in_proj_a.weight")
        _, _, _, en = model.resident(p + "linear_attn.norm.weight")
        _, _, _, eq = model.resident(p + "linear_attn.in_proj_qkv.weight")
        _, _, _, ec = model.resident(p + "linear_attn.conv1d.weight")
        vh, dv, qkv_rows = ea.shape[0], en.shape[0], eq.shape[0]
        conv_count = int(np.prod([n for n in ec.shape if n]))      # the index pads shapes with zeros
        if (qkv_rows - vh * dv) % (2 * dv) or conv_count % qkv_rows:
            raise G.ModelError("indexCorrupt", "gated-DeltaNet tensor shapes do not give a head layout; pass gdn=")
        gdn = ((qkv_rows - vh * dv) // (2 * dv), vh, dv, dv, conv_count // qkv_rows)
    attn_bits, embed_bits, expert_bits = q["attention"].weightBits, q["embedding"].weightBits, q["routedExpert"].weightBits
    self = cls.__new__(cls)
    self.ctx = ctx
    self.embed, _, _ = t3("language_model.model.embed_tokens.weight", embed_bits)
    self.lm_head, head_bits, _ = t3("language_model.lm_head.weight", embed_bits)
    self.final_norm = bf("language_model.model.norm.weight")
    cfg = HybridConfig(hidden=D, layers=layers, num_heads=a["numHeads"], num_kv_heads=a["numFullKVHeads"],
                       head_dim=a["fullHeadDim"], rotary_dim=int(round(a["partialRotaryFactor"] * a["fullHeadDim"])),
                       rope_theta=a["fullRopeTheta"], gdn=gdn or (1, 1, 32, 32, 1), num_experts=a["numExperts"],
                       top_k=a["topKExperts"], moe_intermediate=a["moeIntermediateSize"], vocab=a["vocabSize"],
                       expert_bits=expert_bits, attn_bits=attn_bits, kv_bits=kv_bits, head_bits=head_bits,
                       embed_bits=embed_bits, logit_softcap=a["finalLogitSoftcap"], gdn_state_bf16=gdn_state_bf16,
                       full_mask=[v == 1 for v in mask], shared_bits=q["sharedExpert"].weightBits)
    self.cfg = cfg
    self.layers = []
    for L in range(layers):
        p = G.LAYER_PREFIX % L
        w = dict(in_norm=bf(p + "input_layernorm.weight"), post_norm=bf(p + "post_attention_layernorm.weight"))
        if cfg.is_linear(L):
            w["in_proj"], rows = stack([p + n for n in G.LINEAR_PROJECTIONS], attn_bits)
            if rows != [cfg.gdn_qkv_dim, cfg.gdn_value_dim, gdn[1], gdn[1]]:
                raise G.ModelError("indexCorrupt", "layer %d: linear_attn projection rows %s do not fit the head layout %s"
                                   % (L, rows, gdn))
            w["out_proj"], _, _ = t3(p + "linear_attn.out_proj.weight", attn_bits)
            w["conv_w"] = bf(p + "linear_attn.conv1d.weight").view(cfg.gdn_qkv_dim, gdn[4])
            w["a_log"], w["dt_bias"] = bf(p + "linear_attn.A_log"), bf(p + "linear_attn.dt_bias")
            w["gdn_norm"] = bf(p + "linear_attn.norm.weight")
        else:
            w["qkv"], rows = stack([p + n for n in G.FULL_PROJECTIONS], attn_bits)
            if rows != [2 * cfg.q_dim, cfg.kv_dim, cfg.kv_dim]:
                raise G.ModelError("indexCorrupt", "layer %d: self_attn projection rows %s do not fit %d heads of %d"
                                   % (L, rows, cfg.num_heads, cfg.head_dim))
            w["o_proj"], _, _ = t3(p + "self_attn.o_proj.weight", attn_bits)
            w["q_norm"], w["k_norm"] = bf(p + "self_attn.q_norm.weight"), bf(p + "self_attn.k_norm.weight")
        w["pool"] = model.expert_pool(L, dev, with_shared=not mixed)
        w["moe"], held = model.moe_layer(L, w["pool"], dev)
        if mixed:
            s_off, _, _ = model.shared_expert_offsets(L)
            blob = torch.from_numpy(model.shared_expert_blob(L)).to(dev)
            gate = model._rows(p + "mlp.shared_expert_gate.weight", q["router"].weightBits, dev, held)
            w["shared"] = dict(blob=blob, offsets=ops.ExpertOffsets(*[int(v) for v in s_off]), bits=cfg.shared_bits, gate=gate)
        keep.append(held)
        self.layers.append(w)
    self._keep = keep
    return cfg, self


HybridWeights.from_gturbo = classmethod(_from_gturbo)


class HybridDecoder:
    """One decode step for `batch` sequences: buffers, recurrent states and KV caches are allocated
    once; step() only enqueues kernels."""

    def __init__(self, ctx, cfg, weights, batch=1, max_context=32768):
        self.ctx, self.cfg, self.w, self.batch, self.max_context = ctx, cfg, weights, batch, max_context
        dev, dt = ctx.device, ctx.dtype
        D = cfg.hidden
        buf = lambda *shape: torch.zeros(shape, dtype=dt, device=dev)
        self.hidden, self.normed, self.branch = buf(batch, D), buf(batch, D), buf(batch, D)
        self.hidden_alt = buf(batch, D)            # the residual rows alternate between two buffers
        self.moe_out = buf(batch, D)
        self.shared_out = buf(batch, D)           # a shared expert of another width than the routed ones
        kh, vh, dk, dv, taps = cfg.gdn
        self.gdn = ops.GDN(ctx, kh, vh, dk, dv, taps)
        self.lin_rows = cfg.gdn_qkv_dim + cfg.gdn_value_dim + 2 * vh
        self.lin_proj, self.conv_out, self.gdn_out = buf(batch, self.lin_rows), buf(batch, cfg.gdn_qkv_dim), buf(batch, cfg.gdn_value_dim)
        self.full_rows = 2 * cfg.q_dim + 2 * cfg.kv_dim
        self.full_proj = buf(batch, self.full_rows)
        self.q, self.gate, self.attn_out = buf(batch, cfg.num_heads, cfg.head_dim), buf(batch, cfg.num_heads, cfg.head_dim), \
            buf(batch, cfg.num_heads, cfg.head_dim)
        self.k_stage, self.v_stage = buf(batch, cfg.kv_dim), buf(batch, cfg.kv_dim)
        self.logits = buf(batch, cfg.vocab)
        self.probs = torch.zeros((batch, cfg.vocab), dtype=torch.float16, device=dev)
        self.tokens = torch.zeros(batch, dtype=torch.int32, device=dev)
        self.next_tokens = torch.zeros(batch, dtype=torch.int32, device=dev)
        self.positions = torch.zeros(batch, dtype=torch.int32, device=dev)
        self.gdn_states, self.kv = {}, {}
        for L in range(cfg.layers):
            if cfg.is_linear(L):
                self.gdn_states[L] = self.gdn.new_state(batch, bf16=cfg.gdn_state_bf16)
            else:
                self.kv[L] = (ops.KVCache(batch, max_context, cfg.kv_dim, cfg.kv_bits, dev),
                              ops.KVCache(batch, max_context, cfg.kv_dim, cfg.kv_bits, dev))
        self.moe = ops.MoE(ctx, cfg.expert_bits)
        self.attn = ops.Attention(ctx)
        self.quant = ops.KVCacheQuantizer(ctx)
        self.softmax = ops.LogitSoftcapSoftmaxTiled(ctx, cfg.vocab)
        self.sampler = ops.SampleTopK64(ctx, cfg.vocab) if cfg.vocab <= 262144 else None
        self.ew = ops.Elementwise(ctx)

    # -- attention branches ---------------------------------------------------------------------
    def _input_projection(self, p_, s_, b_, rows, out, pre):
        """The fused input projections of a layer over its normed input rows.  pre = the norm weight
        of this layer when the residual add of the MoE block before it and this norm are still to
        be done: the projection launch then does both itself (up to four sequences; same bits)
        and the updated residual rows go to the second buffer."""
        cfg = self.cfg
        if pre is None:
            ops.affine_gemv(self.ctx, p_, s_, b_, cfg.attn_bits, self.normed, rows, cfg.hidden, y=out)
            return
        ops.affine_gemv_prenorm(self.ctx, p_, s_, b_, cfg.attn_bits, self.hidden, self.moe_out, pre, self.hidden_alt, rows,
                                cfg.hidden, y=out, normed_scratch=self.normed, eps=cfg.rms_eps)
        self.hidden, self.hidden_alt = self.hidden_alt, self.hidden

    def _linear_attention(self, L, w, pre=None):
        cfg, B = self.cfg, self.batch
        vh = cfg.gdn[1]
        p_, s_, b_ = w["in_proj"]
        self._input_projection(p_, s_, b_, self.lin_rows, self.lin_proj, pre)
        qkv = self.lin_proj[:, :cfg.gdn_qkv_dim]
        z = self.lin_proj[:, cfg.gdn_qkv_dim:cfg.gdn_qkv_dim + cfg.gdn_value_dim]
        a = self.lin_proj[:, cfg.gdn_qkv_dim + cfg.gdn_value_dim:cfg.gdn_qkv_dim + cfg.gdn_value_dim + vh]
        b = self.lin_proj[:, cfg.gdn_qkv_dim + cfg.gdn_value_dim + vh:]
        tail, state = self.gdn_states[L]
        g = self.gdn
        if B >= 8:
            # conv + q / k norm + tail update + delta rule + gated norm of the token in one launch (same
            # bits; measured: 6.07 -> 6.00 ms per step at 16 sequences, no gain below -- one block per key
            # head is half as many blocks as the delta kernel's, and a single token leaves the device empty)
            check(lib.nvmai_hip_gdn_decode_step(self.ctx.handle, ops._stream(), C.byref(g.cfg), ops._ptr(qkv), self.lin_rows,
                                                ops._ptr(tail), ops._ptr(w["conv_w"]), ops._ptr(self.conv_out),
                                                cfg.gdn_qkv_dim, ops._ptr(a), ops._ptr(b), self.lin_rows,
                                                ops._ptr(w["a_log"]), ops._ptr(w["dt_bias"]), ops._ptr(state),
                                                int(state.dtype == torch.bfloat16), ops._ptr(z), self.lin_rows,
                                                ops._ptr(w["gdn_norm"]), ops._ptr(self.gdn_out), cfg.gdn_value_dim, B),
                  "gdn_decode_step")
        else:
            check(lib.nvmai_hip_gdn_conv_norm(self.ctx.handle, ops._stream(), C.byref(g.cfg), ops._ptr(qkv), self.lin_rows,
                                              ops._ptr(tail), ops._ptr(w["conv_w"]), ops._ptr(self.conv_out),
                                              cfg.gdn_qkv_dim, 1, B), "gdn_conv_norm")
            check(lib.nvmai_hip_gdn_delta_gated_norm(self.ctx.handle, ops._stream(), C.byref(g.cfg), ops._ptr(self.conv_out),
                                                     cfg.gdn_qkv_dim, ops._ptr(a), ops._ptr(b), self.lin_rows,
                                                     ops._ptr(w["a_log"]), ops._ptr(w["dt_bias"]), ops._ptr(state),
                                                     int(state.dtype == torch.bfloat16), ops._ptr(z), self.lin_rows,
                                                     ops._ptr(w["gdn_norm"]), ops._ptr(self.gdn_out), cfg.gdn_value_dim, 1, B),
                  "gdn_delta_gated_norm")
        p_, s_, b_ = w["out_proj"]
        ops.affine_gemv(self.ctx, p_, s_, b_, cfg.attn_bits, self.gdn_out, cfg.hidden, cfg.gdn_value_dim, y=self.branch)

    def _full_attention(self, L, w, position, pre=None):
        cfg, B = self.cfg, self.batch
        p_, s_, b_ = w["qkv"]
        self._input_projection(p_, s_, b_, self.full_rows, self.full_proj, pre)
        kc, vc = self.kv[L]
        if cfg.head_dim % 64 == 0 and cfg.kv_bits in (4, 8):
            # split + per-head norm + RoPE + quantize-on-write in one launch: one cache row per sequence,
            # all at `position` (views whose row pitch is the distance between two sequences)
            kview, vview = kc.view(0, position), vc.view(0, position)
            kview.stride, vview.stride = kc.batch_stride, vc.batch_stride
            check(lib.nvmai_hip_attn_qkv_epilogue_kv(self.ctx.handle, ops._stream(), ops._ptr(self.full_proj), self.full_rows,
                                                     1, ops._ptr(w["q_norm"]), ops._ptr(w["k_norm"]), ops._ptr(self.q),
                                                     ops._ptr(self.gate), None, None, cfg.kv_dim, C.byref(kview),
                                                     C.byref(vview), B, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim,
                                                     cfg.rotary_dim, 0, None, position, cfg.rope_theta, cfg.rms_eps),
                  "attn_qkv_epilogue_kv")
        else:
            check(lib.nvmai_hip_attn_qkv_epilogue(self.ctx.handle, ops._stream(), ops._ptr(self.full_proj), self.full_rows, 1,
                                                  ops._ptr(w["q_norm"]), ops._ptr(w["k_norm"]), ops._ptr(self.q),
                                                  ops._ptr(self.gate), ops._ptr(self.k_stage), ops._ptr(self.v_stage),
                                                  cfg.kv_dim, B, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim,
                                                  cfg.rotary_dim, 0, None, position, cfg.rope_theta, cfg.rms_eps),
                  "attn_qkv_epilogue")
            for cache, stage in ((kc, self.k_stage), (vc, self.v_stage)):
                view = cache.view(0, position)
                view.stride = cache.batch_stride
                self.quant.encode(stage, cfg.kv_dim, view, B, cfg.kv_dim)
        # attention and its sigmoid output gate in the same launches
        self.attn.encode_full_gated(self.q, kc, vc, self.gate, cfg.head_dim, cfg.num_heads, cfg.num_kv_heads,
                                    position + 1, out=self.attn_out)
        p_, s_, b_ = w["o_proj"]
        ops.affine_gemv(self.ctx, p_, s_, b_, cfg.attn_bits, self.attn_out.view(B, cfg.q_dim), cfg.hidden, cfg.q_dim,
                        y=self.branch)

    # -- the step ---------------------------------------------------------------------------------
    def forward_hidden(self, position):
        """Embedding lookup of self.tokens through the last layer; leaves the final-normed rows in
        self.normed.  `position` is the index of these tokens in their sequences."""
        cfg, ctx = self.cfg, self.ctx
        e_p, e_s, e_b = self.w.embed
        check(lib.nvmai_hip_embed_lookup(ctx.handle, ops._stream(), ops._ptr(e_p), ops._ptr(e_s), ops._ptr(e_b),
                                         cfg.embed_bits, ops._ptr(self.tokens), 0, self.batch, ops._ptr(self.hidden),
                                         cfg.hidden, cfg.hidden, cfg.vocab, 1.0), "embed_lookup")
        ops.RMSNorm(ctx).encode_bf16w(self.hidden, self.w.layers[0]["in_norm"], out=self.normed, eps=cfg.rms_eps)
        # up to four sequences: the residual add after a MoE block and the input norm of the next layer
        # run inside that layer's projection launch (one launch less per layer)
        fold = self.batch <= 4
        for L, w in enumerate(self.w.layers):
            pre = w["in_norm"] if (fold and L > 0) else None
            if cfg.is_linear(L):
                self._linear_attention(L, w, pre)
            else:
                self._full_attention(L, w, position, pre)
            # residual add + post-attention norm + MoE: the router launch does the add and the norm itself,
            # so the updated residual rows go to the second buffer (other blocks still read the first)
            nxt = self.w.layers[L + 1]["in_norm"] if L + 1 < cfg.layers else self.w.final_norm
            if w.get("shared") is not None:
                # a shared expert of another width (quant.sharedExpert != quant.routedExpert): the routed block on
                # its own, the shared-expert operator at its width over the same normed rows
                # (RealForwardRunner.swift:3866-3912), its output added to the routed sum
                self.moe.decode_layer_prenorm(w["moe"], self.hidden, self.branch, w["post_norm"], self.hidden_alt, self.normed,
                                              self.moe_out, eps=cfg.rms_eps)
                self.hidden, self.hidden_alt = self.hidden_alt, self.hidden
                sh = w["shared"]
                ops.SharedExpertRuntime(ctx, sh["bits"]).encode(sh["blob"], sh["offsets"], self.normed, cfg.hidden,
                                                                cfg.moe_intermediate, shared_gate=sh["gate"], y=self.shared_out)
                self.ew.encode_residual_add(self.moe_out, self.shared_out)
                if not fold or L + 1 == cfg.layers:
                    ops.residual_add_rmsnorm(ctx, self.hidden, self.moe_out, nxt, out=self.normed, eps=cfg.rms_eps)
                continue
            if not fold:
                # five sequences or more: the residual add that closes the layer and the next norm ride in the
                # block's combine launch (the post-attention rows in self.normed are dead by then)
                self.moe.decode_layer_norms(w["moe"], self.hidden, self.branch, w["post_norm"], self.hidden_alt, self.normed,
                                            self.moe_out, nxt, self.normed, eps=cfg.rms_eps)
                self.hidden, self.hidden_alt = self.hidden_alt, self.hidden
                continue
            self.moe.decode_layer_prenorm(w["moe"], self.hidden, self.branch, w["post_norm"], self.hidden_alt, self.normed,
                                          self.moe_out, eps=cfg.rms_eps)
            self.hidden, self.hidden_alt = self.hidden_alt, self.hidden
            if L + 1 == cfg.layers:
                ops.residual_add_rmsnorm(ctx, self.hidden, self.moe_out, nxt, out=self.normed, eps=cfg.rms_eps)
        return self.normed

    # -- prefill: the tokens of ONE sequence, a chunk at a time, through every layer ------------------------
    # RealForwardRunner.prefillChunked / executePrefillChunk (RealForwardRunner.swift:1323-1388, 1503-1733):
    # per chunk encodeLinearAttentionPrefill (:2605-2742) or encodeFullAttentionPrefill (:2744-2913), then
    # encodeRoutedMoEPrefill (:3244+).  The kernels are the prefill ones -- the dense matrix-core product
    # for the projections, the recurrent kernels over the rows of the chunk, causal attention over the
    # quantized cache, the tiled router, the permutation by expert and the grouped GEMM, the shared expert
    # in dense mode -- and they leave the sequence's KV rows, conv tails and recurrent states exactly
    # where step() expects them, so decoding continues at start_position + len(tokens).
    def prefill_chunked(self, tokens, sequence=0, start_position=0, chunk_tokens=2048):
        """tokens: int32 device tensor [n] of sequence `sequence`, the first of them at start_position.
        Returns the final-normed row of the last token, [1, hidden] (the input of head())."""
        n = tokens.numel()
        if n == 0:
            raise ValueError("prefill_chunked needs at least one token")
        if start_position + n > self.max_context:
            raise ValueError("prefill of %d tokens from %d exceeds the cache (%d rows)" % (n, start_position, self.max_context))
        last = None
        for c0 in range(0, n, chunk_tokens):
            last = self._execute_prefill_chunk(tokens[c0:min(n, c0 + chunk_tokens)].contiguous(), sequence,
                                               start_position + c0)
        return last

    def _execute_prefill_chunk(self, tokens, b, start):
        cfg, ctx = self.cfg, self.ctx
        T = tokens.numel()
        e_p, e_s, e_b = self.w.embed
        hidden = torch.empty((T, cfg.hidden), dtype=ctx.dtype, device=ctx.device)
        check(lib.nvmai_hip_embed_lookup(ctx.handle, ops._stream(), ops._ptr(e_p), ops._ptr(e_s), ops._ptr(e_b),
                                         cfg.embed_bits, ops._ptr(tokens), 0, T, ops._ptr(hidden), cfg.hidden, cfg.hidden,
                                         cfg.vocab, 1.0), "embed_lookup")
        norm = ops.RMSNorm(ctx)
        normed = norm.encode_bf16w(hidden, self.w.layers[0]["in_norm"], eps=cfg.rms_eps)
        positions = torch.arange(start, start + T, dtype=torch.int32, device=ctx.device)
        for L, w in enumerate(self.w.layers):
            if cfg.is_linear(L):
                branch = self._linear_attention_prefill(L, w, normed, b, T)
            else:
                branch = self._full_attention_prefill(L, w, normed, b, start, positions, T)
            routed_x = ops.residual_add_rmsnorm(ctx, hidden, branch, w["post_norm"], eps=cfg.rms_eps)
            y = self._routed_moe_prefill(w, routed_x, T)
            nxt = self.w.layers[L + 1]["in_norm"] if L + 1 < cfg.layers else self.w.final_norm
            normed = ops.residual_add_rmsnorm(ctx, hidden, y, nxt, eps=cfg.rms_eps)
        return normed[T - 1:T]

    def _linear_attention_prefill(self, L, w, normed, b, T):
        cfg = self.cfg
        vh = cfg.gdn[1]
        p_, s_, b_ = w["in_proj"]
        proj = ops.affine_gemv(self.ctx, p_, s_, b_, cfg.attn_bits, normed, self.lin_rows, cfg.hidden)
        C_, V = cfg.gdn_qkv_dim, cfg.gdn_value_dim
        qkv, z, a, bb = proj[:, :C_], proj[:, C_:C_ + V], proj[:, C_ + V:C_ + V + vh], proj[:, C_ + V + vh:]
        tail, state = self.gdn_states[L]
        conv = self.gdn.encode_conv_norm(qkv, tail[b:b + 1], w["conv_w"], rows=T)
        out = self.gdn.encode_delta_gated_norm(conv, a, bb, w["a_log"], w["dt_bias"], state[b:b + 1], z, w["gdn_norm"], rows=T)
        p_, s_, b_ = w["out_proj"]
        return ops.affine_gemv(self.ctx, p_, s_, b_, cfg.attn_bits, out, cfg.hidden, cfg.gdn_value_dim)

    def _full_attention_prefill(self, L, w, normed, b, start, positions, T):
        cfg, ctx = self.cfg, self.ctx
        p_, s_, b_ = w["qkv"]
        proj = ops.affine_gemv(ctx, p_, s_, b_, cfg.attn_bits, normed, self.full_rows, cfg.hidden)
        q = torch.empty((T, cfg.num_heads, cfg.head_dim), dtype=ctx.dtype, device=ctx.device)
        gate, out = torch.empty_like(q), torch.empty_like(q)
        kc, vc = self.kv[L]
        if cfg.head_dim % 64 == 0 and cfg.kv_bits in (4, 8):
            # the chunk's K / V rows go into the cache rows start .. start + T - 1 of this sequence
            kview, vview = kc.view(b, start), vc.view(b, start)
            check(lib.nvmai_hip_attn_qkv_epilogue_kv(ctx.handle, ops._stream(), ops._ptr(proj), proj.stride(0), 1,
                                                     ops._ptr(w["q_norm"]), ops._ptr(w["k_norm"]), ops._ptr(q), ops._ptr(gate),
                                                     None, None, cfg.kv_dim, C.byref(kview), C.byref(vview), T, cfg.num_heads,
                                                     cfg.num_kv_heads, cfg.head_dim, cfg.rotary_dim, 0, ops._ptr(positions), 0,
                                                     cfg.rope_theta, cfg.rms_eps), "attn_qkv_epilogue_kv")
        else:
            k = torch.empty((T, cfg.kv_dim), dtype=ctx.dtype, device=ctx.device)
            v = torch.empty_like(k)
            check(lib.nvmai_hip_attn_qkv_epilogue(ctx.handle, ops._stream(), ops._ptr(proj), proj.stride(0), 1,
                                                  ops._ptr(w["q_norm"]), ops._ptr(w["k_norm"]), ops._ptr(q), ops._ptr(gate),
                                                  ops._ptr(k), ops._ptr(v), cfg.kv_dim, T, cfg.num_heads, cfg.num_kv_heads,
                                                  cfg.head_dim, cfg.rotary_dim, 0, ops._ptr(positions), 0, cfg.rope_theta,
                                                  cfg.rms_eps), "attn_qkv_epilogue")
            self.quant.encode(k, cfg.kv_dim, kc.view(b, start), T, cfg.kv_dim)
            self.quant.encode(v, cfg.kv_dim, vc.view(b, start), T, cfg.kv_dim)
        ops.PrefillAttention(ctx).encode_causal(q, kc.view(b, 0), vc.view(b, 0), out, start, T, cfg.head_dim, cfg.num_heads,
                                                cfg.num_kv_heads, start + T)
        self.ew.encode_sigmoid_gate_mul(out, gate)
        p_, s_, b_ = w["o_proj"]
        return ops.affine_gemv(ctx, p_, s_, b_, cfg.attn_bits, out.view(T, cfg.q_dim), cfg.hidden, cfg.q_dim)

    def _routed_moe_prefill(self, w, x, T):
        """The MoE block of a chunk: below 64 rows the decode call (a work list over the distinct
        experts), from 64 rows on the prefill path -- tiled router, permutation by expert, grouped
        GEMM, rank-order reduce -- with the shared expert beside it."""
        cfg, ctx = self.cfg, self.ctx
        D, F, E, K = cfg.hidden, cfg.moe_intermediate, cfg.num_experts, cfg.top_k
        sh = w.get("shared")                 # a shared expert of another width: beside the routed block
        if T < 64 and T * K <= 4096:
            y = self.moe.decode_layer(w["moe"], x)
            if sh is not None:
                self.ew.encode_residual_add(y, ops.SharedExpertRuntime(ctx, sh["bits"]).encode(
                    sh["blob"], sh["offsets"], x, D, F, shared_gate=sh["gate"]))
            return y
        layer = w["moe"]
        idx, wts = self.moe.encode_router(layer.router, x, E, D, K)
        routes = ops.PrefillMoEGrouping(ctx).group_routes(idx, wts, E)
        pool = w["pool"]
        partials, _ = ops.PrefillGroupedRoutedMoE(ctx, cfg.expert_bits).encode(pool[:E], layer.offsets, x, D, F, routes)
        h2 = ops.PrefillMoE(ctx).encode_reduce_token_major(partials, wts, T, K, D)
        if sh is not None:
            shared = ops.SharedExpertRuntime(ctx, sh["bits"]).encode(sh["blob"], sh["offsets"], x, D, F, shared_gate=sh["gate"])
        else:
            shared = ops.SharedExpertRuntime(ctx, cfg.expert_bits).encode(pool[E], layer.offsets, x, D, F,
                                                                          shared_gate=layer.shared_gate)
        return self.ew.encode_residual_add(h2, shared)

    def head(self):
        """LM head over the final-normed rows: logits in self.logits."""
        cfg = self.cfg
        p_, s_, b_ = self.w.lm_head
        ops.affine_gemv(self.ctx, p_, s_, b_, cfg.head_bits, self.normed, cfg.vocab, cfg.hidden, y=self.logits)
        return self.logits

    def sample(self, seeds, temperature=0.6, top_k=20, top_p=0.95):
        """Softcap + softmax and the tiled top-k sampler (Sampler.sample's production path): tokens in
        self.next_tokens."""
        self.softmax.encode(self.logits, self.probs, softcap=self.cfg.logit_softcap)
        check(lib.nvmai_hip_sample_topk64(self.ctx.handle, ops._stream(), ops._ptr(self.probs), self.probs.stride(0),
                                          self.batch, self.cfg.vocab, temperature, top_p,
                                          (C.c_uint64 * self.batch)(*seeds), top_k, ops._ptr(self.next_tokens), None),
              "sample_topk64")
        return self.next_tokens

    def step(self, position, seeds, temperature=0.6, top_k=20, top_p=0.95):
        """tokens (self.tokens) at `position` -> next tokens (self.next_tokens)."""
        self.forward_hidden(position)
        self.head()
        return self.sample(seeds, temperature, top_k, top_p)
