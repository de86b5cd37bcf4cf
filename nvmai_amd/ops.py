"""Host layer over the C ABI: one class or function per reference operator wrapper
(sources/NVMAI/Kernels/...), same argument meaning, errors as exceptions.  Arguments
are torch tensors on the GPU (device memory plumbing); every call only enqueues work
on torch's current stream."""
import ctypes as C

import torch

from . import _lib
from ._lib import ExpertOffsets, GdnConfig, GemvPart, GenerationConfig as _CGenerationConfig, KvView, MoeLayer, PrefillGrouping, Rows, check, lib

ACT_BF16, ACT_FP16 = 0, 1
(PROF_ROUTER, PROF_SELECT, PROF_GROUP, PROF_PHASE1, PROF_PHASE2, PROF_COMBINE, PROF_KV_QUANT,
 PROF_ATTN_PARTIAL, PROF_ATTN_COMBINE, PROF_SOFTMAX, PROF_SAMPLE, PROF_PREFILL_GROUP,
 PROF_PREFILL_GEMM1, PROF_PREFILL_GEMM2, PROF_PREFILL_COMBINE) = range(15)
_ACT_TORCH = {ACT_BF16: torch.bfloat16, ACT_FP16: torch.float16}


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


class Context:
    """nvmai_hip_ctx: stands where the reference has MetalContext (MetalContext.swift)."""

    def __init__(self, device=0, act=ACT_BF16):
        self.act = act
        self.dtype = _ACT_TORCH[act]
        self.device = torch.device("cuda", device)
        h = C.c_void_p()
        check(lib.nvmai_hip_ctx_create(device, act, C.byref(h)), "ctx_create")
        self.handle = h

    def reserve(self, nbytes):
        """Size the workspace now, so that no later call (a captured one above all) has to grow it."""
        check(lib.nvmai_hip_ctx_reserve(self.handle, nbytes), "ctx_reserve")

    @property
    def workspace_bytes(self):
        return lib.nvmai_hip_ctx_workspace_bytes(self.handle)

    def profile_enable(self, on=True):
        check(lib.nvmai_hip_profile_enable(self.handle, int(on)), "profile_enable")

    def profile_read(self, tag):
        """Summed milliseconds and launch count of one NVMAI_PROF_* tag."""
        ms, n = C.c_double(), C.c_uint32()
        check(lib.nvmai_hip_profile_read(self.handle, tag, C.byref(ms), C.byref(n)), "profile_read")
        return ms.value, n.value

    def read_probe(self, data):
        """Launch the kernel that only reads `data` (a contiguous device tensor of a multiple of 16 bytes): the
        measuring stick for the HBM fractions of the streaming kernels."""
        check(lib.nvmai_hip_read_probe(self.handle, _stream(), _ptr(data), data.numel() * data.element_size(), None),
              "read_probe")

    def close(self):
        if self.handle:
            lib.nvmai_hip_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def expert_offsets(d, f, bits):
    """CPUExpertFFN.Offsets(d:f:) (CPUExpertFFN.swift:42-59); returns (offsets, stride)."""
    off, stride = ExpertOffsets(), C.c_uint64()
    check(lib.nvmai_expert_offsets_for(d, f, bits, C.byref(off), C.byref(stride)), "expert_offsets")
    return off, stride.value


def rows_desc(kind, weights, scales=None, biases=None):
    r = Rows()
    r.kind = kind
    r.weights, r.scales, r.biases = weights.data_ptr(), 0 if scales is None else scales.data_ptr(), \
        0 if biases is None else biases.data_ptr()
    r._keep = (weights, scales, biases)
    return r


def quantize_affine(ctx, w, bits, packed=None, scales=None, biases=None):
    """Quantization.quantizeInt4Affine / Int8Affine (Quantization.swift:50-102,135-177) for a
    [rows, n] fp32 or bf16 matrix.  Returns (packed u8, scales u16, biases u16)."""
    rows, n = w.shape
    assert w.is_contiguous() and w.dtype in (torch.float32, torch.bfloat16)
    if packed is None:
        packed = torch.empty((rows, n * bits // 8), dtype=torch.uint8, device=w.device)
        scales = torch.empty((rows, n // 64), dtype=torch.int16, device=w.device)
        biases = torch.empty((rows, n // 64), dtype=torch.int16, device=w.device)
    check(lib.nvmai_hip_quantize_affine(ctx.handle, _stream(), _ptr(w), int(w.dtype == torch.bfloat16),
                                        rows, n, bits, _ptr(packed), _ptr(scales), _ptr(biases)),
          "quantize_affine")
    return packed, scales, biases


def dequantize_affine(ctx, packed, scales, biases, bits, want_codes=True, want_values=True):
    count = packed.numel() * 8 // bits
    codes = torch.empty(count, dtype=torch.uint8, device=packed.device) if want_codes else None
    values = torch.empty(count, dtype=ctx.dtype, device=packed.device) if want_values else None
    check(lib.nvmai_hip_dequantize_affine(ctx.handle, _stream(), _ptr(packed), _ptr(scales), _ptr(biases),
                                          count, bits, _ptr(codes), _ptr(values)), "dequantize_affine")
    return codes, values


def pack_expert(ctx, gate, up, down, bits, blob=None):
    """Quantize gate[f,d], up[f,d], down[d,f] into one expert blob in the reference's order
    (CPUExpertFFN.swift:36-40)."""
    f, d = gate.shape
    off, stride = expert_offsets(d, f, bits)
    if blob is None:
        blob = torch.empty(stride, dtype=torch.uint8, device=gate.device)
    for w, wo, so, bo in ((gate, off.gate_w, off.gate_s, off.gate_b), (up, off.up_w, off.up_s, off.up_b),
                          (down, off.down_w, off.down_s, off.down_b)):
        rows, n = w.shape
        quantize_affine(ctx, w.contiguous(), bits, blob[wo:wo + rows * n * bits // 8],
                        blob[so:so + rows * n // 32], blob[bo:bo + rows * n // 32])
    return blob


def affine_gemv(ctx, weights, scales, biases, bits, x, m, n, out_f32=False, y=None, y_f32=None):
    """DequantInt4GEMV.encode / DequantInt8GEMV.encode / AffineQuantGEMV.encode:
    y[t] = W x[t] for x [tokens, n].  y (activation type) and / or y_f32 may be handed in as
    [tokens, >= m] buffers with one common row stride; both are then written and returned."""
    x2 = x.reshape(-1, x.shape[-1])
    tokens = x2.shape[0]
    if y is not None or y_f32 is not None:
        stride = (y if y is not None else y_f32).stride(0)
        assert y is None or y_f32 is None or y.stride(0) == y_f32.stride(0)
        check(lib.nvmai_hip_affine_gemv(ctx.handle, _stream(), _ptr(weights), _ptr(scales), _ptr(biases), bits,
                                        _ptr(x2), x2.stride(0), tokens, m, n, _ptr(y), _ptr(y_f32), stride),
              "affine_gemv")
        return y, y_f32
    y = None if out_f32 else torch.empty((tokens, m), dtype=ctx.dtype, device=x.device)
    yf = torch.empty((tokens, m), dtype=torch.float32, device=x.device) if out_f32 else None
    check(lib.nvmai_hip_affine_gemv(ctx.handle, _stream(), _ptr(weights), _ptr(scales), _ptr(biases), bits,
                                    _ptr(x2), x2.stride(0), tokens, m, n, _ptr(y), _ptr(yf), m),
          "affine_gemv")
    return yf if out_f32 else y


def int4_affine_gemv(weights, scales, biases, x, rows, n):
    """nvmai_int4_affine_gemv (nvmai_kernels.h:22-28): numpy host arrays in, fp32 numpy out."""
    import numpy as np
    w = np.ascontiguousarray(weights, np.uint8)
    s = np.ascontiguousarray(scales, np.uint16)
    b = np.ascontiguousarray(biases, np.uint16)
    xv = np.ascontiguousarray(x, np.float32)
    out = np.empty(rows, np.float32)
    lib.nvmai_int4_affine_gemv(w.ctypes.data, s.ctypes.data, b.ctypes.data, xv.ctypes.data, rows, n,
                               out.ctypes.data)
    return out


class MoE:
    """Mirror of the reference's `MoE` operator class (MoE.swift:31-464): router, routed
    phase 1 / phase 2 over top-k blobs, plus the resident-pool decode layer."""
    max_streamed_experts = 8

    def __init__(self, ctx, bits=4):
        self.ctx, self.bits = ctx, bits

    def encode_router(self, router, hidden, num_experts, d, top_k, effective_scale=None,
                      per_expert_scale=None, want_logits=False):
        """MoE.encodeRouter (MoE.swift:151-213) / PrefillRouter.encodeBlock for [tokens, d] rows."""
        h = hidden.reshape(-1, hidden.shape[-1])
        tokens = h.shape[0]
        idx = torch.empty((tokens, top_k), dtype=torch.int32, device=h.device)
        w = torch.empty((tokens, top_k), dtype=torch.float16, device=h.device)
        logits = torch.empty((tokens, num_experts), dtype=torch.float32, device=h.device) if want_logits else None
        check(lib.nvmai_hip_moe_router_topk(self.ctx.handle, _stream(), C.byref(router), _ptr(h), h.stride(0),
                                            tokens, _ptr(effective_scale), _ptr(per_expert_scale),
                                            num_experts, d, top_k, _ptr(idx), _ptr(w), _ptr(logits)),
              "moe_router_topk")
        return (idx, w, logits) if want_logits else (idx, w)

    @staticmethod
    def _blob_table(blobs):
        return (C.c_void_p * len(blobs))(*[b.data_ptr() for b in blobs])

    def encode_routed_phase1(self, blobs, offsets, x, acts, d, f, top_k, active_slots=None):
        """MoE.encodeRoutedPersistentPhase1U16Load / ...SubsetU16Load (MoE.swift:295-392)."""
        table = self._blob_table(blobs)
        if active_slots is None:
            rc = lib.nvmai_hip_moe_phase1_gate_up_act(self.ctx.handle, _stream(), table, C.byref(offsets),
                                                      self.bits, _ptr(x), _ptr(acts), d, f, top_k)
        else:
            rc = lib.nvmai_hip_moe_phase1_gate_up_act_subset(
                self.ctx.handle, _stream(), table, C.byref(offsets), self.bits, _ptr(x), _ptr(acts), d, f,
                top_k, _ptr(active_slots), active_slots.numel())
        check(rc, "moe_phase1_gate_up_act")

    def encode_routed_phase2_reduce(self, blobs, offsets, acts, routing_weights, residual, y, d, f, top_k):
        """MoE.encodeRoutedPersistentPhase2Reduce (MoE.swift:394-440)."""
        check(lib.nvmai_hip_moe_phase2_down_reduce(self.ctx.handle, _stream(), self._blob_table(blobs),
                                                   C.byref(offsets), self.bits, _ptr(acts),
                                                   _ptr(routing_weights), _ptr(residual), _ptr(y), d, f, top_k),
              "moe_phase2_down_reduce")

    def decode_layer(self, layer, x, y=None, want_routes=False, stats=None):
        """One MoE layer over a decode batch with all experts resident (nvmai_hip_moe_decode_layer)."""
        x2 = x.reshape(-1, x.shape[-1])
        tokens = x2.shape[0]
        if y is None:
            y = torch.empty((tokens, layer.d), dtype=self.ctx.dtype, device=x.device)
        idx = w = None
        if want_routes:
            idx = torch.empty((tokens, layer.top_k), dtype=torch.int32, device=x.device)
            w = torch.empty((tokens, layer.top_k), dtype=torch.float16, device=x.device)
        check(lib.nvmai_hip_moe_decode_layer(self.ctx.handle, _stream(), C.byref(layer), _ptr(x2), x2.stride(0),
                                             tokens, _ptr(y), y.stride(0), _ptr(idx), _ptr(w), _ptr(stats)),
              "moe_decode_layer")
        return (y, idx, w) if want_routes else y

    def decode_layer_noalloc(self, layer, x, y, idx=None, w=None, stats=None):
        """nvmai_hip_moe_decode_layer_noalloc: the same step with its intermediate buffers in the
        library's static device array; every output is the caller's, nothing is allocated."""
        x2 = x.reshape(-1, x.shape[-1])
        check(lib.nvmai_hip_moe_decode_layer_noalloc(self.ctx.handle, _stream(), C.byref(layer), _ptr(x2),
                                                     x2.stride(0), x2.shape[0], _ptr(y), y.stride(0), _ptr(idx),
                                                     _ptr(w), _ptr(stats)), "moe_decode_layer_noalloc")
        return y

    def decode_layer_prenorm(self, layer, hidden, delta, norm_weight, hidden_out, normed, y, eps=1e-6, idx=None,
                             w=None, stats=None):
        """nvmai_hip_moe_decode_layer_prenorm: hidden_out = hidden + delta (delta None: a copy),
        normed = rmsnorm(hidden_out) * norm_weight, y = MoE(normed); below 64 tokens the router
        launch does the add and the norm itself.  Every buffer is the caller's."""
        h2 = hidden.reshape(-1, hidden.shape[-1])
        check(lib.nvmai_hip_moe_decode_layer_prenorm(
            self.ctx.handle, _stream(), C.byref(layer), _ptr(h2), h2.stride(0), _ptr(delta),
            0 if delta is None else delta.stride(0), _ptr(norm_weight), eps, _ptr(hidden_out), hidden_out.stride(0),
            _ptr(normed), normed.stride(0), h2.shape[0], _ptr(y), y.stride(0), _ptr(idx), _ptr(w), _ptr(stats)),
            "moe_decode_layer_prenorm")
        return y


    def decode_layer_norms(self, layer, hidden, delta, norm_weight, hidden_out, normed, y, next_norm_weight, next_normed,
                           eps=1e-6, idx=None, w=None, stats=None):
        """nvmai_hip_moe_decode_layer_norms: decode_layer_prenorm, then hidden_out += y and
        next_normed = rmsnorm(hidden_out) * next_norm_weight (the residual add that closes the layer and
        the norm that opens the next); from five tokens on in the block's combine launch."""
        h2 = hidden.reshape(-1, hidden.shape[-1])
        check(lib.nvmai_hip_moe_decode_layer_norms(
            self.ctx.handle, _stream(), C.byref(layer), _ptr(h2), h2.stride(0), _ptr(delta),
            0 if delta is None else delta.stride(0), _ptr(norm_weight), eps, _ptr(hidden_out), hidden_out.stride(0),
            _ptr(normed), normed.stride(0), h2.shape[0], _ptr(y), y.stride(0), _ptr(idx), _ptr(w), _ptr(stats),
            _ptr(next_norm_weight), _ptr(next_normed), next_normed.stride(0)), "moe_decode_layer_norms")
        return y


def moe_layer_desc(d, f, num_experts, top_k, bits, router, experts, shared_blob=None, shared_gate=None,
                   eff_scale=None, per_expert_scale=None, offsets=None):
    """Fill an nvmai_moe_layer.  experts: uint8 tensor [num_experts, stride] (resident pool).
    offsets: the nine sub-tensor offsets inside a blob when they come from a packed-experts layout
    (Model.routedExpertOffsets); default = CPUExpertFFN.Offsets(d:f:)."""
    L = MoeLayer()
    L.d, L.f, L.num_experts, L.top_k, L.bits = d, f, num_experts, top_k, bits
    L.router = router
    L.experts_base, L.expert_stride = experts.data_ptr(), experts.stride(0)
    if offsets is None:
        L.offsets, _ = expert_offsets(d, f, bits)
    else:
        L.offsets = ExpertOffsets(*[int(v) for v in offsets])
    L.shared_blob = 0 if shared_blob is None else shared_blob.data_ptr()
    if shared_gate is not None:
        L.shared_gate = shared_gate
    L.eff_scale = 0 if eff_scale is None else eff_scale.data_ptr()
    L.per_expert_scale = 0 if per_expert_scale is None else per_expert_scale.data_ptr()
    L._keep = (router, experts, shared_blob, shared_gate, eff_scale, per_expert_scale)
    return L


class SharedExpertRuntime:
    """Mirror of SharedExpertRuntime (SharedExpertInt4.swift:100-153) with the scalar sigmoid
    gate of RealForwardRunner.swift:3884-3900 folded in."""

    def __init__(self, ctx, weight_bits):
        if weight_bits not in (4, 8):
            raise _lib.NvmaiError(-2, "SharedExpertRuntime(weightBits=%d)" % weight_bits)
        self.ctx, self.bits = ctx, weight_bits

    def encode(self, blob, offsets, x, d, f, shared_gate=None, y=None):
        x2 = x.reshape(-1, x.shape[-1])
        tokens = x2.shape[0]
        if y is None:
            y = torch.empty((tokens, d), dtype=self.ctx.dtype, device=x.device)
        gate = C.byref(shared_gate) if shared_gate is not None else None
        check(lib.nvmai_hip_shared_expert(self.ctx.handle, _stream(), _ptr(blob), C.byref(offsets), self.bits,
                                          gate, _ptr(x2), x2.stride(0), tokens, _ptr(y), y.stride(0), d, f),
              "shared_expert")
        return y


# ---------------------------------------------------------------------------------------------
# KV cache, RoPE, attention
# ---------------------------------------------------------------------------------------------
# ---------------------------------------------------------------- prefill
GROUPING_ERRORS = {1: "invalidQueryCount", 2: "invalidTopK", 3: "invalidNumExperts",
                   4: "invalidTileExpertCount", 5: "pairCountMismatch", 6: "tokenOutOfRange",
                   7: "rankOutOfRange", 8: "expertOutOfRange", 9: "duplicateTokenRank",
                   10: "expertSortKeyCountMismatch"}


class PrefillMoEGroupingError(Exception):
    """PrefillMoEGroupingError (PrefillMoEGrouping.swift:52-89); `pair_index` is the first
    failing pair for the per-pair cases."""

    def __init__(self, code, pair_index=None):
        self.code, self.name, self.pair_index = code, GROUPING_ERRORS.get(code, str(code)), pair_index
        super().__init__(self.name if pair_index is None else "%s (pair %d)" % (self.name, pair_index))


class PrefillRouter:
    """PrefillRouter (PrefillRouter.swift:30-117): block router and pair records."""

    def __init__(self, ctx):
        self.ctx = ctx
        self._moe = MoE(ctx)

    def encode_block(self, router, hidden, num_experts, d, top_k, effective_scale=None, per_expert_scale=None):
        """PrefillRouter.encodeBlock (PrefillRouter.swift:41-95): idx u32 and FP16 weights [tokens, top_k]."""
        return self._moe.encode_router(router, hidden, num_experts, d, top_k, effective_scale, per_expert_scale)

    def make_token_expert_pairs(self, indices, weights):
        """PrefillRouter.makeTokenExpertPairs (PrefillRouter.swift:97-117): int32 [tokens*top_k, 4]
        records {token, expert, rank, weight bits}."""
        tokens, top_k = indices.shape
        pairs = torch.empty((tokens * top_k, 4), dtype=torch.int32, device=indices.device)
        check(lib.nvmai_hip_prefill_make_pairs(self.ctx.handle, _stream(), _ptr(indices), _ptr(weights), tokens,
                                               top_k, _ptr(pairs)), "prefill_make_pairs")
        return pairs


class PrefillMoEGroupedRoutes:
    """PrefillMoEGroupedRoutes (PrefillMoEGrouping.swift:31-50) held in device memory."""

    def __init__(self, n_pairs, query_count, top_k, num_experts, tile_expert_count, device):
        i32 = dict(dtype=torch.int32, device=device)
        self.query_count, self.top_k, self.num_experts = query_count, top_k, num_experts
        self.tile_expert_count = tile_expert_count
        self.sorted_pairs = torch.empty((n_pairs, 4), **i32)
        self.per_expert_offsets = torch.empty(num_experts, **i32)
        self.per_expert_counts = torch.empty(num_experts, **i32)
        self.groups_buf = torch.empty((num_experts, 3), **i32)
        self.tiles_buf = torch.empty((num_experts, 4), **i32)
        self.info = torch.empty(8, **i32)           # words 0..4 are written by every grouping call
        self.desc = PrefillGrouping(*(t.data_ptr() for t in (self.sorted_pairs, self.per_expert_offsets,
                                                             self.per_expert_counts, self.groups_buf,
                                                             self.tiles_buf, self.info)))

    def validate(self):
        """Waits for the device and raises what the reference would have thrown."""
        info = self.info.cpu().tolist()
        if info[2]:
            raise PrefillMoEGroupingError(info[2], info[3])
        return info

    @property
    def groups(self):
        return self.groups_buf[: self.validate()[0]]

    @property
    def tiles(self):
        return self.tiles_buf[: self.validate()[1]]


class PrefillMoEGrouping:
    """PrefillMoEGrouping (PrefillMoEGrouping.swift:91-192) on the device."""

    def __init__(self, ctx):
        self.ctx = ctx

    @staticmethod
    def _check(n_pairs, query_count, top_k, num_experts, tile_expert_count, sort_keys):
        code = lib.nvmai_prefill_grouping_check(n_pairs, query_count, top_k, num_experts, tile_expert_count,
                                                sort_keys is not None, 0 if sort_keys is None else sort_keys.numel())
        if code:
            raise PrefillMoEGroupingError(code)

    def group_token_expert_pairs(self, pairs, query_count, top_k, num_experts, tile_expert_count=16,
                                 expert_sort_keys=None, validate=True):
        """groupTokenExpertPairs: pairs int32 [n, 4] in any order; expert_sort_keys int64 [num_experts]."""
        n = pairs.shape[0]
        self._check(n, query_count, top_k, num_experts, tile_expert_count, expert_sort_keys)
        out = PrefillMoEGroupedRoutes(n, query_count, top_k, num_experts, tile_expert_count, pairs.device)
        check(lib.nvmai_hip_prefill_group_pairs(self.ctx.handle, _stream(), _ptr(pairs), n, query_count, top_k,
                                                num_experts, tile_expert_count, _ptr(expert_sort_keys),
                                                0 if expert_sort_keys is None else expert_sort_keys.numel(),
                                                C.byref(out.desc)), "prefill_group_pairs")
        if validate:
            out.validate()
        return out

    def group_routes(self, indices, weights, num_experts, tile_expert_count=16, expert_sort_keys=None,
                     validate=False):
        """makeTokenExpertPairs + groupTokenExpertPairs from the router's outputs, no host step."""
        query_count, top_k = indices.shape
        self._check(query_count * top_k, query_count, top_k, num_experts, tile_expert_count, expert_sort_keys)
        out = PrefillMoEGroupedRoutes(query_count * top_k, query_count, top_k, num_experts, tile_expert_count,
                                      indices.device)
        check(lib.nvmai_hip_prefill_group_routes(self.ctx.handle, _stream(), _ptr(indices), _ptr(weights),
                                                 query_count, top_k, num_experts, tile_expert_count,
                                                 _ptr(expert_sort_keys),
                                                 0 if expert_sort_keys is None else expert_sort_keys.numel(),
                                                 C.byref(out.desc)), "prefill_group_routes")
        if validate:
            out.validate()
        return out


class PrefillGroupedRoutedMoE:
    """PrefillGroupedRoutedMoE.encodeStreamedBatched over all tiles (PrefillGroupedRoutedMoE.swift:413-489)
    with the experts resident: expert e at experts[e] of a [num_experts, stride] uint8 pool."""

    def __init__(self, ctx, bits=4):
        self.ctx, self.bits = ctx, bits

    def encode(self, experts, offsets, hidden, d, f, routes, act_scratch=None, route_partials=None):
        n = routes.sorted_pairs.shape[0]
        if act_scratch is None:
            act_scratch = torch.empty((n, f), dtype=self.ctx.dtype, device=hidden.device)
        if route_partials is None:
            route_partials = torch.empty((n, d), dtype=self.ctx.dtype, device=hidden.device)
        check(lib.nvmai_hip_prefill_grouped_moe(self.ctx.handle, _stream(), _ptr(experts), experts.stride(0),
                                                C.byref(offsets), self.bits, d, f, experts.shape[0], _ptr(hidden),
                                                hidden.stride(0), routes.query_count, routes.top_k,
                                                C.byref(routes.desc), _ptr(act_scratch), _ptr(route_partials)),
              "prefill_grouped_moe")
        return route_partials, act_scratch


    def encode_streamed_batched(self, hidden, sorted_pairs, route_partials, act_scratch, binding, params, err=None):
        """encodeStreamedBatched for one tile (PrefillGroupedRoutedMoE.swift:413-489): the pairs
        [params.pair_start, + params.pair_count) of sorted_pairs through the experts of `binding`."""
        if params.live_expert_count != len(binding.expert_ids):
            raise PrefillGroupedRoutedMoEError("params were made for another binding")
        ptrs = (C.c_void_p * len(binding.views))(*binding.pointers())
        check(lib.nvmai_hip_prefill_grouped_moe_streamed(self.ctx.handle, _stream(), C.byref(params), ptrs, self.bits,
                                                         _ptr(hidden), _ptr(sorted_pairs), sorted_pairs.shape[0],
                                                         _ptr(act_scratch), _ptr(route_partials), _ptr(err)),
              "prefill_grouped_moe_streamed")
        return route_partials


class PrefillGroupedRoutedMoEError(Exception):
    """PrefillGroupedRoutedMoEError.invalidStreamedTileBinding (PrefillGroupedRoutedMoE.swift:325-337)."""


class PrefillStreamedTileLifetimeError(Exception):
    """PrefillStreamedTileLifetimeError (PrefillGroupedRoutedMoE.swift:49-64): .kind is 'duplicateSlots',
    'slotReuseBeforeCompletion' or 'completeWithoutInFlightTile'."""

    def __init__(self, kind, tile_index, conflicting_tile_index=None, slots=()):
        super().__init__("prefill streamed tile %d: %s %s" % (tile_index, kind, list(slots)))
        self.kind, self.tile_index = kind, tile_index
        self.conflicting_tile_index, self.slots = conflicting_tile_index, list(slots)


class PrefillStreamedTileSlotLifetime:
    """PrefillStreamedTileSlotLifetime (PrefillGroupedRoutedMoE.swift:66-102): which cache slots the
    tiles in flight hold, so that a slot is not refilled before the tile reading it has completed."""

    def __init__(self):
        self.in_flight = {}

    def begin(self, tile_index, planned_slots):
        slots = set()
        for slot in planned_slots:
            if slot in slots:
                raise PrefillStreamedTileLifetimeError("duplicateSlots", tile_index, slots=sorted(planned_slots))
            slots.add(slot)
        for other, other_slots in self.in_flight.items():
            overlap = slots & other_slots
            if overlap:
                raise PrefillStreamedTileLifetimeError("slotReuseBeforeCompletion", tile_index, other, sorted(overlap))
        self.in_flight[tile_index] = slots

    def complete(self, tile_index):
        if self.in_flight.pop(tile_index, None) is None:
            raise PrefillStreamedTileLifetimeError("completeWithoutInFlightTile", tile_index)


class PrefillStreamedTileBinding:
    """PrefillStreamedTileBinding (PrefillGroupedRoutedMoE.swift:185-323): the experts of one tile, at
    most sixteen, each with the view (a device tensor, or (tensor, byte offset)) its blob was fetched
    into; a global expert id maps to its index here, the kernel's local slot."""

    def __init__(self, expert_ids, views):
        expert_ids = [int(e) for e in expert_ids]
        if not expert_ids:
            raise PrefillGroupedRoutedMoEError("tile binding must include at least one expert")
        if len(expert_ids) > 16:
            raise PrefillGroupedRoutedMoEError("tile binding has %d experts; maximum is 16" % len(expert_ids))
        if len(expert_ids) != len(views):
            raise PrefillGroupedRoutedMoEError("expertIDs.count %d != views.count %d" % (len(expert_ids), len(views)))
        seen = set()
        for e in expert_ids:
            if e < 0:
                raise PrefillGroupedRoutedMoEError("expert id %d must be non-negative" % e)
            if e in seen:
                raise PrefillGroupedRoutedMoEError("duplicate expert id %d in tile binding" % e)
            seen.add(e)
        self.expert_ids, self.views = expert_ids, list(views)

    def local_slot(self, expert):
        return self.expert_ids.index(int(expert)) if int(expert) in self.expert_ids else None

    def pointers(self):
        out = []
        for v in self.views:
            t, off = v if isinstance(v, tuple) else (v, 0)
            out.append(t.data_ptr() + int(off))
        return out

    @staticmethod
    def expert_ids_for_tile(tile_index, groups, tiles):
        """expertIDs(forTile:routes:): groups / tiles are the host copies of a grouping's records
        (rows of (expert, pair_start, pair_count) and (group_start, group_count, pair_start, pair_count))."""
        if not 0 <= tile_index < len(tiles):
            raise PrefillGroupedRoutedMoEError("tile index %d is out of range" % tile_index)
        group_start, group_count = int(tiles[tile_index][0]), int(tiles[tile_index][1])
        if not 0 < group_count <= 16:
            raise PrefillGroupedRoutedMoEError("tile has %d live experts; expected 1...16" % group_count)
        if group_start < 0 or group_start + group_count > len(groups):
            raise PrefillGroupedRoutedMoEError("tile group range %d..<%d exceeds %d"
                                               % (group_start, group_start + group_count, len(groups)))
        return [int(groups[g][0]) for g in range(group_start, group_start + group_count)]

    def validate_covers_pairs(self, pair_experts, pair_start, pair_count):
        """validateCoversPairs: pair_experts = the expert of every sorted pair (host sequence)."""
        if pair_start < 0 or pair_count < 0 or pair_start + pair_count > len(pair_experts):
            raise PrefillGroupedRoutedMoEError("pair range %d..<%d exceeds %d"
                                               % (pair_start, pair_start + pair_count, len(pair_experts)))
        for e in pair_experts[pair_start:pair_start + pair_count]:
            if self.local_slot(e) is None:
                raise PrefillGroupedRoutedMoEError("route expert %d is not bound in tile" % int(e))


def prefill_streamed_params(pair_start, pair_count, d, routed_intermediate, top_k, hidden_stride_elements, binding,
                            offsets):
    """PrefillGroupedRoutedMoEStreamedParams.init (PrefillGroupedRoutedMoE.swift:139-183)."""
    p = _lib.PrefillStreamedParams()
    p.pair_start, p.pair_count, p.d, p.routed_intermediate = pair_start, pair_count, d, routed_intermediate
    p.top_k, p.hidden_stride_elements, p.live_expert_count = top_k, hidden_stride_elements, len(binding.expert_ids)
    for i in range(16):
        p.local_expert[i] = binding.expert_ids[i] if i < len(binding.expert_ids) else 0xFFFFFFFF
    p.gate_w_off, p.gate_s_off, p.gate_b_off = offsets.gate_w, offsets.gate_s, offsets.gate_b
    p.up_w_off, p.up_s_off, p.up_b_off = offsets.up_w, offsets.up_s, offsets.up_b
    p.down_w_off, p.down_s_off, p.down_b_off = offsets.down_w, offsets.down_s, offsets.down_b
    return p


class MPPPrefillInt4QMM:
    """MPPPrefillInt4QMM.encode (MPPPrefillInt4QMM.swift:63-128): y[m, n] = x[m, k] . W[n, k]^T on the
    matrix cores for one affine 4/8-bit matrix."""
    tile_k = 64

    def __init__(self, ctx, weight_bits=4):
        if weight_bits not in (4, 8):
            raise _lib.NvmaiError(-2, "MPPPrefillInt4QMM(weight_bits)")
        self.ctx, self.bits = ctx, weight_bits

    def encode(self, weights, scales, biases, x, n, k, y=None):
        x2 = x.reshape(-1, x.shape[-1])
        m = x2.shape[0]
        if y is None:
            y = torch.empty((m, n), dtype=self.ctx.dtype, device=x.device)
        check(lib.nvmai_hip_affine_qmm(self.ctx.handle, _stream(), _ptr(weights), _ptr(scales), _ptr(biases), self.bits,
                                       _ptr(x2), x2.stride(0), _ptr(y), y.stride(0), m, n, k), "affine_qmm")
        return y


class PrefillMoE:
    """PrefillMoE.encodeReduceTokenMajor (PrefillMoE.swift:11-40)."""

    def __init__(self, ctx):
        self.ctx = ctx

    def encode_reduce_token_major(self, route_partials, route_weights, query_count, top_k, d, h2=None):
        if h2 is None:
            h2 = torch.empty((query_count, d), dtype=self.ctx.dtype, device=route_partials.device)
        check(lib.nvmai_hip_prefill_moe_reduce_token_major(self.ctx.handle, _stream(), _ptr(route_partials),
                                                           _ptr(route_weights), _ptr(h2), h2.stride(0), query_count,
                                                           top_k, d), "prefill_moe_reduce_token_major")
        return h2


def kv_row_layout(elements, bits):
    """KVCacheManager.rowLayout (KVCacheManager.swift:437-446) -> (stride, value_bytes)."""
    s, v = C.c_uint32(), C.c_uint32()
    check(lib.nvmai_kv_row_layout(elements, bits, C.byref(s), C.byref(v)), "kv_row_layout")
    return s.value, v.value


class KVCache:
    """One layer's K or V rows for `batch` sequences: the part of KVCacheManager
    (KVCacheManager.swift) the kernels see.  rows[b, p, :] is the row of position p."""

    def __init__(self, batch, max_context, elements, bits, device="cuda"):
        self.bits, self.elements = bits, elements
        self.stride, self.value_bytes = kv_row_layout(elements, bits)
        self.rows = torch.zeros((batch, max_context, self.stride), dtype=torch.uint8, device=device)

    def view(self, batch_index=0, position=0):
        """KVView (KVCacheManager.swift:19-31) starting at `position` of one sequence."""
        v = KvView()
        v.base = self.rows[batch_index, position].data_ptr()
        v.stride, v.value_bytes, v.bits, v.group_size = self.stride, self.value_bytes, self.bits, 64
        return v

    @property
    def batch_stride(self):
        return self.rows.stride(0)


class KVCacheQuantizer:
    """Mirror of KVCacheQuantizer (KVCacheQuantizer.swift:6-50)."""

    def __init__(self, ctx):
        self.ctx = ctx

    def encode(self, source, source_token_stride_elements, destination, token_count, element_count):
        check(lib.nvmai_hip_kv_quantize_affine(self.ctx.handle, _stream(), _ptr(source),
                                               source_token_stride_elements, C.byref(destination), token_count,
                                               element_count), "kv_quantize_affine")


def rope_neox_subdim(ctx, data, rotary_dim, theta, positions=None, position=0):
    """RoPE.encodeNeoxSubdim (RoPE.swift:48) in place on data[tokens, heads, head_dim]."""
    tokens, heads, hd = data.shape
    check(lib.nvmai_hip_rope_neox_subdim(ctx.handle, _stream(), _ptr(data), tokens, heads, hd, rotary_dim,
                                         _ptr(positions), position, theta), "rope_neox_subdim")
    return data


class Attention:
    """Mirror of Attention (Attention.swift): decode attention over a KV cache."""

    def __init__(self, ctx):
        self.ctx = ctx

    @staticmethod
    def split_geometry(num_q_heads, num_kv_heads, seq_len, kv_start, prefer_gqa_swa):
        """Attention.splitGeometry (Attention.swift:148-168)."""
        vals = [C.c_uint32() for _ in range(4)]
        check(lib.nvmai_attention_split_geometry(num_q_heads, num_kv_heads, seq_len, kv_start,
                                                 int(prefer_gqa_swa), *[C.byref(x) for x in vals]),
              "attention_split_geometry")
        return tuple(x.value for x in vals)

    def encode_full(self, q, k_cache, v_cache, head_dim, num_q_heads, num_kv_heads, seq_len, scale=None,
                    kv_start=0, out=None):
        """Attention.encodeFull (Attention.swift:207-239); q [batch, num_q_heads, head_dim]."""
        batch = q.shape[0]
        if out is None:
            out = torch.empty_like(q)
        kview, vview = k_cache.view(), v_cache.view()
        check(lib.nvmai_hip_attention_decode(self.ctx.handle, _stream(), _ptr(q), C.byref(kview), C.byref(vview),
                                             k_cache.batch_stride, _ptr(out), batch, head_dim, num_q_heads,
                                             num_kv_heads, seq_len, kv_start, 0.0 if scale is None else scale),
              "attention_decode")
        return out

    def encode_full_gated(self, q, k_cache, v_cache, gate, head_dim, num_q_heads, num_kv_heads, seq_len, scale=None,
                          kv_start=0, out=None):
        """encode_full followed by Elementwise.encodeSigmoidGateMul(out, gate) in the same launches
        (RealForwardRunner.swift:2257-2276); gate is laid out like q.  Same bits as the two calls."""
        batch = q.shape[0]
        if out is None:
            out = torch.empty_like(q)
        kview, vview = k_cache.view(), v_cache.view()
        check(lib.nvmai_hip_attention_decode_gated(self.ctx.handle, _stream(), _ptr(q), C.byref(kview), C.byref(vview),
                                                   k_cache.batch_stride, _ptr(out), _ptr(gate), gate.stride(0), batch,
                                                   head_dim, num_q_heads, num_kv_heads, seq_len, kv_start,
                                                   0.0 if scale is None else scale),
              "attention_decode_gated")
        return out

    def encode_swa(self, q, k_cache, v_cache, head_dim, num_q_heads, num_kv_heads, seq_len, window, scale=None):
        """Attention.encodeSWA (Attention.swift:170-205): the last `window` positions."""
        return self.encode_full(q, k_cache, v_cache, head_dim, num_q_heads, num_kv_heads, seq_len, scale,
                                kv_start=seq_len - window if seq_len > window else 0)

    def encode_ragged(self, q, k_cache, v_cache, head_dim, num_q_heads, num_kv_heads, seq_lens, max_seq_len,
                      kv_starts=None, scale=None, out=None):
        """One decode query per sequence, each with its own key range: seq_lens / kv_starts are
        uint32 device tensors of one word per sequence."""
        batch = q.shape[0]
        if out is None:
            out = torch.empty_like(q)
        kview, vview = k_cache.view(), v_cache.view()
        check(lib.nvmai_hip_attention_decode_ragged(self.ctx.handle, _stream(), _ptr(q), C.byref(kview),
                                                    C.byref(vview), k_cache.batch_stride, _ptr(out), batch, head_dim,
                                                    num_q_heads, num_kv_heads, _ptr(seq_lens), _ptr(kv_starts),
                                                    max_seq_len, 0.0 if scale is None else scale),
              "attention_decode_ragged")
        return out


class PrefillAttention:
    """Mirror of PrefillAttention (PrefillAttention.swift:70-167), causalTiled path."""

    def __init__(self, ctx):
        self.ctx = ctx

    def encode_causal(self, q, k_view, v_view, out, start_position, query_count, head_dim, num_q_heads,
                      num_kv_heads, kv_valid_count, sliding_window=0, q_token_stride=None, o_token_stride=None,
                      scale=None, kv_ring_capacity=0):
        """q / out: tensors whose row t starts t * token stride elements in; k_view / v_view:
        KvView of the cache rows from position 0."""
        row = num_q_heads * head_dim
        check(lib.nvmai_hip_attention_prefill_causal(
            self.ctx.handle, _stream(), _ptr(q), row if q_token_stride is None else q_token_stride,
            C.byref(k_view), C.byref(v_view), _ptr(out), row if o_token_stride is None else o_token_stride,
            start_position, query_count, kv_valid_count, sliding_window, head_dim, num_q_heads, num_kv_heads,
            kv_ring_capacity, 0.0 if scale is None else scale), "attention_prefill_causal")
        return out


# ---------------------------------------------------------------------------------------------
# logits -> token
# ---------------------------------------------------------------------------------------------
def sampler_seed_for(seed, position):
    """Sampler.seedFor (Sampler.swift:304-325)."""
    return lib.nvmai_sampler_seed_for(seed, position)


class LogitSoftcapSoftmaxTiled:
    """Mirror of LogitSoftcapSoftmaxTiled (LogitOutput.swift:54-141)."""

    def __init__(self, ctx, vocab):
        if vocab <= 0:
            raise _lib.NvmaiError(-1, "LogitSoftcapSoftmaxTiled(vocab)")
        self.ctx, self.vocab = ctx, vocab

    def encode(self, logits, probs=None, softcap=30.0):
        z = logits.reshape(-1, logits.shape[-1])
        if z.shape[1] != self.vocab:
            raise _lib.NvmaiError(-1, "vocab mismatch: built for %d, got %d" % (self.vocab, z.shape[1]))
        if probs is None:
            probs = torch.empty(z.shape, dtype=torch.float16, device=z.device)
        check(lib.nvmai_hip_softmax_tiled(self.ctx.handle, _stream(), _ptr(z), z.stride(0), _ptr(probs),
                                          probs.stride(0), z.shape[0], self.vocab, softcap), "softmax_tiled")
        return probs


def _seed_array(seeds, rows):
    seeds = [seeds] * rows if isinstance(seeds, int) else list(seeds)
    return (C.c_uint64 * rows)(*[s & 0xFFFFFFFFFFFFFFFF for s in seeds])


class SampleTopK64:
    """Mirror of SampleTopK64 (LogitOutput.swift:202-333)."""

    def __init__(self, ctx, vocab):
        if not 0 < vocab <= 262144:
            raise _lib.NvmaiError(-2, "SampleTopK64 unsupported vocabulary %d" % vocab)
        self.ctx, self.vocab = ctx, vocab
        g1 = (vocab + 1023) // 1024
        g2 = (g1 * 64 + 1023) // 1024
        self.scratch_bytes = (g1 * 64 + g2 * 64) * 8        # LogitOutput.swift:236-243

    def encode(self, probs, temperature, top_p, seed, top_k=64, want_top64=False):
        p = probs.reshape(-1, probs.shape[-1])
        rows = p.shape[0]
        out = torch.empty(rows, dtype=torch.int32, device=p.device)
        top = torch.empty((rows, 64, 2), dtype=torch.int32, device=p.device) if want_top64 else None
        check(lib.nvmai_hip_sample_topk64(self.ctx.handle, _stream(), _ptr(p), p.stride(0), rows, self.vocab,
                                          temperature, top_p, _seed_array(seed, rows), top_k, _ptr(out), _ptr(top)),
              "sample_topk64")
        return (out, top) if want_top64 else out


class Sample:
    """Mirror of Sample (LogitOutput.swift:152-199): the generic sampler."""

    def __init__(self, ctx):
        self.ctx = ctx

    def encode(self, probs, temperature=1.0, top_k=0, top_p=1.0, seed=0, position=0):
        """seed and position: one value or one per row.  Greedy at temperature <= 0, the Gumbel-max
        draw when top_k == 0 and top_p is outside (0, 1), else the truncating path."""
        p = probs.reshape(-1, probs.shape[-1])
        rows = p.shape[0]
        out = torch.empty(rows, dtype=torch.int32, device=p.device)
        pos = position if isinstance(position, (list, tuple)) else [position] * rows
        check(lib.nvmai_hip_sample(self.ctx.handle, _stream(), _ptr(p), p.stride(0), rows, p.shape[1], temperature,
                                   top_k, top_p, _seed_array(seed, rows), (C.c_uint32 * rows)(*pos), _ptr(out)),
              "sample")
        return out


def residual_add_rmsnorm(ctx, hidden, delta, weight, out=None, eps=1e-6):
    """Elementwise.encodeResidualAdd + RMSNorm.encodeBF16W in one launch: hidden += delta (in place),
    returns RMSNorm(hidden) * weight.  hidden, delta: [rows, d] activations."""
    h2, d2 = hidden.reshape(-1, hidden.shape[-1]), delta.reshape(-1, delta.shape[-1])
    if out is None:
        out = torch.empty_like(h2)
    check(lib.nvmai_hip_residual_add_rmsnorm(ctx.handle, _stream(), _ptr(h2), h2.stride(0), _ptr(d2), d2.stride(0),
                                             _ptr(weight), _ptr(out), out.stride(0), h2.shape[0], h2.shape[1], eps),
          "residual_add_rmsnorm")
    return out


def affine_gemv_prenorm(ctx, weights, scales, biases, bits, hidden, delta, norm_weight, hidden_out, m, n, y=None,
                        normed_scratch=None, eps=1e-6):
    """hidden_out = round(hidden + delta); y = W . (rmsnorm(hidden_out) * norm_weight): a layer's input norm
    and its input projection in one launch for up to four rows (same bits as the two calls).  delta may
    be None; normed_scratch [rows, n] is only used for shapes without the one-launch form."""
    h2 = hidden.reshape(-1, hidden.shape[-1])
    rows = h2.shape[0]
    if y is None:
        y = torch.empty((rows, m), dtype=ctx.dtype, device=h2.device)
    d2 = None if delta is None else delta.reshape(-1, delta.shape[-1])
    check(lib.nvmai_hip_affine_gemv_prenorm(ctx.handle, _stream(), _ptr(weights), _ptr(scales), _ptr(biases), bits,
                                            _ptr(h2), h2.stride(0), _ptr(d2), 0 if d2 is None else d2.stride(0),
                                            _ptr(norm_weight), eps, _ptr(hidden_out), hidden_out.stride(0),
                                            _ptr(normed_scratch), 0 if normed_scratch is None else normed_scratch.stride(0),
                                            rows, m, n, _ptr(y), y.stride(0)), "affine_gemv_prenorm")
    return y


def affine_gemv_fused(ctx, parts, bits, x, n):
    """GDN.encodeInputProjections / FusedQKVGEMV.encode: parts = [(weights, scales, biases, rows, y), ...],
    y_i = W_i x for the rows of x; one launch when the parts lie back to back in memory."""
    x2 = x.reshape(-1, x.shape[-1])
    arr = (GemvPart * len(parts))()
    for i, (w, s_, b_, rows, y) in enumerate(parts):
        arr[i].weights, arr[i].scales, arr[i].biases = w.data_ptr(), s_.data_ptr(), b_.data_ptr()
        arr[i].rows, arr[i].y, arr[i].y_stride = rows, y.data_ptr(), (y.stride(0) if y.dim() > 1 else rows)
    check(lib.nvmai_hip_affine_gemv_fused(ctx.handle, _stream(), arr, len(parts), bits, _ptr(x2), x2.stride(0),
                                          x2.shape[0], n), "affine_gemv_fused")


class GDN:
    """Mirror of GDN (GDN.swift:13-341), gated-DeltaNet linear attention.  The reference's conv,
    tail-update and q / k norm dispatches are one call here, the delta step and the gated output
    norm another; `rows` tokens per sequence (1 = decode) for `batch` sequences."""

    def __init__(self, ctx, num_k_heads, num_v_heads, key_head_dim, value_head_dim, conv_kernel_size=4):
        self.ctx = ctx
        self.cfg = GdnConfig(num_k_heads, num_v_heads, key_head_dim, value_head_dim, conv_kernel_size)
        self.qkv_dim = 2 * num_k_heads * key_head_dim + num_v_heads * value_head_dim
        self.value_dim = num_v_heads * value_head_dim

    def new_state(self, batch=1, bf16=False):
        """(conv tail [batch, K - 1, C] activations, recurrent state [batch, Hv, Dv, Dk]) zeroed
        (GDNStateManager's buffers)."""
        c = self.cfg
        tail = torch.zeros((batch, c.conv_kernel_size - 1, self.qkv_dim), dtype=self.ctx.dtype, device=self.ctx.device)
        state = torch.zeros((batch, c.num_v_heads, c.value_head_dim, c.key_head_dim),
                            dtype=torch.bfloat16 if bf16 else torch.float32, device=self.ctx.device)
        return tail, state

    def encode_conv_norm(self, qkv_raw, tail, conv_weight, conv_out=None, rows=1):
        """encodeConvDecode / encodeConvPrefill + encodeConvTailUpdate + encodeQKNorm."""
        q2 = qkv_raw.reshape(-1, qkv_raw.shape[-1])
        batch = q2.shape[0] // rows
        if conv_out is None:
            conv_out = torch.empty((q2.shape[0], self.qkv_dim), dtype=self.ctx.dtype, device=q2.device)
        check(lib.nvmai_hip_gdn_conv_norm(self.ctx.handle, _stream(), C.byref(self.cfg), _ptr(q2), q2.stride(0),
                                          _ptr(tail), _ptr(conv_weight), _ptr(conv_out), conv_out.stride(0), rows, batch),
              "gdn_conv_norm")
        return conv_out

    def encode_delta_gated_norm(self, conv_out, a_proj, b_proj, a_log, dt_bias, state, z, norm_weight, out=None, rows=1):
        """encodeDeltaStepDecode / encodeDeltaStepPrefill + encodeGatedNorm."""
        batch = conv_out.shape[0] // rows
        if out is None:
            out = torch.empty((conv_out.shape[0], self.value_dim), dtype=self.ctx.dtype, device=conv_out.device)
        check(lib.nvmai_hip_gdn_delta_gated_norm(self.ctx.handle, _stream(), C.byref(self.cfg), _ptr(conv_out),
                                                 conv_out.stride(0), _ptr(a_proj), _ptr(b_proj), a_proj.stride(0),
                                                 _ptr(a_log), _ptr(dt_bias), _ptr(state),
                                                 int(state.dtype == torch.bfloat16), _ptr(z), z.stride(0),
                                                 _ptr(norm_weight), _ptr(out), out.stride(0), rows, batch),
              "gdn_delta_gated_norm")
        return out


    def encode_decode_step(self, qkv_raw, tail, conv_weight, a_proj, b_proj, a_log, dt_bias, state, z, norm_weight,
                           out=None, conv_scratch=None):
        """One token per sequence: encode_conv_norm + encode_delta_gated_norm in one launch (same bits);
        conv_scratch [batch, C] is only used for shapes without a fused kernel."""
        q2 = qkv_raw.reshape(-1, qkv_raw.shape[-1])
        batch = q2.shape[0]
        if out is None:
            out = torch.empty((batch, self.value_dim), dtype=self.ctx.dtype, device=q2.device)
        check(lib.nvmai_hip_gdn_decode_step(self.ctx.handle, _stream(), C.byref(self.cfg), _ptr(q2), q2.stride(0),
                                            _ptr(tail), _ptr(conv_weight), _ptr(conv_scratch),
                                            0 if conv_scratch is None else conv_scratch.stride(0), _ptr(a_proj),
                                            _ptr(b_proj), a_proj.stride(0), _ptr(a_log), _ptr(dt_bias), _ptr(state),
                                            int(state.dtype == torch.bfloat16), _ptr(z), z.stride(0), _ptr(norm_weight),
                                            _ptr(out), out.stride(0), batch),
              "gdn_decode_step")
        return out


class GenerationConfig:
    """GenerationConfig (Sampler.swift:19-81), the fields the sampler reads; top_k / top_p / seed may be
    None as in the reference (defaults: GenerationDefaults, Sampler.swift:6-11)."""

    def __init__(self, temperature=0.6, top_k=20, top_p=0.95, repetition_penalty=1.0, seed=None):
        self.temperature, self.top_k, self.top_p = temperature, top_k, top_p
        self.repetition_penalty, self.seed = repetition_penalty, seed

    def _c(self):
        c = _CGenerationConfig()
        c.temperature = self.temperature
        c.top_k = 0 if self.top_k is None else self.top_k
        c.top_p = 0.0 if self.top_p is None else self.top_p
        c.repetition_penalty = self.repetition_penalty
        c.seed, c.has_seed = (0, 0) if self.seed is None else (self.seed, 1)
        return c


class Sampler:
    """Mirror of Sampler (Sampler.swift:133-325): logits -> one token id through the repetition
    penalty, softcap + softmax and the tiled or generic sampler.  The penalty history is kept as the
    reference keeps it (a table of distinct ids, seeded from the first call's history, then one id
    per call) and lives on the device as an id list."""
    PATHS = {0: "greedyGPU", 1: "gpuSampled", 2: "hostPenalty"}

    def __init__(self, ctx, vocab=262144, logit_softcap=30.0, sampler_path="tiled"):
        if sampler_path not in ("tiled", "generic"):
            raise ValueError("invalid sampler path %r" % sampler_path)       # GeneratorError.invalidSamplerPath
        self.ctx, self.vocab, self.logit_softcap = ctx, vocab, logit_softcap
        self.sampler_path = 0 if sampler_path == "tiled" else 1
        self.probs = torch.empty(vocab, dtype=torch.float16, device=ctx.device)
        self.reset_penalty_history()

    def reset_penalty_history(self):
        self._seen, self._ids, self._seeded = set(), [], False
        self._ids_dev, self._ids_count = None, 0

    def _fold_history(self, history):
        new = list(history) if not self._seeded else list(history[-1:])
        self._seeded = True
        for i in new:
            if 0 <= i < self.vocab and i not in self._seen:
                self._seen.add(i)
                self._ids.append(i)
        if self._ids_count != len(self._ids):
            self._ids_dev = torch.tensor(self._ids, dtype=torch.int32, device=self.ctx.device)
            self._ids_count = len(self._ids)

    def sample(self, logits, history, config, position, out_token=None):
        """Sampler.sample (Sampler.swift:171-234); logits: activations [vocab], edited in place by the
        penalty.  Returns (token tensor, path name)."""
        if out_token is None:
            out_token = torch.empty(1, dtype=torch.int32, device=logits.device)
        penalty = config.repetition_penalty != 1.0 and len(history) > 0
        if penalty:
            self._fold_history(history)
        path = C.c_int(-1)
        cfg = config._c()
        check(lib.nvmai_hip_sampler_sample(self.ctx.handle, _stream(), _ptr(logits), _ptr(self.probs), self.vocab,
                                           _ptr(self._ids_dev) if penalty else None,
                                           self._ids_count if penalty else 0, C.byref(cfg), position,
                                           self.logit_softcap, self.sampler_path, _ptr(out_token), C.byref(path)),
              "sampler_sample")
        return out_token, self.PATHS[path.value]


def repetition_penalty(ctx, logits, history_ids, penalty, logit_softcap=0.0):
    """Sampler.applyRepetitionPenaltyInPlace (Sampler.swift:259-293) on the device, in place."""
    check(lib.nvmai_hip_repetition_penalty(ctx.handle, _stream(), _ptr(logits), logits.shape[-1], _ptr(history_ids),
                                           history_ids.numel(), penalty, logit_softcap), "repetition_penalty")
    return logits


class RMSNorm:
    """Mirror of RMSNorm (RMSNorm.swift:20-142): x [rows, d] (rows = 1, or heads for the per-head
    calls); weight: BF16 bits as an int16 tensor [d], or None."""

    def __init__(self, ctx):
        self.ctx = ctx

    def _run(self, x, weight, out, eps):
        x2 = x.reshape(-1, x.shape[-1])
        if out is None:
            out = torch.empty_like(x2)
        o2 = out.reshape(-1, out.shape[-1])
        check(lib.nvmai_hip_rmsnorm(self.ctx.handle, _stream(), _ptr(x2), x2.stride(0), _ptr(weight), _ptr(o2),
                                    o2.stride(0), x2.shape[0], x2.shape[1], eps), "rmsnorm")
        return out

    def encode_bf16w(self, x, weight, out=None, eps=1e-6):
        return self._run(x, weight, out, eps)

    def encode_no_scale(self, x, out=None, eps=1e-6):
        return self._run(x, None, out, eps)

    encode_bf16w_per_head = encode_bf16w
    encode_no_scale_per_head = encode_no_scale


class AffineQuantEmbeddingLookup:
    """Mirror of AffineQuantEmbeddingLookup: rows of a 4- or 8-bit affine table as activations."""

    def __init__(self, ctx, weight_bits):
        if weight_bits not in (4, 8):
            raise _lib.NvmaiError(-2, "AffineQuantEmbeddingLookup(weightBits=%d)" % weight_bits)
        self.ctx, self.bits = ctx, weight_bits

    def encode(self, table, scales, biases, token_ids, d, vocab, out_scale=1.0, out=None):
        """token_ids: an int (one row) or an int32 device tensor [n]."""
        single = not torch.is_tensor(token_ids)
        n = 1 if single else token_ids.numel()
        if out is None:
            out = torch.empty((n, d), dtype=self.ctx.dtype, device=table.device)
        check(lib.nvmai_hip_embed_lookup(self.ctx.handle, _stream(), _ptr(table), _ptr(scales), _ptr(biases), self.bits,
                                         None if single else _ptr(token_ids), int(token_ids) if single else 0, n,
                                         _ptr(out), out.stride(0), d, vocab, out_scale), "embed_lookup")
        return out


class LMHeadChain:
    """Mirror of LMHeadChainInt4.encodeGreedyDecode (LMHeadChainInt4.swift:58-130) for 4- and
    8-bit heads: RMSNorm, one logit per vocabulary row, argmax."""

    def __init__(self, ctx, weight_bits=4):
        if weight_bits not in (4, 8):
            raise _lib.NvmaiError(-2, "LMHeadChain(weightBits=%d)" % weight_bits)
        self.ctx, self.bits = ctx, weight_bits

    def encode_greedy_decode(self, hidden, norm_weight, weights, scales, biases, d, vocab, rms_eps=1e-6, out=None):
        h = hidden.reshape(-1, hidden.shape[-1])
        if out is None:
            out = torch.empty(h.shape[0], dtype=torch.int32, device=h.device)
        check(lib.nvmai_hip_lm_head_greedy(self.ctx.handle, _stream(), _ptr(h), h.stride(0), h.shape[0],
                                           _ptr(norm_weight), _ptr(weights), _ptr(scales), _ptr(biases), self.bits,
                                           _ptr(out), d, vocab, rms_eps), "lm_head_greedy")
        return out


class Elementwise:
    """Mirror of Elementwise (Elementwise.swift:28-121) plus silu_mul_fp16 (utility.metal:32-45)."""

    def __init__(self, ctx):
        self.ctx = ctx

    def encode_silu_mul(self, gate, up, out=None):
        if out is None:
            out = torch.empty_like(gate)
        check(lib.nvmai_hip_silu_mul(self.ctx.handle, _stream(), _ptr(gate), _ptr(up), _ptr(out), gate.numel()), "silu_mul")
        return out

    def encode_sigmoid_gate_mul(self, out, gate):
        check(lib.nvmai_hip_sigmoid_gate_mul(self.ctx.handle, _stream(), _ptr(out), _ptr(gate), out.numel()),
              "sigmoid_gate_mul")
        return out

    def encode_sigmoid_scalar_mul(self, y, gate):
        check(lib.nvmai_hip_sigmoid_scalar_mul(self.ctx.handle, _stream(), _ptr(y), _ptr(gate), y.numel()),
              "sigmoid_scalar_mul")
        return y

    def encode_residual_add(self, hidden, delta):
        check(lib.nvmai_hip_residual_add(self.ctx.handle, _stream(), _ptr(hidden), _ptr(delta), hidden.numel()),
              "residual_add")
        return hidden

    def encode_split_q_gate(self, packed, heads, dim):
        q = torch.empty((heads, dim), dtype=packed.dtype, device=packed.device)
        gate = torch.empty_like(q)
        check(lib.nvmai_hip_split_q_gate(self.ctx.handle, _stream(), _ptr(packed), _ptr(q), _ptr(gate), heads, dim),
              "split_q_gate")
        return q, gate

    def encode_concat_rows(self, lhs, rhs):
        rows, dim = lhs.shape
        out = torch.empty((rows, 2 * dim), dtype=lhs.dtype, device=lhs.device)
        check(lib.nvmai_hip_concat_rows(self.ctx.handle, _stream(), _ptr(lhs), _ptr(rhs), _ptr(out), rows, dim),
              "concat_rows")
        return out
