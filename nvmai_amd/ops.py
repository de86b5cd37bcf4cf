"""Host layer over the C ABI: one class or function per reference operator wrapper
(sources/NVMAI/Kernels/...), same argument meaning, errors as exceptions.  Arguments
are torch tensors on the GPU (device memory plumbing); every call only enqueues work
on torch's current stream."""
import ctypes as C

import torch

from . import _lib
from ._lib import ExpertOffsets, MoeLayer, Rows, check, lib

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

    def profile_enable(self, on=True):
        check(lib.nvmai_hip_profile_enable(self.handle, int(on)), "profile_enable")

    def profile_read(self, tag):
        """Summed milliseconds and launch count of one NVMAI_PROF_* tag."""
        ms, n = C.c_double(), C.c_uint32()
        check(lib.nvmai_hip_profile_read(self.handle, tag, C.byref(ms), C.byref(n)), "profile_read")
        return ms.value, n.value

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


def affine_gemv(ctx, weights, scales, biases, bits, x, m, n, out_f32=False):
    """DequantInt4GEMV.encode / DequantInt8GEMV.encode / AffineQuantGEMV.encode:
    y[t] = W x[t] for x [tokens, n]."""
    x2 = x.reshape(-1, x.shape[-1])
    tokens = x2.shape[0]
    y = None if out_f32 else torch.empty((tokens, m), dtype=ctx.dtype, device=x.device)
    yf = torch.empty((tokens, m), dtype=torch.float32, device=x.device) if out_f32 else None
    check(lib.nvmai_hip_affine_gemv(ctx.handle, _stream(), _ptr(weights), _ptr(scales), _ptr(biases), bits,
                                    _ptr(x2), x2.stride(0), tokens, m, n, _ptr(y), _ptr(yf), m),
          "affine_gemv")
    return yf if out_f32 else y


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


def moe_layer_desc(d, f, num_experts, top_k, bits, router, experts, shared_blob=None, shared_gate=None,
                   eff_scale=None, per_expert_scale=None):
    """Fill an nvmai_moe_layer.  experts: uint8 tensor [num_experts, stride] (resident pool)."""
    L = MoeLayer()
    L.d, L.f, L.num_experts, L.top_k, L.bits = d, f, num_experts, top_k, bits
    L.router = router
    L.experts_base, L.expert_stride = experts.data_ptr(), experts.stride(0)
    L.offsets, _ = expert_offsets(d, f, bits)
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
