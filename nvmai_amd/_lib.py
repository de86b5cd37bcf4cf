"""ctypes view of libnvmai_hip.so (the C ABI declared in include/nvmai_hip.h).

The library is the product; there is no fallback.  If it has not been built the
import fails loudly.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnvmai_hip.so")


class NvmaiLibraryMissing(ImportError):
    pass


def load():
    if not os.path.exists(LIB_PATH):
        raise NvmaiLibraryMissing(
            "%s is missing: run `python -m nvmai_amd.build` (hipcc, gfx950) first" % LIB_PATH)
    return C.CDLL(LIB_PATH)


lib = load()

vp, u32, u64, i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32


class Rows(C.Structure):
    """nvmai_rows"""
    _fields_ = [("weights", vp), ("scales", vp), ("biases", vp), ("kind", i32)]


class ExpertOffsets(C.Structure):
    """nvmai_expert_offsets"""
    _fields_ = [(n, u32) for n in ("gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b",
                                   "down_w", "down_s", "down_b")]


class MoeLayer(C.Structure):
    """nvmai_moe_layer"""
    _fields_ = [("d", u32), ("f", u32), ("num_experts", u32), ("top_k", u32), ("bits", u32),
                ("router", Rows), ("experts_base", vp), ("expert_stride", u64),
                ("offsets", ExpertOffsets), ("shared_blob", vp), ("shared_gate", Rows),
                ("eff_scale", vp), ("per_expert_scale", vp)]


class KvView(C.Structure):
    """nvmai_kv_view"""
    _fields_ = [("base", vp), ("stride", u32), ("value_bytes", u32), ("bits", u32), ("group_size", u32)]


class GenerationConfig(C.Structure):
    """nvmai_generation_config"""
    _fields_ = [("temperature", C.c_float), ("top_k", i32), ("top_p", C.c_float), ("repetition_penalty", C.c_float),
                ("seed", u64), ("has_seed", i32)]


class GdnConfig(C.Structure):
    """nvmai_gdn_config"""
    _fields_ = [(n, u32) for n in ("num_k_heads", "num_v_heads", "key_head_dim", "value_head_dim", "conv_kernel_size")]


class GemvPart(C.Structure):
    """nvmai_gemv_part"""
    _fields_ = [("weights", vp), ("scales", vp), ("biases", vp), ("rows", u32), ("y", vp), ("y_stride", u32)]


class PrefillStreamedParams(C.Structure):
    """nvmai_prefill_streamed_params == PrefillGroupedRoutedMoEStreamedParams, 128 bytes"""
    _fields_ = ([(n, u32) for n in ("pair_start", "pair_count", "d", "routed_intermediate", "top_k",
                                    "hidden_stride_elements", "live_expert_count")] +
                [("local_expert", u32 * 16)] +
                [(n, u32) for n in ("gate_w_off", "gate_s_off", "gate_b_off", "up_w_off", "up_s_off", "up_b_off",
                                    "down_w_off", "down_s_off", "down_b_off")])


class PrefillGrouping(C.Structure):
    """nvmai_prefill_grouping"""
    _fields_ = [(n, vp) for n in ("sorted_pairs", "expert_offsets", "expert_counts", "groups", "tiles", "info")]


# name -> argtypes (every function returns int unless listed in _OTHER)
SIGNATURES = {
    "nvmai_hip_ctx_create": [C.c_int, C.c_int, C.POINTER(vp)],
    "nvmai_hip_ctx_reserve": [vp, C.c_size_t],
    "nvmai_hip_profile_enable": [vp, C.c_int],
    "nvmai_hip_profile_read": [vp, C.c_int, C.POINTER(C.c_double), C.POINTER(u32)],
    "nvmai_hip_read_probe": [vp, vp, vp, u64, vp],
    "nvmai_expert_offsets_for": [u32, u32, u32, C.POINTER(ExpertOffsets), C.POINTER(u64)],
    "nvmai_hip_quantize_affine": [vp, vp, vp, C.c_int, u32, u32, u32, vp, vp, vp],
    "nvmai_hip_dequantize_affine": [vp, vp, vp, vp, vp, u64, u32, vp, vp],
    "nvmai_hip_affine_gemv": [vp, vp, vp, vp, vp, u32, vp, u32, u32, u32, u32, vp, vp, u32],
    "nvmai_hip_moe_router_topk": [vp, vp, C.POINTER(Rows), vp, u32, u32, vp, vp, u32, u32, u32,
                                  vp, vp, vp],
    "nvmai_hip_moe_phase1_gate_up_act": [vp, vp, C.POINTER(vp), C.POINTER(ExpertOffsets), u32, vp,
                                         vp, u32, u32, u32],
    "nvmai_hip_moe_phase1_gate_up_act_subset": [vp, vp, C.POINTER(vp), C.POINTER(ExpertOffsets),
                                                u32, vp, vp, u32, u32, u32, vp, u32],
    "nvmai_hip_moe_phase2_down_reduce": [vp, vp, C.POINTER(vp), C.POINTER(ExpertOffsets), u32, vp,
                                         vp, vp, vp, u32, u32, u32],
    "nvmai_hip_shared_expert": [vp, vp, vp, C.POINTER(ExpertOffsets), u32, C.POINTER(Rows), vp,
                                u32, u32, vp, u32, u32, u32],
    "nvmai_hip_moe_decode_layer": [vp, vp, C.POINTER(MoeLayer), vp, u32, u32, vp, u32, vp, vp, vp],
    "nvmai_hip_moe_decode_layer_prenorm": [vp, vp, C.POINTER(MoeLayer), vp, u32, vp, u32, vp, C.c_float, vp, u32, vp, u32,
                                           u32, vp, u32, vp, vp, vp],
    "nvmai_hip_moe_decode_layer_norms": [vp, vp, C.POINTER(MoeLayer), vp, u32, vp, u32, vp, C.c_float, vp, u32, vp, u32,
                                         u32, vp, u32, vp, vp, vp, vp, vp, u32],
    "nvmai_hip_moe_decode_layer_noalloc": [vp, vp, C.POINTER(MoeLayer), vp, u32, u32, vp, u32, vp, vp, vp],
    "nvmai_kv_row_layout": [u32, u32, C.POINTER(u32), C.POINTER(u32)],
    "nvmai_hip_kv_quantize_affine": [vp, vp, vp, u32, C.POINTER(KvView), u32, u32],
    "nvmai_hip_rope_neox_subdim": [vp, vp, vp, u32, u32, u32, u32, vp, u32, C.c_float],
    "nvmai_hip_attention_decode": [vp, vp, vp, C.POINTER(KvView), C.POINTER(KvView), u64, vp, u32, u32, u32,
                                   u32, u32, u32, C.c_float],
    "nvmai_hip_attention_decode_gated": [vp, vp, vp, C.POINTER(KvView), C.POINTER(KvView), u64, vp, vp, u32, u32, u32,
                                         u32, u32, u32, u32, C.c_float],
    "nvmai_hip_attention_decode_ragged": [vp, vp, vp, C.POINTER(KvView), C.POINTER(KvView), u64, vp, u32, u32, u32,
                                          u32, vp, vp, u32, C.c_float],
    "nvmai_hip_attention_prefill_causal": [vp, vp, vp, u32, C.POINTER(KvView), C.POINTER(KvView), vp, u32, u32, u32,
                                           u32, u32, u32, u32, u32, u32, C.c_float],
    "nvmai_attention_split_geometry": [u32, u32, u32, u32, C.c_int, C.POINTER(u32), C.POINTER(u32),
                                       C.POINTER(u32), C.POINTER(u32)],
    "nvmai_hip_softmax_tiled": [vp, vp, vp, u32, vp, u32, u32, u32, C.c_float],
    "nvmai_hip_sample_topk64": [vp, vp, vp, u32, u32, u32, C.c_float, C.c_float, C.POINTER(u64), u32, vp, vp],
    "nvmai_prefill_grouping_check": [C.c_int64] * 5 + [C.c_int, C.c_int64],
    "nvmai_hip_prefill_make_pairs": [vp, vp, vp, vp, u32, u32, vp],
    "nvmai_hip_prefill_group_pairs": [vp, vp, vp, u64, u32, u32, u32, u32, vp, u64, C.POINTER(PrefillGrouping)],
    "nvmai_hip_prefill_group_routes": [vp, vp, vp, vp, u32, u32, u32, u32, vp, u64, C.POINTER(PrefillGrouping)],
    "nvmai_hip_prefill_grouped_moe": [vp, vp, vp, u64, C.POINTER(ExpertOffsets), u32, u32, u32, u32, vp, u32,
                                      u32, u32, C.POINTER(PrefillGrouping), vp, vp],
    "nvmai_hip_prefill_grouped_moe_streamed": [vp, vp, C.POINTER(PrefillStreamedParams), C.POINTER(vp), u32, vp, vp, u64,
                                               vp, vp, vp],
    "nvmai_hip_affine_qmm": [vp, vp, vp, vp, vp, u32, vp, u32, vp, u32, u32, u32, u32],
    "nvmai_hip_prefill_moe_reduce_token_major": [vp, vp, vp, vp, vp, u32, u32, u32, u32],
    "nvmai_hip_silu_mul": [vp, vp, vp, vp, vp, u32],
    "nvmai_hip_sigmoid_gate_mul": [vp, vp, vp, vp, u32],
    "nvmai_hip_sigmoid_scalar_mul": [vp, vp, vp, vp, u32],
    "nvmai_hip_residual_add": [vp, vp, vp, vp, u32],
    "nvmai_hip_split_q_gate": [vp, vp, vp, vp, vp, u32, u32],
    "nvmai_hip_concat_rows": [vp, vp, vp, vp, vp, u32, u32],
    "nvmai_hip_rmsnorm": [vp, vp, vp, u32, vp, vp, u32, u32, u32, C.c_float],
    "nvmai_hip_embed_lookup": [vp, vp, vp, vp, vp, u32, vp, u32, u32, vp, u32, u32, u32, C.c_float],
    "nvmai_hip_lm_head_greedy": [vp, vp, vp, u32, u32, vp, vp, vp, vp, u32, vp, u32, u32, C.c_float],
    "nvmai_hip_repetition_penalty": [vp, vp, vp, u32, vp, u32, C.c_float, C.c_float],
    "nvmai_hip_sampler_sample": [vp, vp, vp, vp, u32, vp, u32, C.POINTER(GenerationConfig), C.c_int64, C.c_float,
                                 C.c_int, vp, C.POINTER(C.c_int)],
    "nvmai_hip_residual_add_rmsnorm": [vp, vp, vp, u32, vp, u32, vp, vp, u32, u32, u32, C.c_float],
    "nvmai_hip_affine_gemv_prenorm": [vp, vp, vp, vp, vp, u32, vp, u32, vp, u32, vp, C.c_float, vp, u32, vp, u32, u32, u32, u32,
                                      vp, u32],
    "nvmai_hip_attn_qkv_epilogue": [vp, vp, vp, u32, C.c_int, vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32,
                                    C.c_int, vp, u32, C.c_float, C.c_float],
    "nvmai_hip_attn_qkv_epilogue_kv": [vp, vp, vp, u32, C.c_int, vp, vp, vp, vp, vp, vp, u32, C.POINTER(KvView),
                                       C.POINTER(KvView), u32, u32, u32, u32, u32, C.c_int, vp, u32, C.c_float, C.c_float],
    "nvmai_hip_gdn_conv_norm": [vp, vp, C.POINTER(GdnConfig), vp, u32, vp, vp, vp, u32, u32, u32],
    "nvmai_hip_gdn_decode_step": [vp, vp, C.POINTER(GdnConfig), vp, u32, vp, vp, vp, u32, vp, vp, u32, vp, vp, vp, C.c_int,
                                  vp, u32, vp, vp, u32, u32],
    "nvmai_hip_gdn_delta_gated_norm": [vp, vp, C.POINTER(GdnConfig), vp, u32, vp, vp, u32, vp, vp, vp, C.c_int, vp, u32,
                                       vp, vp, u32, u32, u32],
    "nvmai_hip_affine_gemv_fused": [vp, vp, C.POINTER(GemvPart), u32, u32, vp, u32, u32, u32],
    "nvmai_hip_sample": [vp, vp, vp, u32, u32, u32, C.c_float, u32, C.c_float, C.POINTER(u64), C.POINTER(u32), vp],
}
_OTHER = {
    "nvmai_hip_ctx_destroy": (None, [vp]),
    "nvmai_hip_ctx_workspace_bytes": (C.c_size_t, [vp]),
    "nvmai_hip_moe_decode_layer_noalloc_scratch_bytes": (C.c_size_t, []),
    "nvmai_hip_status_string": (C.c_char_p, [C.c_int]),
    "nvmai_int4_affine_gemv": (None, [vp, vp, vp, vp, C.c_size_t, C.c_size_t, vp]),
    "nvmai_sampler_seed_for": (u64, [u64, C.c_int64]),
}


def _declare():
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = args
    for name, (res, args) in _OTHER.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args


_declare()

STATUS = {0: "ok", -1: "invalid_arg", -2: "unsupported", -3: "alignment", -4: "scratch",
          -5: "hip", -6: "no_device"}


class NvmaiError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        self.name = STATUS.get(status, str(status))
        super().__init__("%s: %s" % (where, lib.nvmai_hip_status_string(status).decode()))


def check(status, where):
    if status != 0:
        raise NvmaiError(status, where)
