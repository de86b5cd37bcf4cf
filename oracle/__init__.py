"""ctypes binding of the CPU oracle -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this package.  The shipped library (nvmai_amd) never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnvmai_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libnvmai_ref.so")


def build():
    """Compile the oracle (and the reference C kernel when its tree is mounted)."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


lib = _load()


def build_native(path):
    """The same two C files at -O3 -march=native (still -ffp-contract=off, no fast-math: the same
    results, only faster) for the timed cpu_baseline legs of bench.py; compiled where it runs,
    because a binary made for another CPU's instruction set may not.  Returns a CDLL, or None
    when there is no compiler."""
    cmd = ["gcc", "-O3", "-march=native", "-std=c11", "-ffp-contract=off", "-fPIC", "-shared", "-o", path,
           os.path.join(_HERE, "nvmai_oracle.c"), os.path.join(_HERE, "nvmai_oracle_bench.c"), "-lm", "-lpthread"]
    try:
        subprocess.run(cmd, check=True, capture_output=True)
        return C.CDLL(path)
    except (OSError, subprocess.CalledProcessError):
        return None

u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
size_t = C.c_size_t


def _sig(name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_sig("orc_bf16_bits", C.c_uint16, C.c_float)
_sig("orc_bf16_to_float", C.c_float, C.c_uint16)
_sig("orc_f16_bits", C.c_uint16, C.c_float)
_sig("orc_f16_to_float", C.c_float, C.c_uint16)
_sig("orc_seedtree_key", C.c_uint64, C.c_uint64, C.c_char_p)
_sig("orc_quantize_affine", None, f32p, size_t, size_t, C.c_int, u8p, u16p, u16p)
_sig("orc_dequantize_affine", None, u8p, u16p, u16p, size_t, size_t, C.c_int, f32p)
_sig("orc_unpack_codes", None, u8p, size_t, C.c_int, u8p)
_sig("orc_expert_offsets", None, size_t, size_t, C.c_int, u32p)
_sig("orc_pack_expert", None, f32p, f32p, f32p, size_t, size_t, C.c_int, u8p)
_sig("orc_int4_affine_gemv", None, u8p, u16p, u16p, f32p, size_t, size_t, f32p)
_sig("orc_affine_gemv", None, u8p, u16p, u16p, f32p, size_t, size_t, C.c_int, f32p)
_sig("orc_affine_gemv_unfactored", None, u8p, u16p, u16p, f32p, size_t, size_t, C.c_int, f32p)
_sig("orc_expert_ffn_accumulate", None, u8p, u32p, C.c_int, f32p, size_t, size_t,
     C.c_float, f32p, f32p)
_sig("orc_router_logits", None, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, f32p,
     C.c_void_p, size_t, size_t, f32p)
_sig("orc_router_topk", None, f32p, size_t, size_t, C.c_void_p, u32p, u16p)
_sig("orc_make_pairs", None, u32p, u16p, size_t, size_t, u32p)
_sig("orc_kv_row_layout", None, size_t, C.c_int, C.POINTER(size_t), C.POINTER(size_t))
_sig("orc_kv_quantize", None, f32p, size_t, size_t, size_t, C.c_int, u8p, size_t, size_t)
_sig("orc_kv_dequant_row", None, u8p, size_t, C.c_int, size_t, f32p)
_sig("orc_rope_neox_subdim", None, f32p, size_t, size_t, size_t, size_t, u32p, C.c_float)
_sig("orc_split_geometry", None, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int,
     C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
     C.POINTER(C.c_uint32))
_sig("orc_attention_decode", None, f32p, C.c_void_p, C.c_void_p, C.c_int, size_t, size_t,
     size_t, size_t, size_t, size_t, size_t, C.c_float, size_t, size_t, f32p)
_sig("orc_softmax_f16", None, f32p, size_t, C.c_float, u16p)
_sig("orc_softmax_tiled_f16", None, f32p, size_t, C.c_float, u16p)
_sig("orc_xorshift64star", C.c_uint64, C.POINTER(C.c_uint64))
_sig("orc_uniform01", C.c_float, C.POINTER(C.c_uint64))
_sig("orc_seed_for", C.c_uint64, C.c_uint64, C.c_int64)
_sig("orc_sample_generic", C.c_uint32, u16p, size_t, C.c_float, C.c_uint32, C.c_float,
     C.c_uint64)
_sig("orc_sample_gumbel", C.c_uint32, u16p, size_t, C.c_float, C.c_uint64, C.c_uint32)
_sig("orc_sample", C.c_uint32, u16p, size_t, C.c_float, C.c_uint32, C.c_float, C.c_uint64, C.c_uint32)
_sig("orc_gumbel_for", C.c_float, C.c_uint64, C.c_uint32, C.c_uint32)
_sig("orc_sample_topk64", C.c_uint32, u16p, size_t, C.c_float, C.c_float, C.c_uint64,
     C.c_uint32, C.c_void_p, C.c_void_p)
_sig("orc_repetition_penalty", None, f32p, C.c_int, size_t, np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS"),
     size_t, C.c_float, C.c_float)
_sig("orc_sampler_route", C.c_int, C.c_int, C.c_float, C.c_int)
_sig("orc_sampler_sample", C.c_uint32, f32p, size_t, C.c_float, C.c_int, C.c_float, C.c_int, C.c_float,
     C.c_uint64, C.c_int64, u16p)
_sig("orc_gdn_step", None, f32p, f32p, f32p, f32p, u16p, u16p, u16p, u16p, size_t, size_t, size_t, size_t, size_t,
     C.c_int, f32p, f32p, f32p)
_sig("orc_rel_error", C.c_float, f32p, f32p, size_t)
_sig("orc_rmsnorm", None, f32p, size_t, C.c_void_p, size_t, size_t, C.c_float, f32p, size_t)
_sig("orc_elementwise", None, C.c_int, f32p, f32p, size_t, f32p)
_sig("orc_embed_lookup", None, u8p, u16p, u16p, C.c_int, C.c_uint32, size_t, size_t, C.c_float, f32p)
_sig("orc_lm_head_greedy", C.c_uint32, f32p, C.c_void_p, u8p, u16p, u16p, C.c_int, size_t, size_t,
     C.c_float, C.c_int, C.c_void_p)

GROUP = 64


# ---------------------------------------------------------------- conversions
def bf16_bits(a):
    """float32 array -> bf16 bit patterns (Quantization.swift:17-23)."""
    a = np.ascontiguousarray(a, np.float32)
    bits = a.view(np.uint32)
    lsb = (bits >> 16) & 1
    return ((bits + np.uint32(0x7FFF) + lsb) >> 16).astype(np.uint16)


def bf16_to_float(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_bf16(a):
    return bf16_to_float(bf16_bits(a))


def f16_bits(a):
    return np.ascontiguousarray(a, np.float32).astype(np.float16).view(np.uint16)


def f16_to_float(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


# ---------------------------------------------------------------- PRNGs
class SplitMix64:
    """SplitMix64.swift:11-23."""
    MASK = (1 << 64) - 1

    def __init__(self, seed):
        self.state = seed & self.MASK

    def next(self):
        self.state = (self.state + 0x9E3779B97F4A7C15) & self.MASK
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & self.MASK
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & self.MASK
        return z ^ (z >> 31)

    def uniform(self, lo, hi):
        u = np.float32(self.next() >> 40) / np.float32(16777216.0)
        return np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u

    def uniform_array(self, n, lo, hi):
        return np.array([self.uniform(lo, hi) for _ in range(n)], np.float32)


def seed_tree(root, label):
    """SeedTree.swift:12-19."""
    return SplitMix64(lib.orc_seedtree_key(root, label.encode()))


class Lcg:
    """CPUExpertFFNTests.swift:18-23."""
    MASK = (1 << 64) - 1

    def __init__(self, seed, inc=1442695040888963407):
        self.state, self.inc = seed, inc

    def next(self):
        self.state = (self.state * 6364136223846793005 + self.inc) & self.MASK
        v = (self.state >> 33) & 0xFFFFFFFF
        if v >= 1 << 31:
            v -= 1 << 32
        return np.float32(v) / np.float32(2147483647)

    def array(self, n):
        return np.array([self.next() for _ in range(n)], np.float32)


# ---------------------------------------------------------------- quantizer
def quantize_affine(w, bits):
    w = np.ascontiguousarray(w, np.float32)
    if w.ndim == 1:
        w = w[None, :]
    rows, n = w.shape
    packed = np.zeros((rows, n * bits // 8), np.uint8)
    scales = np.zeros((rows, n // GROUP), np.uint16)
    biases = np.zeros((rows, n // GROUP), np.uint16)
    lib.orc_quantize_affine(w, rows, n, bits, packed, scales, biases)
    return packed, scales, biases


def dequantize_affine(packed, scales, biases, n, bits):
    rows = packed.shape[0]
    out = np.zeros((rows, n), np.float32)
    lib.orc_dequantize_affine(packed, scales, biases, rows, n, bits, out)
    return out


def unpack_codes(packed, bits):
    packed = np.ascontiguousarray(packed, np.uint8).reshape(-1)
    count = packed.size * 8 // bits
    codes = np.zeros(count, np.uint8)
    lib.orc_unpack_codes(packed, count, bits, codes)
    return codes


def expert_offsets(d, f, bits):
    out = np.zeros(10, np.uint32)
    lib.orc_expert_offsets(d, f, bits, out)
    return out


def pack_expert(gate, up, down, bits):
    f, d = gate.shape
    off = expert_offsets(d, f, bits)
    blob = np.zeros(int(off[9]), np.uint8)
    lib.orc_pack_expert(np.ascontiguousarray(gate, np.float32),
                        np.ascontiguousarray(up, np.float32),
                        np.ascontiguousarray(down, np.float32), d, f, bits, blob)
    return blob


def affine_gemv(packed, scales, biases, x, bits, unfactored=False):
    rows = packed.shape[0]
    n = packed.shape[1] * 8 // bits
    out = np.zeros(rows, np.float32)
    fn = lib.orc_affine_gemv_unfactored if unfactored else lib.orc_affine_gemv
    fn(packed, scales, biases, np.ascontiguousarray(x, np.float32), rows, n, bits, out)
    return out


def expert_ffn_accumulate(blob, bits, x, d, f, route_w, out):
    off = expert_offsets(d, f, bits)
    scratch = np.zeros(2 * f + d, np.float32)
    lib.orc_expert_ffn_accumulate(blob, off, bits, np.ascontiguousarray(x, np.float32),
                                  d, f, route_w, scratch, out)
    return out


# ---------------------------------------------------------------- router
def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def router_logits(kind, weights, scales, biases, x, eff_scale=None):
    """kind 4/8: affine rows; 16: dense bf16 bit patterns [E, d]."""
    x = np.ascontiguousarray(x, np.float32)
    d = x.shape[-1]
    ne = weights.shape[0]
    logits = np.zeros(ne, np.float32)
    lib.orc_router_logits(_ptr(weights), _ptr(scales), _ptr(biases), kind, x,
                          _ptr(eff_scale), ne, d, logits)
    return logits


def router_topk(logits, k, per_expert_scale=None):
    logits = np.ascontiguousarray(logits, np.float32)
    idx = np.zeros(k, np.uint32)
    w = np.zeros(k, np.uint16)
    lib.orc_router_topk(logits, logits.size, k, _ptr(per_expert_scale), idx, w)
    return idx, w


class OrcMoeLayer(C.Structure):
    _fields_ = [("d", size_t), ("f", size_t), ("num_experts", size_t), ("top_k", size_t),
                ("bits", C.c_int), ("router_kind", C.c_int),
                ("router_w", C.c_void_p), ("router_s", C.c_void_p), ("router_b", C.c_void_p),
                ("experts", C.POINTER(C.c_void_p)), ("shared_blob", C.c_void_p),
                ("gate_kind", C.c_int),
                ("gate_w", C.c_void_p), ("gate_s", C.c_void_p), ("gate_b", C.c_void_p)]


lib.orc_moe_layer_forward.restype = None
lib.orc_moe_layer_forward.argtypes = [C.POINTER(OrcMoeLayer), f32p, size_t, u32p, u16p, f32p]


def _moe_layer_struct(d, f, top_k, bits, router, expert_blobs, shared_blob, gate):
    ne = expert_blobs.shape[0]
    L = OrcMoeLayer()
    L.d, L.f, L.num_experts, L.top_k, L.bits = d, f, ne, top_k, bits
    L.router_kind = router[0]
    L.router_w, L.router_s, L.router_b = _ptr(router[1]), _ptr(router[2]), _ptr(router[3])
    ptrs = (C.c_void_p * ne)(*[expert_blobs[e].ctypes.data for e in range(ne)])
    L.experts = ptrs
    L.shared_blob = _ptr(shared_blob)
    if gate is not None:
        L.gate_kind = gate[0]
        L.gate_w, L.gate_s, L.gate_b = _ptr(gate[1]), _ptr(gate[2]), _ptr(gate[3])
    L._keep = (ptrs, router, expert_blobs, shared_blob, gate)
    return L


def moe_layer_forward(x, d, f, top_k, bits, router, expert_blobs, shared_blob=None, gate=None):
    """router / gate: (kind, weights, scales, biases).  expert_blobs: uint8 [E, stride].
    Returns (idx [T,k] u32, w [T,k] f16 bits, y [T,d] f32)."""
    x = np.ascontiguousarray(x, np.float32).reshape(-1, d)
    tokens = x.shape[0]
    L = _moe_layer_struct(d, f, top_k, bits, router, expert_blobs, shared_blob, gate)
    idx = np.zeros((tokens, top_k), np.uint32)
    w = np.zeros((tokens, top_k), np.uint16)
    y = np.zeros((tokens, d), np.float32)
    lib.orc_moe_layer_forward(C.byref(L), x, tokens, idx, w, y)
    return idx, w, y


# ---------------------------------------------------------------- timed legs (bench.py's cpu_baseline only)
def host_cpu():
    """(model string, threads this process may use, capped at the GPU box's CPU share of 16)."""
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    return model, max(1, min(16, n))


_timing = {}


def timing_lib():
    """(CDLL, flags string): the oracle rebuilt at -O3 -march=native in a temporary file, or the
    -O2 library that ships with the tree when no compiler is at hand."""
    if "lib" not in _timing:
        import tempfile
        path = os.path.join(tempfile.gettempdir(), "libnvmai_oracle_native_%d.so" % os.getpid())
        native = build_native(path)
        _timing["lib"] = (native, "-O3 -march=native -ffp-contract=off") if native is not None else \
            (lib, "-O2 -ffp-contract=off (prebuilt)")
    return _timing["lib"]


def time_moe_layer(x, d, f, top_k, bits, router, expert_blobs, shared_blob, gate, threads, warmup=1, reps=5):
    """Median seconds of one decode step of the layer over the tokens of x, tokens shared out over
    `threads` threads; also returns the routing indices of the step."""
    clib, _ = timing_lib()
    x = np.ascontiguousarray(x, np.float32).reshape(-1, d)
    tokens = x.shape[0]
    L = _moe_layer_struct(d, f, top_k, bits, router, expert_blobs, shared_blob, gate)
    idx = np.zeros((tokens, top_k), np.uint32)
    w = np.zeros((tokens, top_k), np.uint16)
    y = np.zeros((tokens, d), np.float32)
    fn = clib.orc_time_moe_layer
    fn.restype = C.c_double
    fn.argtypes = [C.POINTER(OrcMoeLayer), f32p, size_t, C.c_int, C.c_int, C.c_int, u32p, u16p, f32p]
    return fn(C.byref(L), x, tokens, threads, warmup, reps, idx, w, y), idx


def time_attention(q, k_rows, v_rows, bits, nq, nkv, hd, seq, scale, threads, warmup=1, reps=5):
    """q [B, nq, hd] float32; k_rows, v_rows uint8 [B, seq, stride]: median seconds of one decode
    attention call over the B sequences, sequences shared out over the threads."""
    clib, _ = timing_lib()
    q = np.ascontiguousarray(q, np.float32)
    k_rows, v_rows = np.ascontiguousarray(k_rows), np.ascontiguousarray(v_rows)
    b = q.shape[0]
    stride, vb = kv_row_layout(nkv * hd, bits)
    out = np.zeros_like(q)
    fn = clib.orc_time_attention
    fn.restype = C.c_double
    fn.argtypes = [f32p, u8p, u8p, size_t, size_t, C.c_int, size_t, size_t, size_t, size_t, size_t, size_t,
                   C.c_float, C.c_int, C.c_int, C.c_int, f32p]
    return fn(q, k_rows.reshape(-1), v_rows.reshape(-1), k_rows.strides[0], b, bits, stride, vb, nq, nkv, hd, seq,
              scale, threads, warmup, reps, out)


def time_prefill_moe(expert_blobs, bits, x, d, f, idx, w_f16, threads, warmup=1, reps=5):
    clib, _ = timing_lib()
    x = np.ascontiguousarray(x, np.float32).reshape(-1, d)
    tokens = x.shape[0]
    idx = np.ascontiguousarray(idx, np.uint32)
    k = idx.shape[1]
    ne = expert_blobs.shape[0]
    ptrs = (C.c_void_p * ne)(*[expert_blobs[e].ctypes.data for e in range(ne)])
    h2 = np.zeros((tokens, d), np.float32)
    fn = clib.orc_time_prefill_moe
    fn.restype = C.c_double
    fn.argtypes = [C.POINTER(C.c_void_p), u32p, C.c_int, f32p, size_t, size_t, size_t, size_t, u32p, u16p,
                   C.c_int, C.c_int, C.c_int, f32p]
    return fn(ptrs, expert_offsets(d, f, bits), bits, x, tokens, d, f, k, idx,
              np.ascontiguousarray(w_f16, np.uint16), threads, warmup, reps, h2)


# ---------------------------------------------------------------- prefill
PAIR_DTYPE = np.dtype([("token", np.uint32), ("expert", np.uint32), ("rank", np.uint32),
                       ("weight_bits", np.uint32)])
GROUP_DTYPE = np.dtype([("expert", np.uint32), ("pair_start", np.uint32),
                        ("pair_count", np.uint32)])
TILE_DTYPE = np.dtype([("group_start", np.uint32), ("group_count", np.uint32),
                       ("pair_start", np.uint32), ("pair_count", np.uint32)])

GROUP_ERRORS = {-1: "invalidQueryCount", -2: "invalidTopK", -3: "invalidNumExperts",
                -4: "invalidTileExpertCount", -5: "pairCountMismatch",
                -6: "tokenOutOfRange", -7: "rankOutOfRange", -8: "expertOutOfRange",
                -9: "duplicateTokenRank", -10: "expertSortKeyCountMismatch"}


class GroupingError(Exception):
    def __init__(self, code):
        super().__init__(GROUP_ERRORS.get(code, str(code)))
        self.code = code
        self.name = GROUP_ERRORS.get(code)


def make_pairs(idx, w_f16):
    idx = np.ascontiguousarray(idx, np.uint32)
    tokens, k = idx.shape
    pairs = np.zeros(tokens * k, PAIR_DTYPE)
    lib.orc_make_pairs(idx, np.ascontiguousarray(w_f16, np.uint16), tokens, k,
                       pairs.view(np.uint32))
    return pairs


lib.orc_group_pairs.restype = C.c_int
lib.orc_group_pairs.argtypes = [C.c_void_p, size_t, C.c_long, C.c_long, C.c_long, C.c_long,
                                C.c_void_p, size_t, C.c_void_p, u32p, u32p, C.c_void_p,
                                C.POINTER(size_t), C.c_void_p, C.POINTER(size_t)]


def group_pairs(pairs, query_count, top_k, num_experts, tile_expert_count=16, sort_keys=None):
    pairs = np.ascontiguousarray(pairs, PAIR_DTYPE)
    n = pairs.size
    ne = max(int(num_experts), 1)
    sorted_pairs = np.zeros(n, PAIR_DTYPE)
    offsets = np.zeros(ne, np.uint32)
    counts = np.zeros(ne, np.uint32)
    groups = np.zeros(ne, GROUP_DTYPE)
    tiles = np.zeros(ne, TILE_DTYPE)
    ng, nt = size_t(0), size_t(0)
    keys = None if sort_keys is None else np.ascontiguousarray(sort_keys, np.uint64)
    rc = lib.orc_group_pairs(pairs.ctypes.data, n, query_count, top_k, num_experts,
                             tile_expert_count, _ptr(keys), 0 if keys is None else keys.size,
                             sorted_pairs.ctypes.data, offsets, counts, groups.ctypes.data,
                             C.byref(ng), tiles.ctypes.data, C.byref(nt))
    if rc != 0:
        raise GroupingError(rc)
    return dict(sorted=sorted_pairs, offsets=offsets, counts=counts,
                groups=groups[:ng.value], tiles=tiles[:nt.value])


lib.orc_prefill_moe.restype = None
lib.orc_prefill_moe.argtypes = [C.POINTER(C.c_void_p), u32p, C.c_int, f32p, size_t, size_t,
                                size_t, size_t, u32p, u16p, f32p]


def prefill_moe(expert_blobs, bits, x, d, f, idx, w_f16):
    x = np.ascontiguousarray(x, np.float32).reshape(-1, d)
    tokens = x.shape[0]
    idx = np.ascontiguousarray(idx, np.uint32)
    k = idx.shape[1]
    ne = expert_blobs.shape[0]
    ptrs = (C.c_void_p * ne)(*[expert_blobs[e].ctypes.data for e in range(ne)])
    h2 = np.zeros((tokens, d), np.float32)
    lib.orc_prefill_moe(ptrs, expert_offsets(d, f, bits), bits, x, tokens, d, f, k, idx,
                        np.ascontiguousarray(w_f16, np.uint16), h2)
    return h2


# ---------------------------------------------------------------- KV / attention
def kv_row_layout(elements, bits):
    s, v = size_t(0), size_t(0)
    lib.orc_kv_row_layout(elements, bits, C.byref(s), C.byref(v))
    return s.value, v.value


def kv_quantize(src, bits):
    """src float32 [tokens, elements] -> uint8 [tokens, stride]."""
    src = np.ascontiguousarray(src, np.float32)
    tokens, elements = src.shape
    stride, vb = kv_row_layout(elements, bits)
    dst = np.zeros((tokens, stride), np.uint8)
    lib.orc_kv_quantize(src, elements, tokens, elements, bits, dst, stride, vb)
    return dst


def kv_dequant(rows, elements, bits):
    stride, vb = kv_row_layout(elements, bits)
    out = np.zeros((rows.shape[0], elements), np.float32)
    for t in range(rows.shape[0]):
        lib.orc_kv_dequant_row(np.ascontiguousarray(rows[t]), elements, bits, vb, out[t])
    return out


def rope_neox_subdim(data, rotary_dim, positions, theta):
    """data float32 [tokens, heads, head_dim]; returns a rotated copy."""
    out = np.array(data, np.float32, copy=True, order="C")
    tokens, heads, hd = out.shape
    lib.orc_rope_neox_subdim(out, tokens, heads, hd, rotary_dim,
                             np.ascontiguousarray(positions, np.uint32), theta)
    return out


def split_geometry(nq, nkv, seq_len, kv_start=0, prefer_gqa_swa=False):
    vals = [C.c_uint32(0) for _ in range(4)]
    lib.orc_split_geometry(nq, nkv, seq_len, kv_start, int(prefer_gqa_swa),
                           *[C.byref(v) for v in vals])
    return tuple(v.value for v in vals)


def attention_decode(q, k, v, kv_bits, nq, nkv, hd, seq_len, scale, kv_start=0,
                     num_chunks=0, chunk_len=0):
    """k, v: float32 [seq, nkv*hd] (kv_bits=32) or uint8 [seq, stride]."""
    q = np.ascontiguousarray(q, np.float32).reshape(nq, hd)
    stride, vb = (0, 0) if kv_bits == 32 else kv_row_layout(nkv * hd, kv_bits)
    out = np.zeros((nq, hd), np.float32)
    k = np.ascontiguousarray(k)
    v = np.ascontiguousarray(v)
    lib.orc_attention_decode(q, k.ctypes.data, v.ctypes.data, kv_bits, stride, vb, nq, nkv,
                             hd, seq_len, kv_start, scale, num_chunks, chunk_len, out)
    return out


def attention_prefill_causal(q, k, v, kv_bits, nq, nkv, hd, start, kv_valid, scale, window=0, ring=0):
    """q float32 [count, nq*hd]; k, v: float32 [rows, nkv*hd] (kv_bits=32) or uint8 [rows, stride].
    Returns float32 [count, nq*hd]."""
    q = np.ascontiguousarray(q, np.float32)
    count = q.shape[0]
    q = q.reshape(count, nq * hd)
    stride, vb = (0, 0) if kv_bits == 32 else kv_row_layout(nkv * hd, kv_bits)
    k, v = np.ascontiguousarray(k), np.ascontiguousarray(v)
    out = np.zeros((count, nq * hd), np.float32)
    fn = lib.orc_attention_prefill_causal
    fn.restype = None
    fn.argtypes = [f32p, size_t, C.c_void_p, C.c_void_p, C.c_int, size_t, size_t, size_t, size_t, size_t,
                   size_t, size_t, size_t, size_t, size_t, C.c_float, f32p, size_t]
    fn(q, nq * hd, k.ctypes.data, v.ctypes.data, kv_bits, stride, vb, nq, nkv, hd, start, count, kv_valid,
       window, ring, scale, out, nq * hd)
    return out


# ---------------------------------------------------------------- sampler
def softmax_f16(logits, softcap=0.0, tiled=False):
    logits = np.ascontiguousarray(logits, np.float32)
    probs = np.zeros(logits.size, np.uint16)
    (lib.orc_softmax_tiled_f16 if tiled else lib.orc_softmax_f16)(logits, logits.size,
                                                                  softcap, probs)
    return probs


def sample_generic(probs_f16, temperature, top_k, top_p, seed):
    p = np.ascontiguousarray(probs_f16, np.uint16)
    return lib.orc_sample_generic(p, p.size, temperature, top_k, top_p, seed)


def sample_gumbel(probs_f16, temperature, seed, position=0):
    p = np.ascontiguousarray(probs_f16, np.uint16)
    return lib.orc_sample_gumbel(p, p.size, temperature, seed, position)


class GdnLayerState:
    """Conv tail [(taps - 1), C] and recurrent state [Hv, Dv, Dk] of one gated-DeltaNet layer, fp32."""

    def __init__(self, k_heads, v_heads, dk, dv, taps):
        self.shape = (k_heads, v_heads, dk, dv, taps)
        self.tail = np.zeros((taps - 1, 2 * k_heads * dk + v_heads * dv), np.float32)
        self.state = np.zeros((v_heads, dv, dk), np.float32)


def gdn_step(st, qkv_raw, a, b, z, conv_w, a_log, dt_bias, norm_w, act=0):
    """GDNReference.step (GDNReference.swift:41-114) on st (updated in place); weights as BF16 bits.
    Returns the gated output [Hv * Dv], not rounded."""
    kh, vh, dk, dv, taps = st.shape
    out = np.zeros(vh * dv, np.float32)
    f = lambda v: np.ascontiguousarray(v, np.float32)
    u = lambda v: np.ascontiguousarray(v, np.uint16)
    lib.orc_gdn_step(f(qkv_raw), f(a), f(b), f(z), u(conv_w), u(a_log), u(dt_bias), u(norm_w), kh, vh, dk, dv,
                     taps, act, st.tail, st.state, out)
    return out


def repetition_penalty(logits, act, history, penalty, softcap=0.0):
    """Sampler.applyRepetitionPenaltyInPlace (Sampler.swift:259-293) on a copy of `logits`
    (16-bit activation values as float32; act 0 = bf16, 1 = fp16)."""
    out = np.ascontiguousarray(logits, np.float32).copy()
    ids = np.ascontiguousarray(history, np.int32)
    lib.orc_repetition_penalty(out, act, out.size, ids, ids.size, penalty, softcap)
    return out


def sampler_route(tiled_path, temperature, top_k):
    """2 = tiled top-64 sampler, 1 = generic kernel, 0 = generic greedy (Sampler.swift:196-231)."""
    return lib.orc_sampler_route(int(tiled_path), temperature, 0 if top_k is None else top_k)


def sampler_sample(logits, softcap, temperature, top_k, top_p, seed, position, tiled_path=True):
    """Sampler.sample after the penalty; returns (token, fp16 probability bits)."""
    lg = np.ascontiguousarray(logits, np.float32)
    probs = np.empty(lg.size, np.uint16)
    tok = lib.orc_sampler_sample(lg, lg.size, softcap, int(tiled_path), temperature, 0 if top_k is None else top_k,
                                 0.0 if top_p is None else top_p, seed, position, probs)
    return tok, probs


def sample(probs_f16, temperature, top_k, top_p, seed, position=0):
    """The reference kernel's own choice between greedy, Gumbel-max and the truncating path."""
    p = np.ascontiguousarray(probs_f16, np.uint16)
    return lib.orc_sample(p, p.size, temperature, top_k, top_p, seed, position)


def gumbel_for(seed, position, row):
    return lib.orc_gumbel_for(seed, position, row)


def sample_topk64(probs_f16, temperature, top_p, seed, top_k=64, want_top64=False):
    p = np.ascontiguousarray(probs_f16, np.uint16)
    if want_top64:
        idx = np.zeros(64, np.uint32)
        val = np.zeros(64, np.float32)
        tok = lib.orc_sample_topk64(p, p.size, temperature, top_p, seed, top_k,
                                    idx.ctypes.data, val.ctypes.data)
        return tok, idx, val
    return lib.orc_sample_topk64(p, p.size, temperature, top_p, seed, top_k, None, None)


def seed_for(seed, position):
    return lib.orc_seed_for(seed, position)


# ---------------------------------------------------------------- rest of the decode step
def rmsnorm(x, weight_bf16=None, eps=1e-6):
    """x [rows, d] float32 (contiguous); weight_bf16: uint16 [d] or None.  Returns float32 [rows, d]."""
    x = np.ascontiguousarray(x, np.float32)
    x2 = x.reshape(-1, x.shape[-1])
    out = np.zeros_like(x2)
    w = None if weight_bf16 is None else np.ascontiguousarray(weight_bf16, np.uint16)
    lib.orc_rmsnorm(x2, x2.shape[1], _ptr(w), x2.shape[0], x2.shape[1], eps, out, x2.shape[1])
    return out.reshape(x.shape)


EW_SILU_MUL, EW_SIGMOID_MUL, EW_SIGMOID_SCALAR, EW_ADD = 0, 1, 2, 3


def elementwise(op, a, b):
    """utility.metal:32-104 on float32 arrays (b: one value for EW_SIGMOID_SCALAR)."""
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    out = np.zeros_like(a)
    lib.orc_elementwise(op, a.reshape(-1), b.reshape(-1), a.size, out.reshape(-1))
    return out


def split_q_gate(packed, heads, dim):
    """utility.metal:75-92: [heads, 2 dim] -> q [heads, dim], gate [heads, dim]."""
    p = np.asarray(packed).reshape(heads, 2 * dim)
    return p[:, :dim].copy(), p[:, dim:].copy()


def concat_rows(lhs, rhs):
    """utility.metal:107-121: [rows, dim] + [rows, dim] -> [rows, 2 dim]."""
    return np.concatenate([np.asarray(lhs), np.asarray(rhs)], axis=1)


def embed_lookup(table, scales, biases, bits, token, out_scale=1.0):
    vocab, d = table.shape[0], table.shape[1] * 8 // bits
    out = np.zeros(d, np.float32)
    lib.orc_embed_lookup(np.ascontiguousarray(table), np.ascontiguousarray(scales, np.uint16),
                         np.ascontiguousarray(biases, np.uint16), bits, token, vocab, d, out_scale, out)
    return out


def lm_head_greedy(hidden, norm_weight_bf16, weights, scales, biases, bits, eps=1e-6, act=0, want_logits=False):
    """hidden float32 [d]; returns the token (and the logits [vocab] when asked)."""
    h = np.ascontiguousarray(hidden, np.float32)
    vocab, d = weights.shape[0], weights.shape[1] * 8 // bits
    nw = None if norm_weight_bf16 is None else np.ascontiguousarray(norm_weight_bf16, np.uint16)
    logits = np.zeros(vocab, np.float32) if want_logits else None
    tok = lib.orc_lm_head_greedy(h, _ptr(nw), np.ascontiguousarray(weights), np.ascontiguousarray(scales, np.uint16),
                                 np.ascontiguousarray(biases, np.uint16), bits, d, vocab, eps, act, _ptr(logits))
    return (tok, logits) if want_logits else tok


def rel_error(actual, reference):
    """RelError.swift:5-16: max|a-r| / max(max|r|, 1e-6)."""
    a = np.ascontiguousarray(actual, np.float32).reshape(-1)
    r = np.ascontiguousarray(reference, np.float32).reshape(-1)
    return float(lib.orc_rel_error(a, r, a.size))


# ---------------------------------------------------------------- reference C kernel
def load_reference_gemv():
    """The reference's own nvmai_int4_affine_gemv compiled from its source
    (oracle/_ref).  Returns None when it was never built."""
    if not os.path.exists(_REF_PATH):
        return None
    ref = C.CDLL(_REF_PATH)
    ref.nvmai_int4_affine_gemv.restype = None
    ref.nvmai_int4_affine_gemv.argtypes = [u8p, u16p, u16p, f32p, size_t, size_t, f32p]
    return ref.nvmai_int4_affine_gemv


def time_expert_ffn(blobs, d, f, x, reps=41, reference=False):
    """bench.py's cpu_baseline leg for BASELINE configs[0]: median seconds of ONE 4-bit expert FFN on one
    thread (CPUExpertFFN.accumulate, CPUExpertFFN.swift:101-139: gate and up GEMVs, silu(g) * u, down GEMV,
    out += w * down), a different blob of `blobs` [n, stride] every repetition so that the weights do not
    come from the cache.  reference=True: the three GEMVs are the reference's own nvmai_int4_affine_gemv
    (oracle/_ref, its C file compiled by oracle/Makefile) and the lines of Swift around them are numpy;
    otherwise the port orc_expert_ffn_accumulate of the -O3 native timing library.  Returns (seconds,
    the last output) or (None, None) when the reference library was never built."""
    import time
    off = expert_offsets(d, f, 4)
    x = np.ascontiguousarray(x, np.float32)
    out = np.zeros(d, np.float32)
    times = []
    if reference:
        gemv = load_reference_gemv()
        if gemv is None:
            return None, None
        g, u, dn = np.zeros(f, np.float32), np.zeros(f, np.float32), np.zeros(d, np.float32)
        parts = lambda blob, i, rows, cols: (blob[off[3 * i]:off[3 * i] + rows * cols // 2],
                                             blob[off[3 * i + 1]:off[3 * i + 1] + rows * (cols // 64) * 2].view(np.uint16),
                                             blob[off[3 * i + 2]:off[3 * i + 2] + rows * (cols // 64) * 2].view(np.uint16))
        for r in range(-2, reps):
            blob = blobs[r % len(blobs)]
            pg, pu, pd = parts(blob, 0, f, d), parts(blob, 1, f, d), parts(blob, 2, d, f)
            t0 = time.perf_counter()
            gemv(pg[0], pg[1], pg[2], x, f, d, g)
            gemv(pu[0], pu[1], pu[2], x, f, d, u)
            act = (g / (1.0 + np.exp(-g)) * u).astype(np.float32)
            gemv(pd[0], pd[1], pd[2], act, d, f, dn)
            out = dn.copy()
            if r >= 0:
                times.append(time.perf_counter() - t0)
    else:
        clib, _ = timing_lib()
        fn = clib.orc_expert_ffn_accumulate
        fn.restype = None
        fn.argtypes = [u8p, u32p, C.c_int, f32p, size_t, size_t, C.c_float, f32p, f32p]
        scratch = np.zeros(2 * f + d, np.float32)
        for r in range(-2, reps):
            blob = np.ascontiguousarray(blobs[r % len(blobs)])
            out[:] = 0
            t0 = time.perf_counter()
            fn(blob, off, 4, x, d, f, 1.0, scratch, out)
            if r >= 0:
                times.append(time.perf_counter() - t0)
    return float(np.median(times)), out
