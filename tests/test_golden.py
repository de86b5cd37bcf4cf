"""The reference's own known answers, kept as data under tests/golden/, against the CPU oracle
and the host-side functions of the C ABI."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                   "reference_known_answers.json")))


@pytest.fixture(scope="module")
def lib():
    from nvmai_amd import _lib
    return _lib


def test_expert_offsets(lib):
    for c in GOLD["expert_offsets"]["cases"]:
        off = O.expert_offsets(c["d"], c["f"], c["bits"])
        names = ["gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b", "stride"]
        got = dict(zip(names, [int(v) for v in off]))
        for k in ("gate_s", "up_w", "down_w", "stride"):
            if k in c:
                assert got[k] == c[k], (c, k)
        abi_off, stride = lib.ExpertOffsets(), C.c_uint64()
        assert lib.lib.nvmai_expert_offsets_for(c["d"], c["f"], c["bits"], C.byref(abi_off), C.byref(stride)) == 0
        assert stride.value == c["stride"]


def test_kv_row_strides(lib):
    g = GOLD["kv_row_strides"]
    for bits, stride in g["stride_by_bits"].items():
        assert O.kv_row_layout(g["elements"], int(bits))[0] == stride
        s, v = C.c_uint32(), C.c_uint32()
        assert lib.lib.nvmai_kv_row_layout(g["elements"], int(bits), C.byref(s), C.byref(v)) == 0 and s.value == stride


def test_split_geometry(lib):
    for c in GOLD["split_geometry"]["cases"]:
        want = [c["effective_length"], c["num_chunks"], c["chunk_length"], c["partial_threadgroups"]]
        got = O.split_geometry(c["num_q_heads"], c["num_kv_heads"], c["seq_len"], c["kv_start"], c["prefer_gqa_swa"])
        assert list(got) == want
        out = [C.c_uint32() for _ in range(4)]
        assert lib.lib.nvmai_attention_split_geometry(c["num_q_heads"], c["num_kv_heads"], c["seq_len"], c["kv_start"],
                                                      int(c["prefer_gqa_swa"]), *[C.byref(o) for o in out]) == 0
        assert [o.value for o in out] == want


def test_pair_records():
    g = GOLD["pair_records"]
    assert O.PAIR_DTYPE.itemsize == g["record_bytes"]
    assert [O.PAIR_DTYPE.fields[n][1] for n in ("token", "expert", "rank", "weight_bits")] == g["field_offsets"]
    idx = np.array(g["indices"], np.uint32)
    w = O.f16_bits(np.linspace(0.1, 0.6, idx.size, dtype=np.float32)).reshape(idx.shape)
    p = O.make_pairs(idx, w)
    assert list(p["token"]) == g["tokens"] and list(p["rank"]) == g["ranks"] and list(p["expert"]) == g["experts"]
    assert np.array_equal(p["weight_bits"], w.reshape(-1))


def test_grouping_cases():
    for c in GOLD["grouping"]["cases"]:
        pairs = np.zeros(len(c["pairs"]), O.PAIR_DTYPE)
        for i, row in enumerate(c["pairs"]):
            pairs[i] = tuple(row)
        g = O.group_pairs(pairs, c["query_count"], c["top_k"], c["num_experts"], c["tile_expert_count"],
                          sort_keys=c["sort_keys"])
        if "sorted_experts" in c:
            assert list(g["sorted"]["expert"]) == c["sorted_experts"], c["name"]
        if "sorted_token_rank" in c:
            assert [[int(p["token"]), int(p["rank"])] for p in g["sorted"]] == c["sorted_token_rank"]
        if "sorted_weight_bits" in c:
            assert list(g["sorted"]["weight_bits"]) == c["sorted_weight_bits"]
        if "offsets" in c:
            assert list(g["offsets"]) == c["offsets"]
        if "counts" in c:
            assert list(g["counts"]) == c["counts"]
        if "groups" in c:
            assert [list(map(int, x)) for x in g["groups"]] == c["groups"]
        if "group_experts" in c:
            assert list(g["groups"]["expert"]) == c["group_experts"]
        if "tiles" in c:
            assert [list(map(int, x)) for x in g["tiles"]] == c["tiles"]


def test_constant_blob_ffn():
    c = GOLD["constant_blob_ffn"]
    d, f = c["d"], c["f"]
    off = O.expert_offsets(d, f, 4)
    blob = np.zeros(int(off[9]), np.uint8)                     # all codes 0: every weight equals its bias

    def fill(at, rows, cols, scale, bias):
        n = rows * (cols // 64)
        blob[at[0]:at[0] + 2 * n].view(np.uint16)[:] = O.bf16_bits(np.full(n, scale, np.float32))
        blob[at[1]:at[1] + 2 * n].view(np.uint16)[:] = O.bf16_bits(np.full(n, bias, np.float32))
    fill((int(off[1]), int(off[2])), f, d, 1.0, c["gate_bias"])
    fill((int(off[4]), int(off[5])), f, d, 1.0, c["up_bias"])
    fill((int(off[7]), int(off[8])), d, f, 1.0, c["down_bias"])
    x = np.full((1, d), c["x"], np.float32)
    idx = np.arange(c["experts"], dtype=np.uint32)[None, :]
    w = O.f16_bits(np.full((1, c["experts"]), c["route_weight"], np.float32))
    y = O.prefill_moe(np.stack([blob] * c["experts"]), 4, x, d, f, idx, w)
    assert np.abs(y - c["expected_every_output"]).max() <= c["tolerance"]


def test_sampler_production_input_tiled_equals_generic():
    c = GOLD["sampler_production_input"]
    v = c["vocab"]
    i = np.arange(v, dtype=np.uint64)
    with np.errstate(over="ignore"):
        lcg = i * np.uint64(c["lcg_mul"]) + np.uint64(c["lcg_add"])
    p = ((lcg >> np.uint64(40)).astype(np.uint32).astype(np.float64) + 1.0) / 16777217.0
    bits = O.f16_bits(p.astype(np.float32))
    for k in (c["top_k"][0], c["top_k"][3], c["top_k"][-1]):           # a sample of the grid: the generic path is slow
        for t in c["temperature"]:
            seed = c["seeds"][1]
            assert O.sample_topk64(bits, t, 0.95, seed, k) == O.sample_generic(bits, t, k, 0.95, seed)
    g1 = (v + 1023) // 1024
    g2 = (g1 * 64 + 1023) // 1024
    assert (g1 * 64 + g2 * 64) * 8 == c["scratch_bytes"]
