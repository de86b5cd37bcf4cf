"""The C-ABI library loads without a GPU and exports every function the header declares;
host-only entry points (layouts, geometry, argument checks) are exercised here too."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nvmai_hip.h")


@pytest.fixture(scope="module")
def lib():
    from nvmai_amd import _lib
    return _lib


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(nvmai_[a-z0-9_]+)\s*\(", text)))


def test_header_functions_are_exported_and_bound(lib):
    names = _declared_functions()
    assert len(names) >= 25
    bound = set(lib.SIGNATURES) | set(lib._OTHER)
    for name in names:
        assert hasattr(lib.lib, name), "library does not export %s" % name
        assert name in bound, "no ctypes signature for %s" % name
    assert sorted(bound) == names


def test_status_strings(lib):
    for code in range(0, -7, -1):
        assert lib.lib.nvmai_hip_status_string(code)


def test_expert_offsets_match_oracle(lib):
    for d, f, bits in [(2048, 512, 4), (2048, 512, 8), (128, 64, 4)]:
        off, stride = lib.ExpertOffsets(), C.c_uint64()
        assert lib.lib.nvmai_expert_offsets_for(d, f, bits, C.byref(off), C.byref(stride)) == 0
        want = O.expert_offsets(d, f, bits)
        got = [getattr(off, n) for n, _ in lib.ExpertOffsets._fields_] + [stride.value]
        assert got == list(want)
    # CPUExpertFFN.Offsets strides at the production shape
    assert O.expert_offsets(2048, 512, 4)[9] == 1769472 and O.expert_offsets(2048, 512, 8)[9] == 3342336


def test_kv_layout_and_split_geometry_host_functions(lib):
    for elems, bits in [(512, 8), (512, 4), (256, 16), (192, 4)]:
        s, v = C.c_uint32(), C.c_uint32()
        assert lib.lib.nvmai_kv_row_layout(elems, bits, C.byref(s), C.byref(v)) == 0
        assert (s.value, v.value) == O.kv_row_layout(elems, bits)
    out = [C.c_uint32() for _ in range(4)]
    assert lib.lib.nvmai_attention_split_geometry(16, 8, 1536, 512, 1, *[C.byref(o) for o in out]) == 0
    assert [o.value for o in out] == [1024, 16, 64, 128]       # AttentionTests known answer


def test_grouping_check_mirrors_reference_order(lib):
    chk = lib.lib.nvmai_prefill_grouping_check
    assert chk(8, 1, 8, 4, 16, 0, 0) == 0
    assert chk(1, -1, 1, 1, 1, 0, 0) == 1 and chk(1, 1, 0, 1, 1, 0, 0) == 2 and chk(1, 1, 1, 0, 1, 0, 0) == 3
    assert chk(1, 1, 1, 1, 17, 0, 0) == 4 and chk(1, 2, 1, 1, 1, 0, 0) == 5 and chk(1, 1, 1, 2, 1, 1, 1) == 10
    assert chk(5, 1, 1, 2, 1, 1, 1) == 10      # sort-key count is checked before the pair count


def test_sampler_seed_matches_oracle(lib):
    for seed, pos in [(0, 0), (42, 17), (2**63 + 5, 4095)]:
        assert lib.lib.nvmai_sampler_seed_for(seed, pos) == O.seed_for(seed, pos)
