"""Host logic of the streamed prefill tiles: PrefillStreamedTileBinding, the slot lifetime tracker and
the 128-byte parameter block, with the cases of the reference's own tests
(PrefillGroupedRoutedMoETests+Binding.swift:7-160, +Layout.swift:7-30).  No GPU needed: the views here
are CPU tensors, only their addresses are taken."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O


@pytest.fixture(scope="module")
def nv():
    import nvmai_amd
    return nvmai_amd


def _views(n):
    return [torch.zeros(64, dtype=torch.uint8) for _ in range(n)]


def _pair(token, expert, rank):
    return (token, expert, rank, 0x3C00)


def test_binding_maps_global_experts_to_local_slots(nv):
    # streamedTileBindingMapsGlobalExpertsToLocalSlots
    binding = nv.PrefillStreamedTileBinding([3, 9, 17], _views(3))
    assert binding.local_slot(3) == 0 and binding.local_slot(9) == 1 and binding.local_slot(17) == 2
    assert binding.local_slot(5) is None
    pairs = [_pair(0, 3, 0), _pair(0, 9, 1), _pair(1, 3, 0), _pair(1, 17, 1)]
    binding.validate_covers_pairs([p[1] for p in pairs], 0, len(pairs))
    assert len(binding.pointers()) == 3 and all(p != 0 for p in binding.pointers())
    # a view may be a (buffer, byte offset) pair, as a fetched expert lies inside a slot buffer
    buf = torch.zeros(256, dtype=torch.uint8)
    assert nv.PrefillStreamedTileBinding([1], [(buf, 48)]).pointers() == [buf.data_ptr() + 48]


def test_binding_rejects_unbound_route_expert_and_duplicates(nv):
    # streamedTileBindingRejectsUnboundRouteExpert
    binding = nv.PrefillStreamedTileBinding([3, 9], _views(2))
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="17"):
        binding.validate_covers_pairs([3, 17], 0, 2)
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="duplicate"):
        nv.PrefillStreamedTileBinding([3, 3], _views(2))
    # the other preconditions of init (PrefillGroupedRoutedMoE.swift:189-214) and of the pair range (:274-279)
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="at least one"):
        nv.PrefillStreamedTileBinding([], [])
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="maximum is 16"):
        nv.PrefillStreamedTileBinding(list(range(17)), _views(17))
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="views.count"):
        nv.PrefillStreamedTileBinding([1, 2], _views(1))
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="non-negative"):
        nv.PrefillStreamedTileBinding([-1], _views(1))
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="exceeds"):
        binding.validate_covers_pairs([3, 9], 1, 2)


def test_tile_planning_never_exceeds_sixteen_experts(nv):
    # streamedTilePlanningNeverExceedsDefaultSlotCount: 24 pairs over experts 0..19, tiles of 16
    pairs = np.zeros(24, O.PAIR_DTYPE)
    for i in range(24):
        pairs[i] = (i // 8, min(i, 19), i % 8, 0x3C00)
    routes = O.group_pairs(pairs, 3, 8, 128, 16)
    groups = [tuple(int(v) for v in g) for g in routes["groups"]]
    tiles = [tuple(int(v) for v in t) for t in routes["tiles"]]
    first = nv.PrefillStreamedTileBinding.expert_ids_for_tile(0, groups, tiles)
    second = nv.PrefillStreamedTileBinding.expert_ids_for_tile(1, groups, tiles)
    assert first == list(range(16)) and second == list(range(16, 20))
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="out of range"):
        nv.PrefillStreamedTileBinding.expert_ids_for_tile(2, groups, tiles)
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="expected 1...16"):
        nv.PrefillStreamedTileBinding.expert_ids_for_tile(0, groups, [(0, 17, 0, 24)])
    with pytest.raises(nv.PrefillGroupedRoutedMoEError, match="exceeds"):
        nv.PrefillStreamedTileBinding.expert_ids_for_tile(0, groups, [(15, 16, 0, 24)])


def test_slot_lifetime_rejects_reuse_before_completion(nv):
    # streamedTileSlotLifetimeRejectsPlannedCacheSlotReuseBeforeCompletion
    lifetime = nv.PrefillStreamedTileSlotLifetime()
    lifetime.begin(0, [0, 1, 2, 3])
    with pytest.raises(nv.PrefillStreamedTileLifetimeError) as e:
        lifetime.begin(1, [0, 1, 2, 3])
    assert (e.value.kind, e.value.tile_index, e.value.conflicting_tile_index, e.value.slots) == \
        ("slotReuseBeforeCompletion", 1, 0, [0, 1, 2, 3])
    lifetime.complete(0)
    lifetime.begin(1, [0, 1, 2, 3])
    lifetime.complete(1)


def test_slot_lifetime_allows_disjoint_and_sequential_use(nv):
    # streamedTileSlotLifetimeAllowsPinnedNonOverlappingSlots, ...AllowsSequentialReuseAfterCompletion
    lifetime = nv.PrefillStreamedTileSlotLifetime()
    lifetime.begin(0, [0, 1])
    lifetime.begin(1, [2, 3])
    lifetime.complete(0)
    lifetime.complete(1)
    with pytest.raises(nv.PrefillStreamedTileLifetimeError) as e:
        lifetime.begin(2, [4, 4])
    assert (e.value.kind, e.value.tile_index, e.value.slots) == ("duplicateSlots", 2, [4, 4])
    for tile in range(4):
        lifetime.begin(tile, list(range(8)))
        lifetime.complete(tile)
    with pytest.raises(nv.PrefillStreamedTileLifetimeError) as e:
        lifetime.complete(9)
    assert e.value.kind == "completeWithoutInFlightTile"


def test_streamed_params_layout_is_stable(nv):
    # streamedParamsLayoutIsStable: 128 bytes, the field offsets of the Metal struct
    P = nv._lib.PrefillStreamedParams
    assert C.sizeof(P) == 128
    want = dict(pair_start=0, pair_count=4, d=8, routed_intermediate=12, top_k=16, hidden_stride_elements=20,
                live_expert_count=24, local_expert=28, gate_w_off=92, down_b_off=124)
    for name, offset in want.items():
        assert getattr(P, name).offset == offset, name
    assert P.local_expert.offset + 15 * 4 == 88
    off, _ = nv.expert_offsets(64, 64, 4)
    binding = nv.PrefillStreamedTileBinding([5, 2, 11], _views(3))
    p = nv.prefill_streamed_params(7, 40, 64, 64, 2, 72, binding, off)
    words = np.frombuffer(bytes(p), np.uint32)
    assert list(words[:7]) == [7, 40, 64, 64, 2, 72, 3]
    assert list(words[7:10]) == [5, 2, 11] and (words[10:23] == 0xFFFFFFFF).all()
    assert list(words[23:]) == [off.gate_w, off.gate_s, off.gate_b, off.up_w, off.up_s, off.up_b,
                                off.down_w, off.down_s, off.down_b]
