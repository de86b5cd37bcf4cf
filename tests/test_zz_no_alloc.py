"""GPU: the allocation-free decode entry point (nvmai_hip_moe_decode_layer_noalloc) against the
allocating one (nvmai_hip_moe_decode_layer), through the C ABI: routing indices, routing weights
and the 16-bit outputs equal bit for bit, on two calls in a row, the second with fewer tokens (it
finds the first call's contents in the shared static array), and a step too large for the array
is refused."""
import numpy as np
import pytest
import torch

from gpu_util import say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [8, 4])
def test_noalloc_decode_layer_equals_allocating_entry_point(bits):
    import nvmai_amd as nv
    say("no-alloc decode layer", bits)
    ctx = nv.Context(0, nv.ACT_BF16)
    d, f, E, k = 2048, 512, 64, 8
    gen = torch.Generator(device="cuda").manual_seed(900 + bits)
    off, stride = nv.expert_offsets(d, f, bits)
    mk = lambda r, c, s=0.02: torch.empty((r, c), device="cuda").normal_(0.0, s, generator=gen).to(torch.bfloat16)
    pool = torch.empty((E + 1, stride), dtype=torch.uint8, device="cuda")
    for e in range(E + 1):
        nv.pack_expert(ctx, mk(f, d), mk(f, d), mk(d, f), bits, pool[e])
    router = mk(E, d, 0.05)
    gate_w, gate_s, gate_b = (torch.empty((1, d), dtype=torch.uint8, device="cuda"),
                              torch.empty((1, d // 64), dtype=torch.int16, device="cuda"),
                              torch.empty((1, d // 64), dtype=torch.int16, device="cuda"))
    nv.quantize_affine(ctx, mk(1, d, 0.05), 8, gate_w, gate_s, gate_b)
    layer = nv.moe_layer_desc(d, f, E, k, bits, nv.rows_desc(16, router.view(torch.int16)), pool[:E], pool[E],
                              nv.rows_desc(8, gate_w, gate_s, gate_b))
    moe = nv.MoE(ctx, bits)
    assert nv.lib.nvmai_hip_moe_decode_layer_noalloc_scratch_bytes() == 4 << 20
    for tokens in (32, 5, 1):           # five launches with the work list, then fewer tokens, then three launches
        say("no-alloc decode layer", bits, "tokens", tokens)
        x = mk(tokens, d, 1.0)
        y_ref, idx_ref, w_ref = moe.decode_layer(layer, x, want_routes=True)
        torch.cuda.synchronize()
        y = torch.empty_like(y_ref)
        idx = torch.empty_like(idx_ref)
        w = torch.empty_like(w_ref)
        stats = torch.zeros(2, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]      # device-wide: sees the library's own allocations too
        moe.decode_layer_noalloc(layer, x, y, idx, w, stats)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(idx, idx_ref) and torch.equal(w, w_ref)
        assert torch.equal(y, y_ref)
        assert int(stats[1]) == len(np.unique(idx.cpu().numpy()))
    # a step that does not fit the static array is refused and launches nothing
    x = mk(64, d, 1.0)
    y = torch.full((64, d), 3.0, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(nv.NvmaiError) as e:
        moe.decode_layer_noalloc(layer, x, y)
    torch.cuda.synchronize()
    assert e.value.name == "scratch" and bool((y == 3.0).all())
    ctx.close()
