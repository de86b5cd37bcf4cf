"""Pins the oracle's KV layout/quantizer, RoPE and decode attention."""
import numpy as np

import oracle as O


def test_kv_row_layout_known_answers():
    # KVCacheQuantizedAttentionTests.swift:76-88 (Hkv*hd = 512 elements)
    assert O.kv_row_layout(512, 16) == (1024, 1024)
    assert O.kv_row_layout(512, 8) == (544, 512)
    assert O.kv_row_layout(512, 4) == (288, 256)
    # odd packed sizes are even-aligned (KVCacheManager.swift:443)
    assert O.kv_row_layout(66, 4) == (34 + 8, 34)
    assert O.kv_row_layout(65, 8) == (66 + 8, 66)


def _brute_kv_codes(v, bits):
    levels = np.float32(15 if bits == 4 else 255)
    g = v.reshape(v.shape[0], -1, 64)
    mn, mx = g.min(2, keepdims=True), g.max(2, keepdims=True)
    scale = np.where(mx > mn, (mx - mn) / levels, np.float32(0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        t = np.clip(((g - mn).astype(np.float32) / scale).astype(np.float32), 0, levels)
    frac = t - np.trunc(t)
    r = np.where(np.abs(frac) == 0.5, np.trunc(t) + 1, np.rint(t))
    codes = np.where(scale > 0, r, 0).astype(np.uint8)
    return codes.reshape(v.shape), scale[..., 0], mn[..., 0]


def test_kv_quantizer_closed_form_and_invariants():
    rng = np.random.default_rng(2)
    v = O.round_bf16(rng.standard_normal((37, 512)).astype(np.float32))
    v[3, 64:128] = 0.25            # flat group -> scale 0, codes 0
    v[5, :] = v[5, 0]              # a whole flat row
    for bits in (4, 8):
        rows = O.kv_quantize(v, bits)
        stride, vb = O.kv_row_layout(512, bits)
        assert rows.shape == (37, stride)
        codes = np.stack([O.unpack_codes(r[:vb], bits) for r in rows])
        want, scale, bias = _brute_kv_codes(v, bits)
        assert np.array_equal(codes, want)
        sc = rows[:, vb:vb + 16].copy().view(np.uint16)
        bi = rows[:, vb + 16:vb + 32].copy().view(np.uint16)
        assert np.array_equal(sc, O.f16_bits(scale)) and np.array_equal(bi, O.f16_bits(bias))
        lv = 15 if bits == 4 else 255
        g = codes.reshape(37, 8, 64)
        nonflat = scale > 0
        assert np.all(g.min(2)[nonflat] == 0) and np.all(g.max(2)[nonflat] == lv)
        assert not g[3, 1].any() and sc[3, 1] == 0 and not g[5].any()
        # dequant error <= half a step + fp16 rounding of scale and bias
        rec = O.kv_dequant(rows, 512, bits)
        step = scale.repeat(64, axis=1)
        assert np.all(np.abs(rec - v) <= 0.5 * step + 2e-3 * np.maximum(np.abs(v), 1))


def test_kv_codes_are_the_nearest_codes():
    # The property itself in float64, no rounding rule restated: against the UNROUNDED fp32 scale and
    # bias of its group (kv_cache_quantize.metal:56-59 quantizes before the pair is rounded to fp16)
    # every code is at least as close to its value as both neighbouring codes, ties aside.
    rng = np.random.default_rng(23)
    for v in (O.round_bf16(rng.standard_normal((64, 512)).astype(np.float32)),
              rng.uniform(-0.5, 0.5, (16, 512)).astype(np.float32),
              (rng.standard_normal((8, 512)) * 3 + 20).astype(np.float32)):
        for bits in (4, 8):
            levels = 15 if bits == 4 else 255
            rows = O.kv_quantize(v, bits)
            _, vb = O.kv_row_layout(512, bits)
            q = np.stack([O.unpack_codes(r[:vb], bits) for r in rows]).astype(np.float64)
            g = v.reshape(v.shape[0], -1, 64)
            mn, mx = g.min(2), g.max(2)
            s = ((mx - mn) / np.float32(levels)).astype(np.float32).astype(np.float64).repeat(64, axis=1)
            b = mn.astype(np.float64).repeat(64, axis=1)
            w = v.astype(np.float64)
            err = np.abs(w - (q * s + b))
            tol = 1e-4 * s + 1e-12
            up_ok = (q >= levels) | (err <= np.abs(w - ((q + 1) * s + b)) + tol)
            down_ok = (q <= 0) | (err <= np.abs(w - ((q - 1) * s + b)) + tol)
            assert np.all(up_ok & down_ok), "%d-bit KV codes are not the nearest" % bits


def test_kv_quantizer_partial_tail_group():
    v = np.linspace(-1, 1, 3 * 100, dtype=np.float32).reshape(3, 100)
    for bits in (4, 8):
        rows = O.kv_quantize(v, bits)
        stride, vb = O.kv_row_layout(100, bits)
        assert rows.shape[1] == stride
        codes = np.stack([O.unpack_codes(r[:vb], bits)[:100] for r in rows])
        lv = 15 if bits == 4 else 255
        assert np.all(codes[:, 64] == 0) and np.all(codes[:, 99] == lv)   # tail group uses 36 values


def test_rope_identity_passthrough_and_closed_form():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((5, 3, 256)).astype(np.float32)
    pos = np.array([0, 1, 7, 1000, 131071], np.uint32)
    y = O.rope_neox_subdim(x, 64, pos, 1e7)
    assert np.array_equal(y[0], x[0])                       # position 0 is the identity
    assert np.array_equal(y[..., 64:], x[..., 64:])         # RoPEReferenceTests.swift:78-100
    i = np.arange(32)
    ang = pos[:, None].astype(np.float64) * (1e7 ** (-2.0 * i / 64.0))
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    lo, hi = x[..., :32].astype(np.float64), x[..., 32:64].astype(np.float64)
    assert np.abs(y[..., :32] - (lo * c - hi * s)).max() < 2e-2    # fp32 angle at pos 1e5
    small = pos < 2000
    assert np.abs(y[small][..., :32] - (lo * c - hi * s)[small]).max() < 1e-4
    assert np.abs(y[small][..., 32:64] - (lo * s + hi * c)[small]).max() < 1e-4
    # rotation preserves the pair norm
    assert np.allclose(y[..., :32] ** 2 + y[..., 32:64] ** 2, lo ** 2 + hi ** 2, rtol=1e-4)


def test_split_geometry_known_answers():
    # AttentionTests.swift:25-47
    assert O.split_geometry(16, 8, 1536, 512, True) == (1024, 16, 64, 128)
    assert O.split_geometry(16, 2, 1536, 0, False) == (1536, 16, 96, 256)
    assert O.split_geometry(16, 2, 5, 0, False) == (5, 5, 1, 80)
    assert O.split_geometry(16, 2, 1, 0, False) == (1, 1, 1, 16)


def _attention64(q, k, v, nq, nkv, hd, scale):
    out = np.zeros((nq, hd))
    for h in range(nq):
        kv = h // (nq // nkv)
        s = k[:, kv * hd:(kv + 1) * hd].astype(np.float64) @ q[h].astype(np.float64) * scale
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ v[:, kv * hd:(kv + 1) * hd].astype(np.float64)
    return out


def test_attention_matches_textbook_and_split_equals_single():
    rng = np.random.default_rng(6)
    nq, nkv, hd, seq = 16, 2, 256, 77
    q = rng.uniform(-0.5, 0.5, (nq, hd)).astype(np.float32)
    k = rng.uniform(-0.5, 0.5, (seq, nkv * hd)).astype(np.float32)
    v = rng.uniform(-0.5, 0.5, (seq, nkv * hd)).astype(np.float32)
    want = _attention64(q, k, v, nq, nkv, hd, 0.0625)
    single = O.attention_decode(q, k, v, 32, nq, nkv, hd, seq, 0.0625)
    assert O.rel_error(single, want) < 1e-5
    _, nc, cl, _ = O.split_geometry(nq, nkv, seq)
    split = O.attention_decode(q, k, v, 32, nq, nkv, hd, seq, 0.0625, num_chunks=nc, chunk_len=cl)
    assert O.rel_error(split, want) < 1e-5
    one = O.attention_decode(q, k, v, 32, nq, nkv, hd, seq, 0.0625, num_chunks=1, chunk_len=seq)
    assert np.array_equal(one, single)                       # attention.metal:155-159
    # empty range -> zeros (attention.metal:410-416)
    z = O.attention_decode(q, k, v, 32, nq, nkv, hd, seq, 0.0625, kv_start=seq, num_chunks=4, chunk_len=1)
    assert not z.any()


def test_quantized_attention_tracks_unquantized_reference():
    # KVCacheQuantizedAttentionTests.swift:7-74: seq 8, uniform(-0.5,0.5),
    # rel < 0.02 (8-bit) / 0.20 (4-bit) against the unquantized reference
    nq, nkv, hd, seq = 16, 2, 256, 8
    for bits, tol in ((8, 0.02), (4, 0.20)):
        g = O.seed_tree(0x4B56, "kv-cache-%d" % bits)
        h = lambda n: O.f16_to_float(O.f16_bits(g.uniform_array(n, -0.5, 0.5)))
        q = h(nq * hd).reshape(nq, hd)
        k = h(seq * nkv * hd).reshape(seq, -1)
        v = h(seq * nkv * hd).reshape(seq, -1)
        want = _attention64(q, k, v, nq, nkv, hd, 1 / 16.0)
        got = O.attention_decode(q, O.kv_quantize(k, bits), O.kv_quantize(v, bits), bits, nq,
                                 nkv, hd, seq, 0.0625)
        assert O.rel_error(got, want) < tol
        # and it is exactly attention over the dequantized rows
        kd = O.kv_dequant(O.kv_quantize(k, bits), nkv * hd, bits)
        vd = O.kv_dequant(O.kv_quantize(v, bits), nkv * hd, bits)
        assert O.rel_error(got, _attention64(q, kd, vd, nq, nkv, hd, 0.0625)) < 1e-5


# ---------------------------------------------------------------- causal prefill attention
def _prefill_model_f64(q, k, v, nq, nkv, hd, start, kv_valid, window, scale):
    """softmax(q K^T * scale) V per query over its visible keys, float64: what
    PrefillAttentionRef.apply (PrefillAttentionRef.swift:57-99) computes, written with matrix
    products instead of the kernel's running maximum."""
    count = q.shape[0]
    out = np.zeros((count, nq, hd))
    q = q.astype(np.float64).reshape(count, nq, hd)
    k = k.astype(np.float64).reshape(-1, nkv, hd)
    v = v.astype(np.float64).reshape(-1, nkv, hd)
    for t in range(count):
        a = start + t
        first = max(0, a + 1 - window) if window else 0
        last = min(kv_valid, a + 1)
        if last <= first:
            continue
        for h in range(nq):
            kvh = h // (nq // nkv)
            s = k[first:last, kvh] @ q[t, h] * scale
            w = np.exp(s - s.max())
            out[t, h] = (w / w.sum()) @ v[first:last, kvh]
    return out.reshape(count, nq * hd)


def _prefill_fixture(seed, start, chunk, hd, nq, nkv, extra_kv=0, lo=-0.35, hi=0.35):
    rng = np.random.default_rng(seed)
    kv_valid = start + chunk + extra_kv
    q = rng.uniform(lo, hi, (chunk, nq * hd)).astype(np.float32)
    k = rng.uniform(lo, hi, (kv_valid, nkv * hd)).astype(np.float32)
    v = rng.uniform(lo, hi, (kv_valid, nkv * hd)).astype(np.float32)
    return q, k, v, kv_valid


def test_prefill_attention_matches_the_softmax_model():
    # the shapes of PrefillAttentionTests.swift:11-16, 81-87, 101-104 (start, chunk, window, hd, nq, nkv)
    cases = [(0, 3, 0, 8, 4, 2), (4, 3, 0, 8, 4, 2), (2, 4, 16, 8, 4, 2), (7, 4, 5, 8, 4, 2),
             (1023, 1, 1, 256, 16, 8), (1024, 1, 1, 256, 16, 8), (0, 1, 0, 512, 16, 2), (3, 1, 0, 512, 16, 2),
             (1023, 4, 1024, 256, 16, 8), (31, 8, 0, 512, 16, 2)]
    for n, (start, chunk, window, hd, nq, nkv) in enumerate(cases):
        q, k, v, kv_valid = _prefill_fixture(0xA510 + n, start, chunk, hd, nq, nkv)
        got = O.attention_prefill_causal(q, k, v, 32, nq, nkv, hd, start, kv_valid, 1.0, window=window)
        want = _prefill_model_f64(q, k, v, nq, nkv, hd, start, kv_valid, window, 1.0)
        assert np.abs(got - want).max() < 2e-6, (start, chunk, window)
        # query t alone is the decode call over its own key range
        for t in range(chunk):
            a = start + t
            first = max(0, a + 1 - window) if window else 0
            one = O.attention_decode(q[t], k, v, 32, nq, nkv, hd, a + 1, 1.0, kv_start=first)
            assert np.abs(one.reshape(-1) - got[t]).max() < 2e-6


def test_prefill_attention_masks_future_and_invalid_keys():
    # PrefillAttentionTests.swift:58-77: the chunk's own later rows carry huge scores; a query must not see them
    start, chunk, hd, nq, nkv = 5, 4, 8, 4, 2
    q, k, v, kv_valid = _prefill_fixture(0xA620, start, chunk, hd, nq, nkv)
    for row in range(start, kv_valid):
        k[row] = np.tile((row - start + 1) * 2.0 + np.arange(hd) * 0.125, nkv)
        v[row] = np.tile((row - start + 1) * -2.0 - np.arange(hd) * 0.125, nkv)
    got = O.attention_prefill_causal(q, k, v, 32, nq, nkv, hd, start, kv_valid, 1.0)
    want = _prefill_model_f64(q, k, v, nq, nkv, hd, start, kv_valid, 0, 1.0)
    assert np.abs(got - want).max() < 1e-5
    # rows past a query's own position may hold anything, NaN included
    k2, v2 = k.copy(), v.copy()
    k2[start + 1:], v2[start + 1:] = np.nan, np.nan
    first = O.attention_prefill_causal(q[:1], k2, v2, 32, nq, nkv, hd, start, kv_valid, 1.0)
    assert np.array_equal(first, got[:1])
    # kv_valid below the causal limit clamps the range (prefill.metal:765): rows >= kv_valid unseen
    q3, k3, v3, _ = _prefill_fixture(77, 6, 3, 8, 4, 2, extra_kv=0)
    got3 = O.attention_prefill_causal(q3, k3, v3, 32, 4, 2, 8, 6, 7, 1.0)     # all three queries see keys [0, 7)
    want3 = _prefill_model_f64(q3, k3, v3, 4, 2, 8, 6, 7, 0, 1.0)
    assert np.abs(got3 - want3).max() < 2e-6
    assert np.abs(got3[1] - O.attention_decode(q3[1], k3, v3, 32, 4, 2, 8, 7, 1.0).reshape(-1)).max() < 2e-6


def test_prefill_attention_ring_and_quantized_rows():
    # PrefillAttentionTests.swift:27-56: rows stored at p % capacity give the linear answer
    start, chunk, window, hd, nq, nkv, cap = 20, 4, 8, 32, 4, 2, 16
    q, k, v, kv_valid = _prefill_fixture(0xA611, start, chunk, hd, nq, nkv)
    k_ring, v_ring = np.zeros((cap, nkv * hd), np.float32), np.zeros((cap, nkv * hd), np.float32)
    for p in range(kv_valid):
        k_ring[p % cap], v_ring[p % cap] = k[p], v[p]
    linear = O.attention_prefill_causal(q, k, v, 32, nq, nkv, hd, start, kv_valid, 1.0, window=window)
    ring = O.attention_prefill_causal(q, k_ring, v_ring, 32, nq, nkv, hd, start, kv_valid, 1.0, window=window,
                                      ring=cap)
    assert np.array_equal(ring, linear)
    # quantized rows: the answer over the dequantized rows (KVCacheQuantizedAttentionTests.swift:91-157)
    hd, nq, nkv, start, chunk = 256, 16, 2, 4, 4
    q, k, v, kv_valid = _prefill_fixture(0x5052, start, chunk, hd, nq, nkv, lo=-0.5, hi=0.5)
    scale = 1.0 / np.sqrt(hd)
    dense = O.attention_prefill_causal(q, k, v, 32, nq, nkv, hd, start, kv_valid, scale)
    for bits, tol in ((8, 0.025), (4, 0.20)):
        kr, vr = O.kv_quantize(k, bits), O.kv_quantize(v, bits)
        got = O.attention_prefill_causal(q, kr, vr, bits, nq, nkv, hd, start, kv_valid, scale)
        deq = O.attention_prefill_causal(q, O.kv_dequant(kr, nkv * hd, bits), O.kv_dequant(vr, nkv * hd, bits), 32,
                                         nq, nkv, hd, start, kv_valid, scale)
        assert np.array_equal(got, deq)
        rel = O.rel_error(got, dense)                    # RelError.swift:5-16
        assert rel < tol, (bits, rel)
