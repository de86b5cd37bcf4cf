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
