"""Pins the oracle's gated-DeltaNet step (orc_gdn_step, a restatement of GDNReference.swift:41-114).

The reference holds no numeric vector for it (its tests compare the Metal kernels with that CPU
model on a seeded fixture), so the oracle is pinned by what the mathematics fixes: an independent
float64 matrix-form recomputation of the recurrence as the header of gdn.metal states it
(S = g S; kv = S k; S += outer((v - kv) beta, k); y = S q), closed forms for the first token, and
special cases that reduce to textbook facts."""
import numpy as np

import oracle as O

CFG = (2, 4, 32, 32, 4)          # GDNKernelTests.swift:16-18: Hk 2, Hv 4, Dk 32, Dv 32, 4 taps


def _fixture(rows, seed, cfg=CFG):
    """GDNKernelTests.Fixture (GDNKernelTests.swift:63-94): the same ranges, this build's generator."""
    kh, vh, dk, dv, taps = cfg
    C = 2 * kh * dk + vh * dv
    rng = np.random.default_rng(seed)
    u = lambda lo, hi, n: rng.uniform(lo, hi, n).astype(np.float32)
    return dict(conv_w=O.bf16_bits(u(-0.4, 0.4, C * taps)), a_log=O.bf16_bits(u(-1.0, 1.5, vh)),
                dt_bias=O.bf16_bits(u(-0.5, 0.5, vh)), norm_w=O.bf16_bits(u(0.5, 1.5, dv)),
                qkv=O.f16_to_float(O.f16_bits(u(-1, 1, rows * C))).reshape(rows, C),
                a=O.f16_to_float(O.f16_bits(u(-1, 1, rows * vh))).reshape(rows, vh),
                b=O.f16_to_float(O.f16_bits(u(-1, 1, rows * vh))).reshape(rows, vh),
                z=O.f16_to_float(O.f16_bits(u(-1, 1, rows * vh * dv))).reshape(rows, vh * dv))


def _float64_model(fx, cfg, rows):
    """The layer in float64 matrix form, no intermediate rounding."""
    kh, vh, dk, dv, taps = cfg
    C = 2 * kh * dk + vh * dv
    W = O.bf16_to_float(fx["conv_w"]).astype(np.float64).reshape(C, taps)
    A = np.exp(O.bf16_to_float(fx["a_log"]).astype(np.float64))
    dtb = O.bf16_to_float(fx["dt_bias"]).astype(np.float64)
    nw = O.bf16_to_float(fx["norm_w"]).astype(np.float64)
    seq = np.vstack([np.zeros((taps - 1, C)), fx["qkv"][:rows].astype(np.float64)])
    S = np.zeros((vh, dv, dk))
    outs = []
    silu = lambda x: x / (1 + np.exp(-x))
    for t in range(rows):
        conv = silu((seq[t:t + taps] * W.T).sum(0))
        q = conv[:kh * dk].reshape(kh, dk)
        k = conv[kh * dk:2 * kh * dk].reshape(kh, dk)
        v = conv[2 * kh * dk:].reshape(vh, dv)
        q = q / np.sqrt((q * q).mean(1, keepdims=True) + 1e-6) / dk
        k = k / np.sqrt((k * k).mean(1, keepdims=True) + 1e-6) / np.sqrt(dk)
        g = np.exp(-A * np.log1p(np.exp(fx["a"][t].astype(np.float64) + dtb)))
        beta = 1 / (1 + np.exp(-fx["b"][t].astype(np.float64)))
        y = np.zeros((vh, dv))
        for h in range(vh):
            hk = h // (vh // kh)
            S[h] *= g[h]
            kv = S[h] @ k[hk]
            S[h] += np.outer((v[h] - kv) * beta[h], k[hk])
            y[h] = S[h] @ q[hk]
        y = y / np.sqrt((y * y).mean(1, keepdims=True) + 1e-6) * nw
        outs.append((y * silu(fx["z"][t].astype(np.float64).reshape(vh, dv))).reshape(-1))
    return np.array(outs), S


def test_gdn_step_matches_float64_matrix_form():
    rows = 6
    for act, tol in ((1, 2e-2), (0, 8e-2)):           # fp16 as the reference rounds; bf16 has 3 bits fewer
        fx = _fixture(rows, 0x51D)
        st = O.GdnLayerState(*CFG)
        got = np.array([O.gdn_step(st, fx["qkv"][t], fx["a"][t], fx["b"][t], fx["z"][t], fx["conv_w"], fx["a_log"],
                                   fx["dt_bias"], fx["norm_w"], act) for t in range(rows)])
        want, S = _float64_model(fx, CFG, rows)
        # the reference's own bar for its kernels against its CPU model (GDNKernelTests.swift:170-175, 180-185)
        assert np.all(np.abs(got - want) <= np.maximum(tol, np.abs(want) * 2 * tol))
        assert np.abs(st.state - S).max() <= 5e-2
        # the tail holds the last three raw rows, oldest first
        assert np.array_equal(st.tail, fx["qkv"][rows - 3:rows] if act == 1 else O.round_bf16(fx["qkv"][rows - 3:rows]))


def test_gdn_first_token_closed_form():
    # From a zero state the first token's y is beta * v * (k . q) whatever the decay is, and the state
    # becomes beta * outer(v, k); with q and k normalised per head k . k = 1 and q . k = cos / sqrt(Dk).
    kh, vh, dk, dv, taps = CFG
    fx = _fixture(1, 7)
    st = O.GdnLayerState(*CFG)
    O.gdn_step(st, fx["qkv"][0], fx["a"][0], fx["b"][0], fx["z"][0], fx["conv_w"], fx["a_log"], fx["dt_bias"],
               fx["norm_w"], 1)
    C = 2 * kh * dk + vh * dv
    W = O.bf16_to_float(fx["conv_w"]).reshape(C, taps)
    acc = fx["qkv"][0] * W[:, taps - 1]
    conv = O.f16_to_float(O.f16_bits(acc / (1 + np.exp(-acc))))
    k = conv[kh * dk:2 * kh * dk].reshape(kh, dk).astype(np.float64)
    k = k / np.sqrt((k * k).mean(1, keepdims=True) + 1e-6) / np.sqrt(dk)
    v = conv[2 * kh * dk:].reshape(vh, dv)
    beta = 1 / (1 + np.exp(-fx["b"][0].astype(np.float64)))
    for h in range(vh):
        want = beta[h] * np.outer(v[h], k[h // (vh // kh)])
        assert np.abs(st.state[h] - want).max() < 2e-3
    assert abs((k * k).sum(1) - 1).max() < 1e-3           # unit keys after the folded 1 / sqrt(Dk)


def test_gdn_decay_and_gate_special_cases():
    kh, vh, dk, dv, taps = CFG
    C = 2 * kh * dk + vh * dv
    fx = _fixture(3, 11)
    # (a) beta -> 0 (b very negative): the state only decays; from zero it stays zero and y = 0
    st = O.GdnLayerState(*CFG)
    out = O.gdn_step(st, fx["qkv"][0], fx["a"][0], np.full(vh, -200.0, np.float32), fx["z"][0], fx["conv_w"],
                     fx["a_log"], fx["dt_bias"], fx["norm_w"], 1)
    assert not st.state.any() and not out.any()
    # (b) a huge softplus argument gives g = exp(-exp(A) * x) -> 0: the old state is forgotten and the
    #     step equals a first step from zero state
    st1, st2 = O.GdnLayerState(*CFG), O.GdnLayerState(*CFG)
    O.gdn_step(st1, fx["qkv"][0], fx["a"][0], fx["b"][0], fx["z"][0], fx["conv_w"], fx["a_log"], fx["dt_bias"],
               fx["norm_w"], 1)
    big_a = np.full(vh, 60.0, np.float32)
    st2.tail[:] = st1.tail
    o1 = O.gdn_step(st1, fx["qkv"][1], big_a, fx["b"][1], fx["z"][1], fx["conv_w"], fx["a_log"], fx["dt_bias"],
                    fx["norm_w"], 1)
    o2 = O.gdn_step(st2, fx["qkv"][1], big_a, fx["b"][1], fx["z"][1], fx["conv_w"], fx["a_log"], fx["dt_bias"],
                    fx["norm_w"], 1)
    assert np.allclose(o1, o2, atol=1e-6) and np.allclose(st1.state, st2.state, atol=1e-7)
    # (c) z = 0 closes the output gate (silu(0) = 0)
    st = O.GdnLayerState(*CFG)
    out = O.gdn_step(st, fx["qkv"][0], fx["a"][0], fx["b"][0], np.zeros(vh * dv, np.float32), fx["conv_w"],
                     fx["a_log"], fx["dt_bias"], fx["norm_w"], 1)
    assert not out.any() and st.state.any()
