"""Pins oracle/qk_oracle_deltanet.py (the restated gated-DeltaNet decode step) by closed forms and
invariants of the delta rule."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import qk_oracle_deltanet as OD  # noqa: E402

DS, HK, HV = 128, 4, 8
F = np.float32


def rand(shape, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(F)


def unit(v):
    return (v / np.linalg.norm(v)).astype(F)


def conv_vec(q, k, v):
    return np.concatenate([q.reshape(-1), k.reshape(-1), v.reshape(-1)]).astype(F)


def test_ab_limits_and_formula():
    x = rand(2048, 1)
    aw, bw = rand((HV, 2048), 2, 0.02), rand((HV, 2048), 3, 0.02)
    dt, a = rand(HV, 4), -np.abs(rand(HV, 5))
    g, b = OD.ab(x, aw, bw, dt, a)
    d = aw.astype(np.float64) @ x + dt
    np.testing.assert_allclose(g, a * np.log(1 + np.exp(d)), rtol=1e-6)
    np.testing.assert_allclose(b, 1 / (1 + np.exp(-(bw.astype(np.float64) @ x))), rtol=1e-6)
    # softplus(v) -> v for large v, -> exp(v) for very negative v; beta in (0, 1)
    g_big, _ = OD.ab(x, aw * 0, bw, np.full(HV, 50, F), np.ones(HV, F))
    g_small, _ = OD.ab(x, aw * 0, bw, np.full(HV, -30, F), np.ones(HV, F))
    assert np.allclose(g_big, 50.0) and np.allclose(g_small, np.exp(-30.0), rtol=1e-5)
    assert np.all((b > 0) & (b < 1))


def test_conv_window_and_unit_heads():
    ch, qk = (2 * HK + HV) * DS, 2 * HK * DS
    ker = rand((ch, 4), 6)
    st = np.zeros((ch, 3), F)
    xs = [rand(ch, 10 + i) for i in range(5)]
    outs = [OD.conv(st, x, ker, DS, qk) for x in xs]
    # the window holds the last three inputs, oldest first
    assert np.array_equal(st[:, 0], xs[2]) and np.array_equal(st[:, 1], xs[3]) and np.array_equal(st[:, 2], xs[4])
    # the 5th output convolves inputs 2..5 with taps 0..3, then SiLU; v channels pass through unscaled
    c = (xs[1].astype(np.float64) * ker[:, 0] + xs[2].astype(np.float64) * ker[:, 1] +
         xs[3].astype(np.float64) * ker[:, 2] + xs[4].astype(np.float64) * ker[:, 3])
    silu = c / (1 + np.exp(-c))
    np.testing.assert_allclose(outs[4][qk:], silu[qk:], rtol=1e-6, atol=1e-7)
    heads = outs[4][:qk].reshape(-1, DS).astype(np.float64)
    np.testing.assert_allclose(np.linalg.norm(heads, axis=1), 1.0, rtol=1e-6)
    np.testing.assert_allclose(heads, silu[:qk].reshape(-1, DS) / np.linalg.norm(silu[:qk].reshape(-1, DS), axis=1)[:, None],
                               rtol=1e-5, atol=1e-7)
    # an all-zero head is divided by eps, not by zero
    st0 = np.zeros((ch, 3), F)
    assert np.isfinite(OD.conv(st0, np.zeros(ch, F), ker, DS, qk)).all()


def test_delta_rule_closed_forms():
    ones, z = np.ones(DS, F), np.full(HV * DS, 30.0, F)      # silu(30) = 30 to 1e-12
    q = np.stack([unit(rand(DS, 20 + i)) for i in range(HK)])
    k = np.stack([unit(rand(DS, 30 + i)) for i in range(HK)])
    v = rand((HV, DS), 40)
    g0, b1 = np.zeros(HV, F), np.ones(HV, F)
    for kdiv in (0, 2):
        S = np.zeros((HV, DS, DS), F)
        att = OD.step(conv_vec(q, k, v), g0, b1, S, ones, z, HK, HV, kdiv=kdiv).reshape(HV, DS)
        for h in range(HV):
            kh = h // kdiv if kdiv else h % HK
            # empty memory, beta 1, no decay: S = v k^T, o = v (k.q) / sqrt(dS)
            np.testing.assert_allclose(S[h], np.outer(v[h], k[kh]), rtol=1e-6, atol=1e-8)
            o = v[h].astype(np.float64) * float(k[kh].astype(np.float64) @ q[kh]) / np.sqrt(DS)
            want = o / np.sqrt((o * o).mean() + 1e-6) * 30.0
            np.testing.assert_allclose(att[h], want, rtol=1e-4, atol=1e-5)
        # writing another value under the same unit key replaces the stored one: S k = v2
        v2 = rand((HV, DS), 41)
        OD.step(conv_vec(q, k, v2), g0, b1, S, ones, z, HK, HV, kdiv=kdiv)
        for h in range(HV):
            kh = h // kdiv if kdiv else h % HK
            np.testing.assert_allclose(S[h].astype(np.float64) @ k[kh], v2[h], rtol=1e-4, atol=1e-5)
    # beta 0: only the decay acts
    S = rand((HV, DS, DS), 42)
    S0 = S.copy()
    g = np.log(np.linspace(0.5, 0.9, HV)).astype(F)
    OD.step(conv_vec(q, k, v), g, np.zeros(HV, F), S, ones, z, HK, HV)
    np.testing.assert_allclose(S, S0 * np.exp(g)[:, None, None], rtol=1e-6)


def test_step_against_the_matrix_form():
    q, k, v = rand((HK, DS), 50), rand((HK, DS), 51, 0.1), rand((HV, DS), 52)
    g, b = -np.abs(rand(HV, 53, 0.3)), (1 / (1 + np.exp(-rand(HV, 54)))).astype(F)
    w, z = 1 + 0.1 * rand(DS, 55), rand(HV * DS, 56)
    S = rand((HV, DS, DS), 57, 0.2)
    S64 = S.astype(np.float64)
    att = OD.step(conv_vec(q, k, v), g, b, S, w, z, HK, HV).reshape(HV, DS)
    for h in range(HV):
        kh = h % HK
        d = np.exp(np.float64(g[h]))
        Sn = S64[h] * d + np.outer(b[h] * (v[h] - d * (S64[h] @ k[kh])), k[kh])
        np.testing.assert_allclose(S[h], Sn, rtol=2e-5, atol=2e-6)
        o = Sn @ q[kh] / np.sqrt(DS)
        want = o / np.sqrt((o * o).mean() + 1e-6) * w * (z[h * DS:(h + 1) * DS] / (1 + np.exp(-z[h * DS:(h + 1) * DS].astype(np.float64))))
        np.testing.assert_allclose(att[h], want, rtol=2e-4, atol=2e-5)
