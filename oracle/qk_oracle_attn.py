"""CPU restatement of the reference's full-attention decode step, in numpy float64.
TEST INFRASTRUCTURE ONLY: imported by tests/ (and the benchmark's checks); the product never imports it.

Follows the reference's CPU mirror of the attention block (src/main.cpp:2138-2201) and, where that
is silent, the shaders it mirrors (shaders/fa_prep_srv.comp:26-76, fa_attn_srv.comp:27-95):
  rope_table   cos / sin per (position, frequency), float arithmetic as src/main.cpp:2011-2020
  prep         per head RMS norm (rmsRef :2138-2143), rotation of the pairs (j, j + n_rot/2)
               (ropeRef :2144-2152), queries out, keys and values into the caches (:2167-2176)
  attend       scores / sqrt(dh), softmax over positions 0..pos, weighted values, sigmoid gate from
               the second half of the head's qfull row, KV head = h / (hQ/hKV) (:2177-2200)

Pinned in tests/test_attn_oracle.py by what the mathematics fixes: one key gives the value row
times the gate; equal keys give the mean of the values; a KV head of zeros / ones shows which query
heads read it; the gate is taken from the right half; position 0 is not rotated, a rotation keeps
each pair's length and makes q.k depend on the distance of the positions only; the norm output has
unit mean square for unit weights; and an independent evaluation with scipy's softmax."""
import numpy as np


def rope_table(tmax, n_rot, freq_base=1e7):
    half = n_rot // 2
    p = np.arange(tmax, dtype=np.float32)[:, None]
    j = np.arange(half, dtype=np.float32)[None, :]
    inv = np.power(np.float32(freq_base), np.float32(-2.0) * j / np.float32(n_rot)).astype(np.float32)
    th = (p * inv).astype(np.float32)
    return np.stack([np.cos(th), np.sin(th)], axis=-1).astype(np.float32)


def _rms(v, w, eps):
    v = v.astype(np.float64)
    return v / np.sqrt((v * v).mean() + eps) * w.astype(np.float64)


def _rope(v, cs, n_rot):
    half = n_rot // 2
    c, s = cs[:, 0].astype(np.float64), cs[:, 1].astype(np.float64)
    out = v.copy()
    x0, x1 = v[:half], v[half:n_rot]
    out[:half] = x0 * c - x1 * s
    out[half:n_rot] = x0 * s + x1 * c
    return out


def prep(qfull, kin, vin, qn, kn, rope, pos, kc, vc, n_rot, eps=1e-6):
    """One slot.  qfull [hQ][2*dh], kin / vin [hKV][dh], caches [hKV][tmax][dh] (updated in place at
    pos).  Returns qhat [hQ][dh] float32."""
    hQ, dh = qfull.shape[0], qfull.shape[1] // 2
    qhat = np.empty((hQ, dh), dtype=np.float32)
    for h in range(hQ):
        qhat[h] = _rope(_rms(qfull[h, :dh], qn, eps), rope[pos], n_rot).astype(np.float32)
    for h in range(kin.shape[0]):
        kc[h, pos] = _rope(_rms(kin[h], kn, eps), rope[pos], n_rot).astype(np.float32)
        vc[h, pos] = vin[h]
    return qhat


def attend(qhat, kc, vc, qfull, pos):
    """One slot: att [hQ][dh] float32 over positions 0..pos."""
    hQ, dh = qhat.shape
    hKV = kc.shape[0]
    att = np.empty((hQ, dh), dtype=np.float32)
    for h in range(hQ):
        kv = h // (hQ // hKV)
        K = kc[kv, :pos + 1].astype(np.float64)
        V = vc[kv, :pos + 1].astype(np.float64)
        sc = K @ qhat[h].astype(np.float64) / np.sqrt(float(dh))
        e = np.exp(sc - sc.max())
        o = (e[:, None] * V).sum(axis=0) / e.sum()
        gate = 1.0 / (1.0 + np.exp(-qfull[h, dh:].astype(np.float64)))
        att[h] = (o * gate).astype(np.float32)
    return att
