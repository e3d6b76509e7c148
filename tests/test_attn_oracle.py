"""Pins oracle/qk_oracle_attn.py (the restated attention decode step) by closed forms, invariants
and an independent evaluation; and the library's host-side RoPE table against it."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import qk_oracle_attn as OA  # noqa: E402

HQ, HKV, DH, NROT = 16, 2, 256, 64


def rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def test_one_key_gives_the_value_row_times_the_gate():
    qhat, qfull = rand((HQ, DH), 1), rand((HQ, 2 * DH), 2)
    kc, vc = rand((HKV, 8, DH), 3), rand((HKV, 8, DH), 4)
    att = OA.attend(qhat, kc, vc, qfull, 0)
    for h in range(HQ):
        want = vc[h // 8, 0] / (1.0 + np.exp(-qfull[h, DH:].astype(np.float64)))
        np.testing.assert_allclose(att[h], want, rtol=1e-6)


def test_equal_keys_give_the_mean_value_and_heads_map_to_their_kv_head():
    qhat, qfull = rand((HQ, DH), 5), np.zeros((HQ, 2 * DH), np.float32)   # gate 0 -> sigmoid = 1/2
    kc = np.repeat(rand((HKV, 1, DH), 6), 10, axis=1)
    vc = rand((HKV, 10, DH), 7)
    att = OA.attend(qhat, kc, vc, qfull, 9)
    for h in range(HQ):
        np.testing.assert_allclose(att[h], 0.5 * vc[h // 8].astype(np.float64).mean(axis=0), rtol=1e-5, atol=1e-7)
    vc[0], vc[1] = 0.0, 1.0
    att = OA.attend(qhat, rand((HKV, 10, DH), 8), vc, qfull, 9)
    assert np.all(att[:8] == 0.0) and np.allclose(att[8:], 0.5)
    # the gate comes from the second half of the head's row, the first half is not looked at
    qfull2 = qfull.copy()
    qfull2[:, :DH] = 77.0
    assert np.array_equal(OA.attend(qhat, kc, vc, qfull2, 9), OA.attend(qhat, kc, vc, qfull, 9))
    qfull2[3, DH + 5] = 50.0
    assert np.isclose(OA.attend(qhat, kc, vc, qfull2, 9)[3, 5], 2 * OA.attend(qhat, kc, vc, qfull, 9)[3, 5])


def test_against_an_independent_softmax():
    from scipy.special import softmax
    qhat, qfull = rand((HQ, DH), 9), rand((HQ, 2 * DH), 10)
    kc, vc = rand((HKV, 40, DH), 11), rand((HKV, 40, DH), 12)
    pos = 33
    K = np.repeat(kc[:, :pos + 1].astype(np.float64), 8, axis=0)            # [hQ][n][dh]
    V = np.repeat(vc[:, :pos + 1].astype(np.float64), 8, axis=0)
    P = softmax(np.einsum("hd,hnd->hn", qhat.astype(np.float64), K) / 16.0, axis=1)
    want = np.einsum("hn,hnd->hd", P, V) / (1.0 + np.exp(-qfull[:, DH:].astype(np.float64)))
    np.testing.assert_allclose(OA.attend(qhat, kc, vc, qfull, pos), want, rtol=2e-6, atol=1e-7)
    # keys beyond pos are not read
    kc[:, pos + 1:] = np.nan
    assert np.isfinite(OA.attend(qhat, kc, vc, qfull, pos)).all()


def test_prep_norm_and_rotation():
    rope = OA.rope_table(128, NROT)
    qfull, kin, vin = rand((HQ, 2 * DH), 13), rand((HKV, DH), 14), rand((HKV, DH), 15)
    ones = np.ones(DH, np.float32)
    kc, vc = np.zeros((HKV, 128, DH), np.float32), np.zeros((HKV, 128, DH), np.float32)
    q0 = OA.prep(qfull, kin, vin, ones, ones, rope, 0, kc, vc, NROT, eps=0.0)
    # position 0: no rotation; unit weights: unit mean square; values copied; only row 0 written
    np.testing.assert_allclose((q0.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-6)
    x = qfull[2, :DH].astype(np.float64)
    np.testing.assert_allclose(q0[2], x / np.sqrt((x * x).mean()), rtol=1e-6)
    assert np.array_equal(vc[:, 0], vin) and not kc[:, 1:].any() and not vc[:, 1:].any()
    # a rotation keeps each pair's length and leaves the dims beyond n_rot alone
    q7 = OA.prep(qfull, kin, vin, ones, ones, rope, 7, kc, vc, NROT, eps=0.0)
    half = NROT // 2
    np.testing.assert_allclose(q7[:, :half] ** 2 + q7[:, half:NROT] ** 2, q0[:, :half] ** 2 + q0[:, half:NROT] ** 2,
                               rtol=1e-5)
    assert np.array_equal(q7[:, NROT:], q0[:, NROT:])
    # the pair (j, j + half) turns by pos * base^(-2j/n_rot): frequency 0 turns by one radian a position
    ang = np.arctan2(q7[0, half], q7[0, 0]) - np.arctan2(q0[0, half], q0[0, 0])
    assert np.isclose((ang - 7.0 + np.pi) % (2 * np.pi) - np.pi, 0.0, atol=1e-5)
    # q.k depends on the distance of the positions only
    w = 1.0 + 0.1 * rand(DH, 16)
    def qk(pq, pk):
        kc2, vc2 = np.zeros_like(kc), np.zeros_like(vc)
        q = OA.prep(qfull, kin, vin, w, w, rope, pq, kc2, vc2, NROT)
        OA.prep(qfull, kin, vin, w, w, rope, pk, kc2, vc2, NROT)
        return float(q[5].astype(np.float64) @ kc2[0, pk].astype(np.float64))
    assert np.isclose(qk(9, 4), qk(25, 20), rtol=1e-4) and not np.isclose(qk(9, 4), qk(9, 5), rtol=1e-3)
    # norm weights multiply elementwise (before the rotation)
    q_w = OA.prep(qfull, kin, vin, 2 * ones, ones, rope, 0, kc, vc, NROT, eps=0.0)
    np.testing.assert_allclose(q_w, 2 * q0, rtol=1e-6)


def test_library_rope_table(qk):
    """The library's host routine (float powf / cosf / sinf as the reference) against the oracle's
    float32 numpy table: a last-place difference of an angle of a few thousand radians moves its
    cosine by up to 3e-4."""
    got = qk.rope_table(4096, NROT, 1e7)
    want = OA.rope_table(4096, NROT, 1e7)
    assert got.shape == want.shape == (4096, 32, 2)
    assert np.max(np.abs(got - want)) < 1e-3
    assert np.array_equal(got[0], np.stack([np.ones(32), np.zeros(32)], -1).astype(np.float32))
    np.testing.assert_allclose(got[:, 0, 0], np.cos(np.arange(4096, dtype=np.float64)), atol=1e-6)
