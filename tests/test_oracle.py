"""Pins the CPU oracle (oracle/qk_oracle.c): against the reference's own header compiled in
this container (oracle/_ref, skipped where the reference tree is absent), against the
compiler-independent facts the formats fix, and against numpy float64 evaluations."""
import numpy as np
import pytest

QUANT = ["q8_0", "q6_k", "iq4_xs", "iq3_xxs"]


def tid(orc, name):
    return {"q8_0": orc.Q8_0, "q6_k": orc.Q6_K, "iq4_xs": orc.IQ4_XS, "iq3_xxs": orc.IQ3_XXS,
            "f16": orc.F16, "f32": orc.F32}[name]


@pytest.fixture(scope="module")
def ref(orc):
    r = orc.ref()
    if r is None:
        pytest.skip("oracle/_ref/libqkref.so not built (reference tree absent)")
    return r


# ---- half conversion ---------------------------------------------------------------------

def test_f16_to_f32_all_halves_vs_ieee(orc):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([orc.lib().qko_f16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.all(np.isnan(got[nan]))


def test_f16_to_f32_all_halves_vs_reference(orc, ref):
    for v in range(65536):
        a = np.float32(orc.lib().qko_f16_to_f32(v)).view(np.uint32)
        b = np.float32(ref.qkref_f16_to_f32(v)).view(np.uint32)
        assert a == b, hex(v)


def test_f32_to_f16_vs_reference_and_ieee(orc, ref, qk):
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(1e-3),
        rng.standard_normal(20000).astype(np.float32),
        (2.0 ** rng.uniform(-30, 20, 20000)).astype(np.float32) * rng.choice([-1, 1], 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65520.0, 1e10, -1e10, 2.0 ** -14, 2.0 ** -14 * 0.99999, 2.0 ** -15,
                  np.inf, -np.inf, 6.1e-5, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11], dtype=np.float32),
        # all halves exactly, and the midpoints between neighbouring halves (ties-to-even)
        np.arange(0x0400, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32),
    ])
    mids = np.arange(0x0400, 0x7BFF, dtype=np.uint16)
    mids = (mids.view(np.float16).astype(np.float64) + (mids + 1).view(np.float16).astype(np.float64)) / 2
    vals = np.concatenate([vals, mids.astype(np.float32)])
    got = np.array([orc.lib().qko_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    want_ref = np.array([ref.qkref_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want_ref)
    # the numpy recipe used by the synthetic generators is the same function
    assert np.array_equal(qk.synth.f32_to_f16_bits(vals), got)
    # and it is IEEE round-to-nearest-even wherever |v| >= 2^-14 and finite in half
    ok = (np.abs(vals) >= 2.0 ** -14) & (np.abs(vals) < 65520.0)
    with np.errstate(over="ignore"):
        ieee = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got[ok], ieee[ok])
    small = np.abs(vals) < 2.0 ** -14
    assert np.all((got[small] & 0x7FFF) == 0)


def test_f32_to_f16_nan_becomes_inf(orc):
    assert orc.lib().qko_f32_to_f16(float("nan")) & 0x7FFF == 0x7C00


# ---- tables --------------------------------------------------------------------------------

def test_sign_table_and_masks(orc, ref):
    for i in range(128):
        assert orc.lib().qko_ksign(i) == ref.qkref_ksigns(i)
        assert orc.lib().qko_ksign(i) == (i | ((bin(i).count("1") & 1) << 7))
    for j in range(8):
        assert ref.qkref_kmask(j) == 1 << j


def test_grid_bytes_are_codebook_magnitudes(orc):
    # every magnitude of every codeword is one of the eight IQ3 levels
    blk = np.zeros((256, 98), dtype=np.uint8)
    blk[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    blk[:, 2] = np.arange(256)  # first grid index of group 0 -> elements 0..3
    out = orc.dequant(orc.IQ3_XXS, blk, 256 * 256).reshape(256, 256)
    mags = out[:, :4] / 0.25  # db = 1*(0.5+0)*0.5
    assert set(np.unique(mags)) <= {4.0, 12.0, 20.0, 28.0, 36.0, 44.0, 52.0, 62.0}
    assert np.all(out[0, :8] == 1.0)  # codeword 0 = four 4s: d*0.25*4


def test_tables_vs_reference(orc, ref):
    blk = np.zeros((256, 98), dtype=np.uint8)
    blk[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    blk[:, 2] = np.arange(256)
    out = orc.dequant(orc.IQ3_XXS, blk, 256 * 256).reshape(256, 256)
    for i in range(256):
        cw = ref.qkref_iq3xxs_grid(i)
        assert [int(v * 4) for v in out[i, :4]] == [(cw >> (8 * j)) & 255 for j in range(4)]
    b4 = np.zeros((16, 136), dtype=np.uint8)
    b4[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    b4[:, 4:8] = 0x11   # low scale bits 1 -> ls = 1 | (0<<4) = 1 -> dl = 1-32 = -31
    for n in range(16):
        b4[n, 8:] = n | (n << 4)
    o4 = orc.dequant(orc.IQ4_XS, b4, 16 * 256).reshape(16, 256)
    for n in range(16):
        assert np.all(o4[n] == -31.0 * ref.qkref_iq4nl(n))


# ---- dequantisation --------------------------------------------------------------------------

@pytest.mark.parametrize("name", QUANT)
def test_block_sizes(orc, ref, name):
    t = tid(orc, name)
    be = 32 if name == "q8_0" else 256
    assert orc.row_bytes(t, be) == ref.qkref_block_bytes(t) == {"q8_0": 34, "q6_k": 210, "iq4_xs": 136, "iq3_xxs": 98}[name]
    assert orc.row_bytes(t, be + 1) == 0


@pytest.mark.parametrize("name", QUANT)
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_dequant_bitwise_vs_reference(orc, ref, qk, name, seed):
    t = tid(orc, name)
    be = 32 if name == "q8_0" else 256
    nb = 4096
    blocks = qk.synth.blocks_host(t, nb, seed)
    if seed == 2:  # fully random bytes, random (finite) halves as scales
        rng = np.random.default_rng(99)
        blocks = rng.integers(0, 256, size=blocks.shape, dtype=np.uint8)
        off = qk.synth.D_OFFSET[t]
        blocks[:, off + 1] &= 0x7B | 0x80  # keep the exponent below 31: no Inf/NaN scales
    a = orc.dequant(t, blocks, nb * be)
    b = orc.dequant(t, blocks, nb * be, use_ref=True)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_dequant_closed_forms(orc):
    one = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    # Q8_0 with d = 1: y = q
    b = np.zeros((1, 34), dtype=np.uint8)
    b[0, 0:2] = one
    q = np.arange(-16, 16, dtype=np.int8)
    b[0, 2:] = q.view(np.uint8)
    assert np.array_equal(orc.dequant(orc.Q8_0, b, 32), q.astype(np.float32))
    # Q6_K with ql = qh = 0: q = -32 everywhere, y = d*sc*(-32)
    b = np.zeros((1, 210), dtype=np.uint8)
    b[0, 192:208] = np.arange(1, 17, dtype=np.uint8)
    b[0, 208:210] = one
    y = orc.dequant(orc.Q6_K, b, 256)
    assert np.array_equal(y, np.repeat(np.arange(1, 17), 16).astype(np.float32) * -32.0)
    # Q6_K: one element at a time -- element e gets value (q-32) with q from the right bits
    for e in [0, 31, 32, 63, 64, 95, 96, 127, 128, 200, 255]:
        n, c, l = e >> 7, (e >> 5) & 3, e & 31
        b = np.zeros((1, 210), dtype=np.uint8)
        b[0, 192:208] = 1
        b[0, 208:210] = one
        b[0, 64 * n + 32 * (c & 1) + l] = (0x5 << 4) if c >= 2 else 0x5
        b[0, 128 + 32 * n + l] = 0x2 << (2 * c)
        y = orc.dequant(orc.Q6_K, b, 256)
        assert y[e] == (0x5 | (0x2 << 4)) - 32
        partner = e + 64 if c < 2 else e - 64   # shares the ql byte (other nibble = 0)
        others = np.delete(y, [e])
        assert np.all(others == -32.0), (e, partner)
    # IQ3_XXS with aux = 0, qs = 0: every weight = d*0.25*4 = d
    b = np.zeros((1, 98), dtype=np.uint8)
    b[0, 0:2] = np.frombuffer(np.float16(0.5).tobytes(), dtype=np.uint8)
    assert np.all(orc.dequant(orc.IQ3_XXS, b, 256) == 0.5)
    # IQ3_XXS signs: selector s for group l of block-group ib flips exactly the bits of ksign(s)
    b = np.zeros((1, 98), dtype=np.uint8)
    b[0, 0:2] = one
    aux = (0b0000011 << 7) | (0xF << 28)   # l = 1 gets selector 3 (even parity), scale 15
    b[0, 66 + 4 * 2: 66 + 4 * 2 + 4] = np.frombuffer(np.uint32(aux).tobytes(), dtype=np.uint8)  # ib = 2
    y = orc.dequant(orc.IQ3_XXS, b, 256)
    db = 1.0 * (0.5 + 15) * 0.5
    grp = y[64 + 8: 64 + 16]
    assert np.array_equal(grp, np.array([-1, -1, 1, 1, 1, 1, 1, 1], dtype=np.float32) * 4 * db)
    assert np.all(y[64:72] == 4 * db) and np.all(y[:64] == 1.0)


def test_f16_rows(orc):
    h = np.arange(0, 0x7C00, 7, dtype=np.uint16)
    y = orc.dequant(orc.F16, h.view(np.uint8), h.size)
    assert np.array_equal(y, h.view(np.float16).astype(np.float32))


# ---- dot products, argmax --------------------------------------------------------------------

@pytest.mark.parametrize("name", QUANT + ["f16", "f32"])
def test_gemv_vs_float64_matmul(orc, qk, name):
    t = tid(orc, name)
    M, K = 48, 1024
    W = qk.synth.tensor_host(t, M, K, seed=5)
    x = np.random.default_rng(6).standard_normal((3, K)).astype(np.float32)
    Wf = orc.dequant(t, W, M * K).reshape(M, K).astype(np.float64)
    want = (x.astype(np.float64) @ Wf.T)
    got = orc.gemv(t, W, x, M, K)
    assert np.allclose(got, want.astype(np.float32), rtol=2e-7, atol=0)
    assert orc.row_bytes(t, K) * M == W.size


def test_gemm_q8_0_vs_float64_matmul(orc, qk):
    M, K, N = 40, 256, 9
    W = qk.synth.tensor_host(orc.Q8_0, M, K, seed=7)
    X = np.random.default_rng(8).uniform(-1, 1, (N, K)).astype(np.float32)
    Wf = orc.dequant(orc.Q8_0, W, M * K).reshape(M, K).astype(np.float64)
    want = (X.astype(np.float64) @ Wf.T).astype(np.float32)
    got = orc.gemm_q8_0(W, X, M, K)
    assert got.shape == (N, M)
    assert np.allclose(got, want, rtol=2e-7, atol=0)


def test_argmax_first_occurrence(orc):
    rng = np.random.default_rng(3)
    for _ in range(50):
        v = rng.standard_normal(1000).astype(np.float32)
        assert orc.argmax(v) == int(np.argmax(v))
    v = np.zeros(100, dtype=np.float32)
    v[[17, 40, 99]] = 5.0
    assert orc.argmax(v) == 17


# ---- router ----------------------------------------------------------------------------------

def test_select_vs_numpy(orc):
    rng = np.random.default_rng(11)
    for _ in range(100):
        E, k = int(rng.choice([8, 64, 256, 512])), int(rng.choice([1, 2, 8, 10, 16]))
        k = min(k, E)
        logits = rng.standard_normal(E) * 3
        s = orc.select_f64(logits, k)
        order = np.argsort(-logits, kind="stable")[:k]
        assert list(s.ids[:k]) == list(order)
        w = np.exp(logits[order] - logits[order[0]])
        w /= w.sum()
        assert np.allclose(s.w[:k], w, rtol=1e-14)
        full = np.exp(logits - logits.max())
        full /= full.sum()
        assert np.allclose(s.w[:k], full[order] / full[order].sum(), rtol=1e-12)  # softmax then renormalise
        assert abs(sum(s.w[:k]) - 1) < 1e-12
        assert all(s.w[i] >= s.w[i + 1] for i in range(k - 1))
        if k < E:
            assert np.isclose(s.gap, logits[order[-1]] - np.sort(logits)[::-1][k])
        f = orc.select_f32(logits.astype(np.float32), k)
        assert list(f.ids[:k]) == list(np.argsort(-logits.astype(np.float32), kind="stable")[:k])
        assert np.allclose(f.w[:k], w, atol=1e-6)


def test_select_ties_and_nonfinite(orc):
    logits = np.zeros(256, dtype=np.float32)
    logits[[200, 3, 77]] = 1.0
    f = orc.select_f32(logits, 8)
    assert list(f.ids[:8]) == [3, 77, 200, 0, 1, 2, 4, 5]
    d = orc.select_f64(logits.astype(np.float64), 8)
    assert list(d.ids[:8]) == [3, 77, 200, 0, 1, 2, 4, 5]
    logits = np.full(256, np.nan, dtype=np.float32)
    logits[9] = np.inf
    logits[5] = -1.0
    f = orc.select_f32(logits, 8)
    assert f.ids[0] == 5 and all(i < 256 for i in f.ids[:8])
    assert np.isfinite(list(f.w[:8])).all()


# ---- fused MoE step ----------------------------------------------------------------------------

def dense_moe_f64(orc, h, x):
    """Dequantise everything, evaluate the layer in float64 with numpy."""
    H, F, E, k = h.n_embd, h.n_ff, h.n_expert, h.n_used
    x = x.astype(np.float64)
    logits = h.gate_inp.astype(np.float64) @ x
    order = np.argsort(-logits, kind="stable")[:k]
    w = np.exp(logits[order] - logits[order[0]])
    w /= w.sum()
    silu = lambda v: v / (1 + np.exp(-v))  # noqa: E731
    G = orc.dequant(h.gu_type, h.gate_exps, E * F * H).reshape(E, F, H).astype(np.float64)
    U = orc.dequant(h.gu_type, h.up_exps, E * F * H).reshape(E, F, H).astype(np.float64)
    D = orc.dequant(h.down_type, h.down_exps, E * H * F).reshape(E, H, F).astype(np.float64)
    y = np.zeros(H)
    for e, we in zip(order, w):
        hh = (silu(G[e] @ x) * (U[e] @ x)).astype(np.float32).astype(np.float64)
        y += we * (D[e] @ hh)
    Gs = orc.dequant(orc.Q8_0, h.gate_shexp, F * H).reshape(F, H).astype(np.float64)
    Us = orc.dequant(orc.Q8_0, h.up_shexp, F * H).reshape(F, H).astype(np.float64)
    Ds = orc.dequant(orc.Q8_0, h.down_shexp, H * F).reshape(H, F).astype(np.float64)
    hh = (silu(Gs @ x) * (Us @ x)).astype(np.float32).astype(np.float64)
    wsh = 1 / (1 + np.exp(-(h.gate_inp_shexp.astype(np.float64) @ x)))
    y += wsh * (Ds @ hh)
    return y, order, w, wsh


@pytest.mark.parametrize("down", ["iq4_xs", "q6_k"])
def test_moe_ref_vs_dense_float64(orc, qk, down):
    h = qk.synth.HostLayer(seed=21, n_embd=256, n_ff=256, n_expert=8, n_used=2, down_type=tid(orc, down),
                           d_scale=1e-2)
    x = np.random.default_rng(22).standard_normal(256).astype(np.float32)
    r = orc.moe_ref(h, x, want_h=True, want_logits=True)
    y, order, w, wsh = dense_moe_f64(orc, h, x)
    assert list(r["sel"].ids[:2]) == list(order)
    assert np.allclose(r["sel"].w[:2], w, rtol=1e-13)
    assert np.isclose(r["sel"].w_shared, wsh, rtol=1e-13)
    assert 0 < r["sel"].w_shared < 1
    # the reference adds each expert's float-rounded contribution into a float accumulator
    assert np.allclose(r["y"], y, rtol=0, atol=4e-7 * np.abs(y).max())
    assert r["h"].shape == (3, 256)


def test_moe_ref_all_experts_is_dense_softmax_mlp(orc, qk):
    h = qk.synth.HostLayer(seed=31, n_embd=256, n_ff=256, n_expert=4, n_used=4, d_scale=1e-2)
    x = np.random.default_rng(32).standard_normal(256).astype(np.float32)
    r = orc.moe_ref(h, x)
    logits = h.gate_inp.astype(np.float64) @ x.astype(np.float64)
    p = np.exp(logits - logits.max())
    p /= p.sum()
    got = np.zeros(4)
    got[list(r["sel"].ids[:4])] = list(r["sel"].w[:4])
    assert np.allclose(got, p, rtol=1e-13)


# ---- pair grouping -------------------------------------------------------------------------------

def test_group_pairs_vs_stable_sort(orc):
    rng = np.random.default_rng(41)
    for n_tokens, E, k in [(16, 256, 8), (128, 256, 8), (5, 8, 2), (1, 4, 4)]:
        sel = np.zeros((n_tokens, 40), dtype=np.uint32)
        for t in range(n_tokens):
            sel[t, :k] = rng.choice(E, size=k, replace=False)
        sel[0, 0] = E + 5  # out-of-range ids clamp to E-1
        offsets, pairs = orc.group_pairs(sel.view(np.uint8).reshape(n_tokens, 160), n_tokens, E, k)
        ids = np.minimum(sel[:, :k].reshape(-1), E - 1)
        order = np.argsort(ids, kind="stable")
        want_pairs = ((order // k) << 4) | (order % k)
        assert np.array_equal(pairs, want_pairs.astype(np.uint32))
        counts = np.bincount(ids, minlength=E)
        assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32))
        assert offsets[E] == n_tokens * k and np.all(np.diff(offsets.astype(np.int64)) >= 0)


# ---- acceptance metrics --------------------------------------------------------------------------

def test_metrics(orc):
    ref_ = np.array([1.0, -2.0, 0.0, 4.0], dtype=np.float32)
    got = ref_ + np.array([0.01, 0.0, 0.0005, 0.0], dtype=np.float32)
    rms = np.sqrt(np.mean(ref_.astype(np.float64) ** 2))
    floor = max(1e-3, 1e-3 * rms)
    want = max(0.01 / 1.0, 0.0005 / floor)
    assert np.isclose(orc.max_rel_err(got, ref_), want, rtol=1e-5)
    assert np.isclose(orc.max_err_over_rms(got, ref_), 0.01 / rms, rtol=1e-5)
    assert np.isclose(orc.rel_maxabs_err(got, ref_), 0.01 / 4.0, rtol=1e-5)
    assert orc.max_rel_err(np.array([np.nan], dtype=np.float32), np.array([1.0], dtype=np.float32)) == np.inf


# ---- layer glue -------------------------------------------------------------------------------

def _rms64(v, w, eps):
    v64 = v.astype(np.float64)
    return v64 / np.sqrt(np.mean(v64 * v64, axis=-1, keepdims=True) + eps) * w.astype(np.float64)


@pytest.mark.parametrize("n", [2048, 4096, 100, 7])
def test_add_rms_vs_float64(orc, n):
    rng = np.random.default_rng(n)
    a, b, c = (rng.standard_normal((3, n)).astype(np.float32) * np.float32(s) for s in (1.0, 0.3, 5.0))   # three rows each
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    eps = 1e-6
    # one, two and three inputs; the stored sum is numpy's float32 sum taken left to right
    for bb, cc in ((None, None), (b, None), (b, c)):
        v = a if bb is None else (a + bb if cc is None else (a + bb) + cc)
        assert v.dtype == np.float32
        s, xn = orc.add_rms(a, w, eps, b=bb, c=cc, want_sum=True)
        assert np.array_equal(s.view(np.uint32), v.view(np.uint32))
        want = _rms64(v, w, eps)
        assert np.max(np.abs(xn - want)) <= 2e-7 * np.max(np.abs(want))


def test_add_rms_invariants(orc):
    rng = np.random.default_rng(5)
    n = 2048
    a = rng.standard_normal((4, n)).astype(np.float32)
    ones = np.ones(n, dtype=np.float32)
    # unit weights: mean(xn^2) = ms / (ms + eps)
    for eps in (1e-6, 0.5):
        xn = orc.add_rms(a, ones, eps).astype(np.float64)
        ms = np.mean(a.astype(np.float64) ** 2, axis=1)
        assert np.allclose(np.mean(xn * xn, axis=1), ms / (ms + eps), rtol=1e-6)
    # eps = 0: scaling the input by a power of two changes nothing, bit for bit
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    x1, x2 = orc.add_rms(a, w, 0.0), orc.add_rms(a * np.float32(4.0), w, 0.0)
    assert np.array_equal(x1.view(np.uint32), x2.view(np.uint32))
    # a wrong operand order or a dropped input shows: b enters the norm
    b = rng.standard_normal((4, n)).astype(np.float32)
    assert not np.allclose(orc.add_rms(a, w, 1e-6, b=b), orc.add_rms(a, w, 1e-6))
    # the weight multiplies the output elementwise
    assert np.allclose(orc.add_rms(a, w, 1e-6), orc.add_rms(a, ones, 1e-6) * w, rtol=1e-6)


def test_embed_is_dequant_of_the_chosen_rows(orc, qk):
    rng = np.random.default_rng(9)
    for t, be in ((qk.Q6_K, 256), (qk.Q8_0, 32)):
        V, K = 50, 512
        W = qk.synth.tensor_host(t, V, K, seed=3)
        rb = orc.row_bytes(t, K)
        ids = rng.integers(0, V, 12).astype(np.uint32)
        got = orc.embed(t, W, V, K, ids, idx=2, per_req=3, rows=4)
        for r in range(4):
            tok = ids[2 + 3 * r]
            want = orc.dequant(t, W.reshape(-1)[tok * rb:(tok + 1) * rb], K)
            assert np.array_equal(got[r].view(np.uint32), want.view(np.uint32))
    with pytest.raises(ValueError):
        orc.embed(qk.Q8_0, W, V, K, np.array([V], dtype=np.uint32), 0, 1, 1)


def test_threaded_row_loops_give_the_single_thread_bits(qk, orc):
    """The all-cores CPU baseline of the benchmark runs the oracle's row loops on several host
    threads; every output element is still computed by one thread with the same scalar code, so
    the results are the single-threaded ones bit for bit (ragged splits included)."""
    rng = np.random.default_rng(21)
    for t, name in ((orc.Q8_0, "q8_0"), (orc.Q6_K, "q6_k"), (orc.IQ4_XS, "iq4_xs"), (orc.IQ3_XXS, "iq3_xxs")):
        W = qk.synth.tensor_host(t, 37, 512, seed=3)
        x = rng.standard_normal((3, 512)).astype(np.float32)
        for nt in (2, 5, 64):
            assert np.array_equal(orc.gemv(t, W, x, 37, 512, threads=nt).view(np.uint32),
                                  orc.gemv(t, W, x, 37, 512).view(np.uint32)), (name, nt)
            assert np.array_equal(orc.gemv(t, W, x[0], 37, 512, threads=nt).view(np.uint32),
                                  orc.gemv(t, W, x[0], 37, 512).view(np.uint32)), (name, nt)
    W = qk.synth.tensor_host(orc.Q8_0, 19, 256, seed=4)
    X = rng.standard_normal((5, 256)).astype(np.float32)
    assert np.array_equal(orc.gemm_q8_0(W, X, 19, 256, threads=3).view(np.uint32), orc.gemm_q8_0(W, X, 19, 256).view(np.uint32))
    for down in (orc.IQ4_XS, orc.Q6_K):
        hl = qk.synth.HostLayer(seed=8, n_ff=256, n_expert=8, n_used=3, down_type=down)
        X = rng.standard_normal((4, 2048)).astype(np.float32)
        want = np.stack([orc.moe_ref(hl, X[r])["y"] for r in range(4)])
        assert np.array_equal(orc.moe_ref_threads(hl, X, 3).view(np.uint32), want.view(np.uint32))
        assert np.array_equal(orc.moe_ref_threads(hl, X[:1], 7).view(np.uint32), want[:1].view(np.uint32))
