"""The gated-DeltaNet decode step on the GPU (qkk_dn_ab, qkk_dn_conv, qkk_dn_step) against the
restated CPU mirror in oracle/qk_oracle_deltanet.py, through the C ABI.  Tolerance 1e-3 relative
max-abs as for the other fp32 kernels; the conv window is a copy and must be bit-exact."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import qk_oracle_deltanet as OD  # noqa: E402

pytestmark = pytest.mark.gpu

DS, HK, HV, NE = 128, 16, 32, 2048      # the reference's shape (src/main.cpp:3085)
CH, QK = (2 * HK + HV) * DS, 2 * HK * DS
F = np.float32
TOL = 1e-3


def rel(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))


def rand(shape, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(F)


class Weights:
    def __init__(self, seed, hk=HK, hv=HV, ne=NE):
        self.hk, self.hv, self.ch, self.qk = hk, hv, (2 * hk + hv) * DS, 2 * hk * DS
        self.alpha_w, self.beta_w = rand((hv, ne), seed, 0.03), rand((hv, ne), seed + 1, 0.03)
        self.dt_bias, self.a_vec = rand(hv, seed + 2), -np.abs(rand(hv, seed + 3)) - F(0.05)
        self.ker = rand((self.ch, 4), seed + 4, 0.5)
        self.norm_w = (1 + 0.1 * rand(DS, seed + 5)).astype(F)


def run_tokens(qk, dev, w, n_slots, n_tok, seed, kdiv=0, ne=NE):
    """n_tok decode steps of n_slots independent slots on the GPU and in the oracle; returns the
    worst relative errors per quantity and the final states."""
    import torch
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    rng = np.random.default_rng(seed)
    st = rng.standard_normal((n_slots, w.ch, 3)).astype(F)
    S = (rng.standard_normal((n_slots, w.hv, DS, DS)) * 0.1).astype(F)          # row-major (row j, column i)
    std, Sd = up(st), up(np.ascontiguousarray(S.transpose(0, 1, 3, 2)))          # device: column-major per head
    wd = {k: up(getattr(w, k)) for k in ("alpha_w", "beta_w", "dt_bias", "a_vec", "ker", "norm_w")}
    worst = dict(gb=0.0, conv=0.0, att=0.0)
    for t in range(n_tok):
        x = rng.standard_normal((n_slots, ne)).astype(F)
        qkv = rng.standard_normal((n_slots, w.ch)).astype(F)
        z = rng.standard_normal((n_slots, w.hv * DS)).astype(F)
        gb = qk.dn_ab(up(x), wd["alpha_w"], wd["beta_w"], wd["dt_bias"], wd["a_vec"])
        st_before = std.clone()
        conv = qk.dn_conv(std, up(qkv), wd["ker"], w.qk)
        # the two in one launch: the same bits, the same window
        gb2, conv2 = qk.dn_ab_conv(up(x), wd["alpha_w"], wd["beta_w"], wd["dt_bias"], wd["a_vec"], st_before, up(qkv), wd["ker"], w.qk)
        assert torch.equal(gb2, gb) and torch.equal(conv2, conv) and torch.equal(st_before, std)
        att = qk.dn_step(conv, gb, Sd, wd["norm_w"], up(z), w.hk, w.hv, kdiv=kdiv)
        torch.cuda.synchronize()
        gb, conv, att = gb.cpu().numpy(), conv.cpu().numpy(), att.cpu().numpy()
        for s in range(n_slots):
            g, b = OD.ab(x[s], w.alpha_w, w.beta_w, w.dt_bias, w.a_vec)
            c = OD.conv(st[s], qkv[s], w.ker, DS, w.qk)
            a = OD.step(c, g, b, S[s], w.norm_w, z[s], w.hk, w.hv, kdiv=kdiv)
            worst["gb"] = max(worst["gb"], rel(gb[s], np.concatenate([g, b])))
            worst["conv"] = max(worst["conv"], rel(conv[s], c))
            worst["att"] = max(worst["att"], rel(att[s], a))
    return worst, std.cpu().numpy(), Sd.cpu().numpy().transpose(0, 1, 3, 2), st, S


@pytest.mark.parametrize("n_slots,n_tok,kdiv", [(1, 6, 0), (3, 4, 2), (16, 2, 0)])
def test_deltanet_steps_match_the_cpu_mirror(qk, dev, n_slots, n_tok, kdiv):
    print(f"[case] deltanet slots={n_slots} tokens={n_tok} kdiv={kdiv}", flush=True)
    worst, st_gpu, S_gpu, st, S = run_tokens(qk, dev, Weights(7), n_slots, n_tok, seed=n_slots + 10 * kdiv, kdiv=kdiv)
    assert worst["gb"] <= 1e-5 and worst["conv"] <= 1e-5 and worst["att"] <= TOL, worst
    assert np.array_equal(st_gpu, st)            # the conv window holds copies of the inputs
    assert rel(S_gpu, S) <= TOL                  # the states after all tokens


def test_deltanet_ab_with_the_norm_in_front(qk, orc, dev, unrun_form):
    """qkk_dn_ab_conv_norm: x is the residual row; decay and write strength come out as from the norm
    launch followed by qkk_dn_ab_conv (to rounding) and match the oracle on the oracle's normalised row;
    the conv half is untouched (bit for bit)."""
    import torch
    print("[case] deltanet ab with the norm in front", flush=True)
    w = Weights(3)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    rng = np.random.default_rng(9)
    for n in (1, 3):
        x = (rng.standard_normal((n, NE)) * 4.0).astype(F)
        nw = rng.uniform(0.5, 1.5, NE).astype(F)
        qkv, st = rng.standard_normal((n, w.ch)).astype(F), rng.standard_normal((n, w.ch, 3)).astype(F)
        wd = [up(getattr(w, k)) for k in ("alpha_w", "beta_w", "dt_bias", "a_vec")]
        st1, st2 = up(st.copy()), up(st.copy())   # two buffers also where up() does not copy
        gb, conv = qk.dn_ab_conv(up(x), *wd, st1, up(qkv), up(w.ker), w.qk, w_norm=up(nw))
        gb0, conv0 = qk.dn_ab_conv(qk.rmsnorm(up(x), up(nw)), *wd, st2, up(qkv), up(w.ker), w.qk)
        torch.cuda.synchronize()
        assert torch.equal(conv, conv0) and torch.equal(st1, st2)
        assert rel(gb.cpu().numpy(), gb0.cpu().numpy().astype(np.float64)) <= 1e-5
        for s in range(n):
            g, b = OD.ab(orc.add_rms(x[s], nw, 1e-6), w.alpha_w, w.beta_w, w.dt_bias, w.a_vec)
            assert rel(gb.cpu().numpy()[s], np.concatenate([g, b])) <= TOL


@pytest.mark.parametrize("n_slots,kdiv,norm", [(1, 0, False), (1, 2, True), (3, 0, True), (16, 2, False)])
def test_deltanet_one_launch_step(qk, orc, dev, unrun_form, n_slots, kdiv, norm):
    """qkk_dn_step_fused (ab + conv + step of the two value heads of a key head in one workgroup) against
    the two launches it replaces: the same arithmetic in the same order, so attention rows, conv window and
    state come out bit for bit the same, over several tokens; the first token also against the oracle."""
    import torch
    print(f"[case] deltanet one-launch step slots={n_slots} kdiv={kdiv} norm={norm}", flush=True)
    w = Weights(11)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    rng = np.random.default_rng(n_slots + kdiv)
    st = rng.standard_normal((n_slots, w.ch, 3)).astype(F)
    S = (rng.standard_normal((n_slots, w.hv, DS, DS)) * 0.1).astype(F)
    St = np.ascontiguousarray(S.transpose(0, 1, 3, 2))                     # device layout: column-major per head
    st_a, st_b, S_a, S_b = up(st.copy()), up(st.copy()), up(St.copy()), up(St.copy())
    wd = {k: up(getattr(w, k)) for k in ("alpha_w", "beta_w", "dt_bias", "a_vec", "ker", "norm_w")}
    nw = rng.uniform(0.5, 1.5, NE).astype(F)
    nwd = up(nw) if norm else None
    for tkn in range(3):
        x = (rng.standard_normal((n_slots, NE)) * 2.0).astype(F)
        qkv = rng.standard_normal((n_slots, w.ch)).astype(F)
        z = rng.standard_normal((n_slots, w.hv * DS)).astype(F)
        xd, qd, zd = up(x), up(qkv), up(z)
        gb, conv = qk.dn_ab_conv(xd, wd["alpha_w"], wd["beta_w"], wd["dt_bias"], wd["a_vec"], st_a, qd, wd["ker"], w.qk, w_norm=nwd)
        att_a = qk.dn_step(conv, gb, S_a, wd["norm_w"], zd, w.hk, w.hv, kdiv=kdiv)
        att_b = qk.dn_step_fused(xd, wd["alpha_w"], wd["beta_w"], wd["dt_bias"], wd["a_vec"], st_b, qd, wd["ker"], S_b,
                                 wd["norm_w"], zd, w.hk, w.hv, kdiv=kdiv, w_norm=nwd)
        torch.cuda.synchronize()
        assert torch.equal(att_b, att_a) and torch.equal(st_b, st_a) and torch.equal(S_b, S_a), tkn
        if tkn == 0:
            for s_ in range(n_slots):
                xs = orc.add_rms(x[s_], nw, 1e-6) if norm else x[s_]
                g, b = OD.ab(xs, w.alpha_w, w.beta_w, w.dt_bias, w.a_vec)
                c = OD.conv(st[s_].copy(), qkv[s_], w.ker, DS, w.qk)
                a = OD.step(c, g, b, S[s_].copy(), w.norm_w, z[s_], w.hk, w.hv, kdiv=kdiv)
                assert rel(att_b.cpu().numpy()[s_], a) <= TOL, s_
    with pytest.raises(qk.QkError):   # three value heads per key head: not this kernel's shape
        qk.dn_step_fused(xd, wd["alpha_w"], wd["beta_w"], wd["dt_bias"], wd["a_vec"], st_b, qd, wd["ker"], S_b, wd["norm_w"], zd,
                         w.hk, w.hv + w.hk, kdiv=kdiv)


def test_deltanet_other_shapes(qk, dev):
    """Fewer heads (1 key head for 2 value heads, both pairings) and n_embd = 4096."""
    print("[case] deltanet other shapes", flush=True)
    for hk, hv, kdiv, ne in ((1, 2, 0, 2048), (1, 2, 2, 2048), (4, 8, 2, 4096), (3, 3, 0, 2048)):
        worst, st_gpu, S_gpu, st, S = run_tokens(qk, dev, Weights(9, hk, hv, ne), 2, 3, seed=hk + hv, kdiv=kdiv, ne=ne)
        assert worst["gb"] <= 1e-5 and worst["conv"] <= 1e-5 and worst["att"] <= TOL, (hk, hv, kdiv, worst)
        assert np.array_equal(st_gpu, st) and rel(S_gpu, S) <= TOL


def test_deltanet_long_run_stays_on_the_oracle(qk, dev):
    """Sixty tokens on one slot: the recurrent state does not drift away from the mirror."""
    print("[case] deltanet sixty tokens", flush=True)
    worst, _, S_gpu, _, S = run_tokens(qk, dev, Weights(11, 2, 4), 1, 60, seed=5)
    assert worst["att"] <= TOL and rel(S_gpu, S) <= TOL, worst


def test_deltanet_argument_checks(qk, dev):
    import torch
    z = lambda *s: torch.zeros(s, device=dev)
    with pytest.raises(qk.QkError) as e:      # n_embd
        qk.dn_ab(z(1, 1024), z(HV, 1024), z(HV, 1024), z(HV), z(HV))
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:      # channels not whole heads
        qk.dn_conv(z(1, 200, 3), z(1, 200), z(200, 4), 128)
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:      # state size
        qk.dn_step(z(1, CH), z(1, 2 * HV), z(1, HV, 64, 64), z(64), z(1, HV * 64), HK, HV, d_state=64)
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:      # pairing beyond the key heads
        qk.dn_step(z(1, (2 * 2 + 8) * DS), z(1, 16), z(1, 8, DS, DS), z(DS), z(1, 8 * DS), 2, 8, kdiv=2)
    assert e.value.code == -2


@pytest.mark.parametrize("n_pos,kdiv", [(1, 0), (2, 0), (16, 0), (17, 2), (37, 2), (128, 0), (1000, 2)])
def test_deltanet_sequence_forms_equal_the_steps(qk, dev, n_pos, kdiv):
    """qkk_dn_conv_seq / qkk_dn_step_seq over n_pos consecutive positions of one slot (a state of
    earlier positions already in place): the outputs and the final window / state of n_pos calls of
    the one-position kernels, and the CPU mirror's within tolerance."""
    import torch
    print(f"[case] deltanet sequence n_pos={n_pos} kdiv={kdiv}", flush=True)
    w = Weights(23)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    rng = np.random.default_rng(n_pos)
    st = rng.standard_normal((1, w.ch, 3)).astype(F)
    S = (rng.standard_normal((1, w.hv, DS, DS)) * 0.1).astype(F)
    qkv = rng.standard_normal((n_pos, w.ch)).astype(F)
    z = rng.standard_normal((n_pos, w.hv * DS)).astype(F)
    gb = np.concatenate([-np.abs(rng.standard_normal((n_pos, w.hv))) * 0.3, rng.random((n_pos, w.hv))], axis=1).astype(F)
    ker, nw = up(w.ker), up(w.norm_w)
    # position by position
    st1, S1 = up(st), up(np.ascontiguousarray(S.transpose(0, 1, 3, 2)))
    conv1, att1 = [], []
    for t in range(n_pos):
        c = qk.dn_conv(st1, up(qkv[t:t + 1]), ker, w.qk)
        conv1.append(c)
        att1.append(qk.dn_step(c, up(gb[t:t + 1]), S1, nw, up(z[t:t + 1]), w.hk, w.hv, kdiv=kdiv))
    # all positions in one launch each
    st2, S2 = up(st), up(np.ascontiguousarray(S.transpose(0, 1, 3, 2)))
    conv2 = qk.dn_conv(st2, up(qkv), ker, w.qk, seq=True)
    att2 = qk.dn_step(conv2, up(gb), S2, nw, up(z), w.hk, w.hv, kdiv=kdiv, seq=True)
    torch.cuda.synchronize()
    conv1, att1 = torch.cat(conv1).cpu().numpy(), torch.cat(att1).cpu().numpy()
    conv2, att2 = conv2.cpu().numpy(), att2.cpu().numpy()
    assert np.array_equal(st1.cpu().numpy(), st2.cpu().numpy())
    assert rel(conv2, conv1) <= 1e-6 and rel(att2, att1) <= 1e-5, (rel(conv2, conv1), rel(att2, att1))
    assert rel(S2.cpu().numpy(), S1.cpu().numpy()) <= 1e-5
    print(f"[info] sequence vs steps: conv {rel(conv2, conv1):.1e} att {rel(att2, att1):.1e}", flush=True)
    if n_pos <= 37:   # and the CPU mirror
        so, So = st[0].copy(), S[0].copy()
        for t in range(n_pos):
            c = OD.conv(so, qkv[t], w.ker, DS, w.qk)
            a = OD.step(c, gb[t, :w.hv], gb[t, w.hv:], So, w.norm_w, z[t], w.hk, w.hv, kdiv=kdiv)
            assert rel(conv2[t], c) <= 1e-5 and rel(att2[t], a) <= TOL, t
        assert rel(S2.cpu().numpy()[0].transpose(0, 2, 1), So) <= TOL


def test_deltanet_sequence_argument_checks(qk, dev):
    import torch
    w = Weights(3)
    z = lambda *s: torch.zeros(s, dtype=torch.float32, device=dev)
    with pytest.raises(ValueError):   # a state of two slots is not a sequence's
        qk.dn_step(z(4, w.ch), z(4, 2 * w.hv), z(2, w.hv, DS, DS), z(DS), z(4, w.hv * DS), w.hk, w.hv, seq=True)
    with pytest.raises(qk.QkError):
        qk.dn_step(z(4, w.ch), z(4, 2 * w.hv), z(1, w.hv, 64, 64), z(64), z(4, w.hv * 64), w.hk, w.hv, d_state=64, seq=True)
