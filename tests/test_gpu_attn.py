"""The full-attention decode step on the GPU (qkk_attn_prep, qkk_attn_decode) against the restated
CPU mirror in oracle/qk_oracle_attn.py, through the C ABI.  Tolerance 1e-3 relative max-abs, as for
the other fp32 kernels (accumulation order differs); cache rows bit-exact where they are copies."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import qk_oracle_attn as OA  # noqa: E402

pytestmark = pytest.mark.gpu

HQ, HKV, DH, NROT = 16, 2, 256, 64
TOL = 1e-3


def rel(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))


def run_slots(qk, dev, tmax, positions, seed, hq=HQ, hkv=HKV):
    """Caches filled with random rows below each slot's position, one prep + decode at the
    positions; returns (gpu outputs, oracle outputs)."""
    import torch
    rng = np.random.default_rng(seed)
    n = len(positions)
    kc = np.zeros((n, hkv, tmax, DH), np.float32)
    vc = np.zeros((n, hkv, tmax, DH), np.float32)
    for s, p in enumerate(positions):
        kc[s, :, :p] = rng.standard_normal((hkv, p, DH))
        vc[s, :, :p] = rng.standard_normal((hkv, p, DH))
    qfull = rng.standard_normal((n, hq, 2 * DH)).astype(np.float32) * 2
    kin = rng.standard_normal((n, hkv, DH)).astype(np.float32)
    vin = rng.standard_normal((n, hkv, DH)).astype(np.float32)
    qn = (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32)
    kn = (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32)
    rope = OA.rope_table(tmax, NROT)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    kcd, vcd, qfd = up(kc), up(vc), up(qfull)
    pos = torch.tensor(positions, dtype=torch.int32, device=dev)
    qhat = qk.attn_prep(qfd, up(kin), up(vin), up(qn), up(kn), up(rope), pos, kcd, vcd, NROT)
    ws = torch.empty(qk.attn_workspace_bytes(n, hq), dtype=torch.uint8, device=dev)
    att = qk.attn_decode(qhat, kcd, vcd, qfd, pos, ws)
    torch.cuda.synchronize()
    want_q, want_att = [], []
    for s, p in enumerate(positions):
        want_q.append(OA.prep(qfull[s], kin[s], vin[s], qn, kn, rope, p, kc[s], vc[s], NROT))
        want_att.append(OA.attend(want_q[-1], kc[s], vc[s], qfull[s], p))
    return dict(qhat=qhat.cpu().numpy(), att=att.cpu().numpy(), kc=kcd.cpu().numpy(), vc=vcd.cpu().numpy(),
                want_q=np.stack(want_q), want_att=np.stack(want_att), want_kc=kc, want_vc=vc, vin=vin)


@pytest.mark.parametrize("tmax,positions", [
    (128, [0]), (128, [1]), (128, [63]), (128, [64]), (128, [127]),          # one key, range edges, last position
    (100, [0, 99, 50, 2]),                                                     # ranges of 2 positions, several slots
    (4096, [4095, 0, 1000, 64, 63, 65, 2047]),                                 # the reference's server context
    (520, [519, 130, 9]),                                                      # ranges of 9: tiles end inside a range
])
def test_attention_decode_matches_the_cpu_mirror(qk, dev, tmax, positions):
    print(f"[case] attention tmax={tmax} positions={positions}", flush=True)
    r = run_slots(qk, dev, tmax, positions, seed=tmax + len(positions))
    assert rel(r["qhat"], r["want_q"]) <= 1e-5
    for s, p in enumerate(positions):
        assert rel(r["kc"][s, :, p], r["want_kc"][s, :, p]) <= 1e-5           # normalised, rotated key row
        assert np.array_equal(r["vc"][s, :, p], r["vin"][s])                  # value row: a copy
        keep = np.ones(r["kc"].shape[2], bool)
        keep[p] = False
        assert np.array_equal(r["kc"][s][:, keep], r["want_kc"][s][:, keep])  # nothing else written
        assert np.array_equal(r["vc"][s][:, keep], r["want_vc"][s][:, keep])
    assert rel(r["att"], r["want_att"]) <= TOL


def test_attention_long_context_and_other_head_counts(qk, dev):
    """8192 positions (ranges of 128 = two tiles); 8 query heads on one KV head; 4 on 4."""
    print("[case] attention long context, other head counts", flush=True)
    r = run_slots(qk, dev, 8192, [8191, 4100], seed=3)
    assert rel(r["att"], r["want_att"]) <= TOL
    for hq, hkv in ((8, 1), (4, 4), (6, 2)):
        r = run_slots(qk, dev, 256, [200, 7], seed=hq, hq=hq, hkv=hkv)
        assert rel(r["qhat"], r["want_q"]) <= 1e-5 and rel(r["att"], r["want_att"]) <= TOL


def test_attention_generation_loop(qk, dev):
    """Tokens appended one by one: every step's output against the oracle run on the same inputs,
    with the cache the kernels built themselves."""
    import torch
    print("[case] attention generation loop", flush=True)
    rng = np.random.default_rng(8)
    tmax, steps = 96, 70
    rope = OA.rope_table(tmax, NROT)
    kc, vc = np.zeros((HKV, tmax, DH), np.float32), np.zeros((HKV, tmax, DH), np.float32)
    ones = np.ones(DH, np.float32)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    kcd, vcd = up(kc[None]), up(vc[None])
    roped, onesd = up(rope), up(ones)
    ws = torch.empty(qk.attn_workspace_bytes(1, HQ), dtype=torch.uint8, device=dev)
    pos = torch.zeros(1, dtype=torch.int32, device=dev)
    for p in range(steps):
        qfull = rng.standard_normal((HQ, 2 * DH)).astype(np.float32)
        kin, vin = rng.standard_normal((HKV, DH)).astype(np.float32), rng.standard_normal((HKV, DH)).astype(np.float32)
        pos.fill_(p)
        qfd = up(qfull[None])
        qhat = qk.attn_prep(qfd, up(kin[None]), up(vin[None]), onesd, onesd, roped, pos, kcd, vcd, NROT)
        att = qk.attn_decode(qhat, kcd, vcd, qfd, pos, ws).cpu().numpy()[0]
        want = OA.attend(OA.prep(qfull, kin, vin, ones, ones, rope, p, kc, vc, NROT), kc, vc, qfull, p)
        assert rel(att, want) <= TOL, p
    assert rel(kcd.cpu().numpy()[0], kc) <= 1e-5 and np.array_equal(vcd.cpu().numpy()[0], vc)


def test_attention_argument_checks(qk, dev):
    import torch
    z = lambda *s: torch.zeros(s, device=dev)
    pos = torch.zeros(1, dtype=torch.int32, device=dev)
    rope = torch.from_numpy(OA.rope_table(64, NROT)).to(dev)
    ws = torch.empty(qk.attn_workspace_bytes(1, HQ), dtype=torch.uint8, device=dev)
    with pytest.raises(qk.QkError) as e:   # head size
        qk.attn_prep(z(1, HQ, 256), z(1, HKV, 128), z(1, HKV, 128), z(128), z(128), rope, pos, z(1, HKV, 64, 128),
                     z(1, HKV, 64, 128), NROT)
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:   # 16 heads on 3 KV heads
        qk.attn_decode(z(1, HQ, DH), z(1, 3, 64, DH), z(1, 3, 64, DH), z(1, HQ, 2 * DH), pos, ws)
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:   # workspace too small
        qk.attn_decode(z(1, HQ, DH), z(1, HKV, 64, DH), z(1, HKV, 64, DH), z(1, HQ, 2 * DH), pos, ws[:1024])
    assert e.value.code == -5
    # a position beyond the cache is clamped to the last row, not followed
    big = torch.tensor([10 ** 9], dtype=torch.int32, device=dev)
    kc, vc = z(1, HKV, 64, DH), z(1, HKV, 64, DH)
    qk.attn_prep(z(1, HQ, 2 * DH) + 1, z(1, HKV, DH) + 1, z(1, HKV, DH) + 3, z(DH) + 1, z(DH) + 1, rope, big, kc, vc, NROT)
    torch.cuda.synchronize()
    assert float(vc[0, 0, 63, 0]) == 3.0 and float(vc[0, :, :63].abs().max()) == 0.0


@pytest.mark.parametrize("tmax,base,n_pos", [(96, 0, 1), (96, 0, 70), (96, 5, 33), (300, 150, 128), (4096, 3000, 40), (4096, 3050, 1023)])
def test_attention_sequence_forms_equal_the_steps(qk, dev, tmax, base, n_pos):
    """qkk_attn_prep_seq / qkk_attn_seq over n_pos consecutive positions of one slot whose cache
    already holds `base` rows: row t sees the cache rows 0..base+t.  Against the decode-step entry
    points called position by position (the same kernels; the number of position ranges depends on
    the row count, so the sums are folded in another order) and, for the shorter cases, the CPU
    mirror."""
    import torch
    print(f"[case] attention sequence tmax={tmax} base={base} n_pos={n_pos}", flush=True)
    rng = np.random.default_rng(tmax + n_pos)
    rope = OA.rope_table(tmax, NROT)
    kc, vc = np.zeros((HKV, tmax, DH), np.float32), np.zeros((HKV, tmax, DH), np.float32)
    kc[:, :base], vc[:, :base] = rng.standard_normal((HKV, base, DH)), rng.standard_normal((HKV, base, DH))
    qn, kn = (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32), (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32)
    qfull = rng.standard_normal((n_pos, HQ, 2 * DH)).astype(np.float32)
    kin, vin = rng.standard_normal((n_pos, HKV, DH)).astype(np.float32), rng.standard_normal((n_pos, HKV, DH)).astype(np.float32)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    roped, qnd, knd = up(rope), up(qn), up(kn)
    qfd, kind, vind = up(qfull), up(kin), up(vin)
    pos = torch.arange(base, base + n_pos, dtype=torch.int32, device=dev)
    # position by position
    k1, v1 = up(kc[None]), up(vc[None])
    ws1 = torch.empty(qk.attn_workspace_bytes(1, HQ), dtype=torch.uint8, device=dev)
    att1 = []
    for t in range(n_pos):
        qh = qk.attn_prep(qfd[t:t + 1], kind[t:t + 1], vind[t:t + 1], qnd, knd, roped, pos[t:t + 1], k1, v1, NROT)
        att1.append(qk.attn_decode(qh, k1, v1, qfd[t:t + 1], pos[t:t + 1], ws1))
    att1 = torch.cat(att1).cpu().numpy()
    # one launch per kernel
    k2, v2 = up(kc[None]), up(vc[None])
    ws2 = torch.empty(qk.attn_workspace_bytes(n_pos, HQ), dtype=torch.uint8, device=dev)
    qh2 = qk.attn_prep(qfd, kind, vind, qnd, knd, roped, pos, k2, v2, NROT, seq=True)
    att2 = qk.attn_decode(qh2, k2, v2, qfd, pos, ws2, seq=True).cpu().numpy()
    assert np.array_equal(k1.cpu().numpy(), k2.cpu().numpy()) and np.array_equal(v1.cpu().numpy(), v2.cpu().numpy())
    assert rel(att2, att1) <= 1e-5, rel(att2, att1)   # the range count differs with the row count: not bitwise
    if n_pos <= 70:
        for t in range(n_pos):
            want = OA.attend(OA.prep(qfull[t], kin[t], vin[t], qn, kn, rope, base + t, kc, vc, NROT), kc, vc, qfull[t], base + t)
            assert rel(att2[t], want) <= TOL, t


@pytest.mark.parametrize("hq,hkv,base,n_pos", [(16, 2, 0, 16), (16, 2, 61, 37), (8, 1, 3, 19), (4, 4, 10, 5), (6, 2, 130, 48),
                                                (2, 2, 0, 3)])
def test_attention_blocks_of_sixteen_rows(qk, dev, unrun_form, hq, hkv, base, n_pos):
    """With the "attn_block" switch three or more consecutive rows go through the kernel that takes sixteen rows and four query heads
    per workgroup (scores and values on the matrix cores): against the CPU mirror row by row, for head
    counts that fill a workgroup's four waves, leave some idle (2, 1 or 3 heads per KV head) or need two
    workgroups per KV head (8), block counts with a ragged last block, and caches that already hold rows."""
    import torch
    print(f"[case] attention blocks hq={hq} hkv={hkv} base={base} n_pos={n_pos}", flush=True)
    tmax = 256
    rng = np.random.default_rng(hq * 100 + n_pos)
    rope = OA.rope_table(tmax, NROT)
    kc, vc = np.zeros((hkv, tmax, DH), np.float32), np.zeros((hkv, tmax, DH), np.float32)
    kc[:, :base], vc[:, :base] = rng.standard_normal((hkv, base, DH)), rng.standard_normal((hkv, base, DH))
    qn, kn = (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32), (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32)
    qfull = (rng.standard_normal((n_pos, hq, 2 * DH)) * 2).astype(np.float32)
    kin, vin = rng.standard_normal((n_pos, hkv, DH)).astype(np.float32), rng.standard_normal((n_pos, hkv, DH)).astype(np.float32)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    kd, vd, qfd = up(kc[None].copy()), up(vc[None].copy()), up(qfull)
    pos = torch.arange(base, base + n_pos, dtype=torch.int32, device=dev)
    ws = torch.empty(qk.attn_workspace_bytes(n_pos, hq), dtype=torch.uint8, device=dev)
    qh = qk.attn_prep(qfd, up(kin), up(vin), up(qn), up(kn), up(rope), pos, kd, vd, NROT, seq=True)
    with qk.option("attn_block", 1):
        att = qk.attn_decode(qh, kd, vd, qfd, pos, ws, seq=True).cpu().numpy()
    for t in range(n_pos):
        want = OA.attend(OA.prep(qfull[t], kin[t], vin[t], qn, kn, rope, base + t, kc, vc, NROT), kc, vc, qfull[t], base + t)
        assert rel(att[t], want) <= TOL, t


def test_attention_sequence_argument_checks(qk, dev):
    import torch
    z = lambda *s: torch.zeros(s, device=dev)
    pos = torch.zeros(4, dtype=torch.int32, device=dev)
    ws = torch.empty(qk.attn_workspace_bytes(1, HQ), dtype=torch.uint8, device=dev)
    with pytest.raises(ValueError):        # four rows of a sequence share one cache
        qk.attn_decode(z(4, HQ, DH), z(4, HKV, 64, DH), z(4, HKV, 64, DH), z(4, HQ, 2 * DH), pos, ws, seq=True)
    with pytest.raises(qk.QkError) as e:   # a workspace for one row
        qk.attn_decode(z(4, HQ, DH), z(1, HKV, 64, DH), z(1, HKV, 64, DH), z(4, HQ, 2 * DH), pos, ws, seq=True)
    assert e.value.code == -5
