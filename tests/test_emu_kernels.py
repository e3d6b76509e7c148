"""The HIP kernels in a host-side build (tests/emu: the kernel sources compiled as C++, one fiber per
GPU thread) on tensors that END AT AN INACCESSIBLE PAGE, against the oracle.  What this pins without
a GPU: every index the kernels form stays inside its tensor -- a device allocation can end at a
mapping boundary exactly like these buffers, and a read behind it is a memory fault there -- and the
kernels' logic (selection, staging through LDS, reductions, tails of ragged shapes) gives the
oracle's numbers.  What it cannot pin: timing, the compiler's code for the device, hardware
behaviour of the cross-lane instructions (modelled after the ISA manual).  The shapes are chosen so
that the LAST row, the LAST expert and ragged tails are touched."""
import numpy as np
import pytest

import emu_util


@pytest.fixture(scope="module")
def emu(qk):
    with emu_util.emulated(qk) as pool:
        yield pool


@pytest.fixture(params=["lane", "stream"])
def form(request, qk, emu):
    """Both forms of the one-row kernels: block fields loaded per lane (the default), and rows streamed as
    16-byte pieces through LDS with the dense rows' x in registers (the "one_row" and "dense_reg" switches)."""
    on = int(request.param == "stream")
    with qk.option("one_row", on), qk.option("dense_reg", on):
        yield request.param


SWITCHES = ("one_row", "dense_reg", "fused_norm", "attn_block", "dn_fused", "gemm_tiled", "moe_rows", "head_rows", "gemv_depth", "head_depth", "rowwise_max")


@pytest.fixture
def switches_back_to_defaults(qk, emu):
    """qk_open applies the QK_* switches of the environment to the library; this puts the defaults back."""
    yield
    for name in SWITCHES:
        qk.set_option(name, 0)


QUANT = ["q8_0", "q6_k", "iq4_xs", "iq3_xxs"]


def type_id(qk, name):
    return {"q8_0": qk.Q8_0, "q6_k": qk.Q6_K, "iq4_xs": qk.IQ4_XS, "iq3_xxs": qk.IQ3_XXS}[name]


@pytest.mark.parametrize("name", QUANT)
@pytest.mark.parametrize("K,M", [(2048, 1), (2048, 9), (2048, 67), (4096, 5), (8192, 3), (1024, 11), (512, 23), (256, 70),
                                 (768, 6)])
def test_gemv_inside_its_tensors(qk, orc, emu, name, K, M, form):
    """Ragged row counts: full chunks go through the staged 16-byte pieces, the rest through per-lane
    loads; the last row ends at the guard page."""
    t = type_id(qk, name)
    if qk.row_bytes(t, K) == 0:
        pytest.skip("K is not a block multiple of this format")
    W = qk.synth.tensor_host(t, M, K, seed=K + M)
    x = np.random.default_rng(M).standard_normal(K).astype(np.float32)
    pad = (-W.nbytes) % 16   # the kernels want 16-byte aligned tensors; the end stays exact for whole pieces
    Wd = emu.tensor(W.reshape(-1))
    Xd, Yd = emu.tensor(x.reshape(1, K)), emu.zeros((1, M), np.float32)
    qk.gemv(t, Wd, Xd, M, K, out=Yd)
    want = orc.gemv(t, W, x, M, K)
    assert orc.rel_maxabs_err(Yd.numpy()[0], want) <= 1e-3, (name, K, M, pad)


def moe_case(qk, orc, emu, hl, x, norm_w=None, mix=None):
    """One call of the step (or of the block with the norm in front) on guarded tensors; returns what
    the kernels gave and the oracle's reference per row."""
    n = x.shape[0]
    layer = emu_util.layer_in_pool(qk, emu, hl)
    ws = emu.workspace(qk.moe_workspace_bytes(layer, n))
    sel = emu.zeros((n, 160), np.uint8)
    if norm_w is None:
        Y = emu.zeros((n, hl.n_embd), np.float32)
        qk.moe_decode(layer, emu.tensor(x), ws, Y=Y, sel=sel)
        got, inp = Y.numpy(), x
    else:
        S = emu.tensor(x)
        W = emu.tensor(norm_w)
        if mix is None:
            qk.moe_layer_rows(layer, S, W, ws, sel=sel)
            base = x
        else:
            T = emu.zeros(x.shape, np.float32)
            qk.moe_layer_rows(layer, S, W, ws, sel=sel, mix=emu.tensor(mix), T=T)
            base = x + mix
            assert np.array_equal(T.numpy(), base)
        inp = np.stack([orc.add_rms(base[r], norm_w, 1e-6) for r in range(n)])
        got = S.numpy() - base
    ids = sel.numpy().view(np.uint32).reshape(-1, 40)[:, :hl.n_used]
    for r in range(n):
        ref = orc.moe_ref(hl, inp[r])
        if ref["sel"].gap > 2e-3:
            assert sorted(ids[r]) == sorted(ref["sel"].ids[:hl.n_used]), r
            scale = np.max(np.abs(ref["y"]))
            assert np.max(np.abs(got[r] - ref["y"])) <= 1e-3 * scale + 4e-7 * np.max(np.abs(inp[r])) * (norm_w is not None), r
    return ids


def rows_that_pick_the_last_expert(hl, n, seed, scale=None):
    rng = np.random.default_rng(seed)
    gi = hl.gate_inp.astype(np.float64)
    rows = []
    while len(rows) < n:
        x = rng.standard_normal(hl.n_embd).astype(np.float32)
        top = np.argsort(-(gi @ (x.astype(np.float64) * (1.0 if scale is None else scale))))[:hl.n_used]
        if hl.n_expert - 1 in top:
            rows.append(x)
    return np.stack(rows)


@pytest.mark.parametrize("down", ["iq4_xs", "q6_k"])
@pytest.mark.parametrize("E,k,F,H,n", [(8, 2, 256, 2048, 1), (8, 2, 512, 2048, 3), (16, 16, 256, 2048, 1), (6, 3, 1024, 2048, 2),
                                       (4, 2, 256, 4096, 2), (20, 10, 512, 2048, 1)])
def test_moe_step_inside_its_tensors(qk, orc, emu, down, E, k, F, H, n, form):
    """The three one-row launches with the LAST expert among the picks: its last rows end at the guard
    page (a Q6_K run of rows is not a whole number of 16-byte pieces -- the staging must not fetch the
    piece behind it)."""
    hl = qk.synth.HostLayer(seed=E + k + F, n_embd=H, n_ff=F, n_expert=E, n_used=k, down_type=type_id(qk, down))
    x = rows_that_pick_the_last_expert(hl, n, seed=F + n)
    ids = moe_case(qk, orc, emu, hl, x)
    assert all(E - 1 in row for row in ids)


@pytest.mark.parametrize("down", ["iq4_xs", "q6_k"])
def test_moe_block_with_norm_inside_its_tensors(qk, orc, emu, down, form):
    """The block with the RMS norm in front and the residual behind, alone and with a mixer's rows
    added on the way, 1 and 3 rows."""
    hl = qk.synth.HostLayer(seed=91, n_ff=256, n_expert=8, n_used=2, down_type=type_id(qk, down))
    rng = np.random.default_rng(3)
    w = rng.uniform(0.5, 1.5, 2048).astype(np.float32)
    for n in (1, 3):
        x = (rows_that_pick_the_last_expert(hl, n, seed=n, scale=w.astype(np.float64)) * np.float32(7.0)).astype(np.float32)
        moe_case(qk, orc, emu, hl, x, norm_w=w)
        mix = rng.standard_normal(x.shape).astype(np.float32)
        moe_case(qk, orc, emu, hl, x, norm_w=w, mix=mix)


def test_moe_static_workspace_in_the_host_build(qk, orc, emu, form):
    """qkk_moe_decode_static against qkk_moe_decode, both through the host-side build: same bits."""
    hl = qk.synth.HostLayer(seed=12, n_ff=256, n_expert=8, n_used=2)
    layer = emu_util.layer_in_pool(qk, emu, hl)
    rng = np.random.default_rng(0)
    for n in (3, 1):
        x = rng.standard_normal((n, 2048)).astype(np.float32)
        ws = emu.workspace(qk.moe_workspace_bytes(layer, n))
        Y0, sel0 = emu.zeros((n, 2048), np.float32), emu.zeros((n, 160), np.uint8)
        Y1, sel1 = emu.zeros((n, 2048), np.float32), emu.zeros((n, 160), np.uint8)
        X = emu.tensor(x)
        qk.moe_decode(layer, X, ws, Y=Y0, sel=sel0)
        qk.moe_decode_static(layer, X, Y1, sel1)
        assert np.array_equal(Y0.numpy().view(np.uint32), Y1.numpy().view(np.uint32))
        assert np.array_equal(sel0.numpy(), sel1.numpy())


@pytest.mark.parametrize("V,batch", [(37, 1), (1000, 1), (300, 3)])
def test_head_inside_its_tensors(qk, orc, emu, V, batch, form):
    """LM head + argmax on a small vocabulary whose last row ends at the guard page."""
    K = 2048
    W = qk.synth.tensor_host(qk.Q6_K, V, K, seed=V)
    x = np.random.default_rng(V).standard_normal((batch, K)).astype(np.float32)
    ws = emu.workspace(qk.head_workspace_bytes(V, batch))
    tok, logits = qk.head_argmax(emu.tensor(W.reshape(-1)), emu.tensor(x), V, K, ws, want_logits=True)
    for b in range(batch):
        want = orc.gemv(qk.Q6_K, W, x[b], V, K)
        assert orc.rel_maxabs_err(logits.numpy()[b], want) <= 1e-3
        top2 = np.sort(want)[-2:]
        if top2[1] - top2[0] > 2e-3 * abs(top2[1]):
            assert int(tok.numpy()[b]) == int(np.argmax(want))


@pytest.mark.parametrize("V,batch", [(300, 3), (128, 16), (1000, 2), (2049, 9)])
def test_head_with_the_waves_splitting_the_rows(qk, orc, emu, V, batch):
    """The LM head for 2..16 rows with a wave owning 16 vocabulary rows for all of K (the "head_rows" switch):
    vocabularies that end inside a block of 128 rows, on one, or one row behind one, the tensor at the guard
    page; logits and ids against the oracle, ids and (to rounding of the sums) logits as the default kernel's,
    the winning row copied to a lower and a higher id so that equal logits meet across waves and workgroups,
    and a second call on the same workspace."""
    K = 2048
    W = qk.synth.tensor_host(qk.Q6_K, V, K, seed=V).reshape(V, -1).copy()
    x = np.random.default_rng(V).standard_normal((batch, K)).astype(np.float32)
    ws = emu.workspace(qk.head_workspace_bytes(V, batch))
    xd = emu.tensor(x)
    tok0, logits0 = qk.head_argmax(emu.tensor(W.reshape(-1)), xd, V, K, ws, want_logits=True)
    tok0, logits0 = tok0.numpy().copy(), logits0.numpy().copy()
    with qk.option("head_rows", 1):
        tok, logits = qk.head_argmax(emu.tensor(W.reshape(-1)), xd, V, K, ws, want_logits=True)
        tok, logits = tok.numpy().copy(), logits.numpy().copy()
        for b in range(batch):
            want = orc.gemv(qk.Q6_K, W.reshape(-1), x[b], V, K)
            assert orc.rel_maxabs_err(logits[b], want) <= 1e-3
            assert int(tok[b]) == int(np.argmax(logits[b]))
        assert orc.rel_maxabs_err(logits, logits0) <= 1e-5
        # ties: row 0's winner copied to the last row and to row 1 (or 0): the lowest id must win
        best = int(tok[0])
        lo = 1 if best != 1 else 0
        W[V - 1] = W[best]
        W[lo] = W[best]
        tok2, _ = qk.head_argmax(emu.tensor(W.reshape(-1)), xd, V, K, ws)
        assert int(tok2.numpy()[0]) == min(best, lo)
    assert qk.get_option("head_rows") == 0


@pytest.mark.parametrize("name", QUANT)
@pytest.mark.parametrize("M,batch", [(37, 1), (9, 2)])
def test_gemv_norm_inside_its_tensors(qk, orc, emu, name, M, batch):
    """The GEMV with the RMS norm in front (no launch of its own) against the oracle's norm + GEMV."""
    t, K = type_id(qk, name), 2048
    W = qk.synth.tensor_host(t, M, K, seed=M)
    rng = np.random.default_rng(M + batch)
    x = (rng.standard_normal((batch, K)) * 3.0).astype(np.float32)
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    Yd = emu.zeros((batch, M), np.float32)
    qk.gemv_norm(t, emu.tensor(W.reshape(-1)), emu.tensor(x), emu.tensor(w), M, K, out=Yd)
    want = orc.gemv(t, W, np.stack([orc.add_rms(x[b], w, 1e-6) for b in range(batch)]), M, K)
    assert orc.rel_maxabs_err(Yd.numpy(), want) <= 1e-3


def test_head_norm_inside_its_tensors(qk, orc, emu):
    """The LM head with the output norm in front against the oracle's norm + GEMV + argmax."""
    V, K = 301, 2048
    W = qk.synth.tensor_host(qk.Q6_K, V, K, seed=V)
    rng = np.random.default_rng(V)
    x = (rng.standard_normal((1, K)) * 2.0).astype(np.float32)
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    ws = emu.workspace(qk.head_workspace_bytes(V, 1))
    tok, logits = qk.head_argmax_norm(emu.tensor(W.reshape(-1)), emu.tensor(x), emu.tensor(w), V, K, ws, want_logits=True)
    want = orc.gemv(qk.Q6_K, W, orc.add_rms(x[0], w, 1e-6), V, K)
    assert orc.rel_maxabs_err(logits.numpy()[0], want) <= 1e-3
    assert int(tok.numpy()[0]) == int(np.argmax(want))


@pytest.mark.parametrize("hq,hkv,base,n_pos", [(16, 2, 0, 16), (8, 2, 45, 19), (3, 1, 60, 4)])
def test_attention_blocks_inside_their_tensors(qk, emu, hq, hkv, base, n_pos):
    """The sixteen-row attention kernel on caches whose LAST row is the last position fed (tmax = base +
    n_pos) and that end at the guard page, against the CPU mirror."""
    import os
    import sys
    import torch
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
    import qk_oracle_attn as OA
    DH, NROT, tmax = 256, 64, base + n_pos
    rng = np.random.default_rng(hq + n_pos)
    rope = OA.rope_table(tmax, NROT)
    kc, vc = np.zeros((hkv, tmax, DH), np.float32), np.zeros((hkv, tmax, DH), np.float32)
    kc[:, :base], vc[:, :base] = rng.standard_normal((hkv, base, DH)), rng.standard_normal((hkv, base, DH))
    qn, kn = (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32), (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32)
    qfull = (rng.standard_normal((n_pos, hq, 2 * DH)) * 2).astype(np.float32)
    kin, vin = rng.standard_normal((n_pos, hkv, DH)).astype(np.float32), rng.standard_normal((n_pos, hkv, DH)).astype(np.float32)
    kd, vd, qfd = emu.tensor(kc[None]), emu.tensor(vc[None]), emu.tensor(qfull)
    pos = emu.tensor(np.arange(base, base + n_pos, dtype=np.int32))
    ws = emu.workspace(qk.attn_workspace_bytes(n_pos, hq))
    qh = qk.attn_prep(qfd, emu.tensor(kin), emu.tensor(vin), emu.tensor(qn), emu.tensor(kn), emu.tensor(rope), pos, kd, vd, NROT,
                      qhat=emu.zeros((n_pos, hq, DH), np.float32), seq=True)
    with qk.option("attn_block", 1):
        att = qk.attn_decode(qh, kd, vd, qfd, pos, ws, att=emu.zeros((n_pos, hq, DH), np.float32), seq=True).numpy()
    for t in range(n_pos):
        want = OA.attend(OA.prep(qfull[t], kin[t], vin[t], qn, kn, rope, base + t, kc, vc, NROT), kc, vc, qfull[t], base + t)
        err = float(np.max(np.abs(att[t].astype(np.float64) - want)) / np.max(np.abs(want)))
        assert err <= 1e-3, (t, err)


@pytest.mark.parametrize("name", ["f16", "f32"])
@pytest.mark.parametrize("K,M", [(2048, 1), (2048, 9), (4096, 3), (512, 70), (768, 6)])
def test_dense_gemv_inside_its_tensors(qk, orc, emu, name, K, M, form):
    """Dense rows: K a whole number of 64 sixteen-byte chunks takes the kernel with x in registers (the row
    after the last one is never fetched: the prefetch re-reads the last row), other K the chunk loop."""
    t = {"f16": qk.F16, "f32": qk.F32}[name]
    W = qk.synth.tensor_host(t, M, K, seed=K + M)
    x = np.random.default_rng(M).standard_normal((1, K)).astype(np.float32)
    Yd = emu.zeros((1, M), np.float32)
    qk.gemv(t, emu.tensor(W.reshape(-1)), emu.tensor(x), M, K, out=Yd)
    want = orc.gemv(t, W, x[0], M, K)
    assert orc.rel_maxabs_err(Yd.numpy()[0], want) <= 1e-3


def test_engine_in_the_host_build_and_its_memory_check(qk, emu, tmp_path, monkeypatch):
    """qk_open through the host-side build: a small whole-model file opens and steps; with sixteen slots of
    4,096 positions the attention caches and their snapshots need 0.6 GB on top of the 0.5 GB of the model and
    the rows of a pass, and a device that reports 1 GB free (QK_EMU_FREE_BYTES) refuses the configuration before
    any tensor is uploaded, with the figures in the message; one slot of 64 positions still fits."""
    model = qk.engine.FullModel(5, kinds="AAR", vocab=64, n_expert=8, n_ff=256, n_used=2, eos=70)
    path = model.write(str(tmp_path / "m.gguf"))
    with qk.engine.Engine(path, n_slots=1, n_ctx=64, chunk=2) as eng:
        assert (eng.n_layer, eng.vocab) == (3, 64)
        assert eng.slot_start(0, [3, 5], 3) == 0
        rc, out, fin = eng.step_chunk()
        assert rc == 1 and 1 <= len(out[0]) <= 2 and all(t < 64 for t in out[0])
    monkeypatch.setenv("QK_EMU_FREE_BYTES", str(1 << 30))
    with pytest.raises(qk.capi.QkError) as e:
        qk.engine.Engine(path, n_slots=16, n_ctx=4096, chunk=2)
    assert "GB" in str(e.value) and "16 slot" in str(e.value)
    with qk.engine.Engine(path, n_slots=1, n_ctx=64, chunk=2) as eng:   # one slot of 64 positions still fits
        assert eng.n_slots == 1


@pytest.mark.parametrize("switches", [{}, {"QK_ONE_ROW": "stream", "QK_DENSE_REG": "1", "QK_FUSED_NORM": "1", "QK_ATTN_BLOCK": "1", "QK_DN_FUSED": "1", "QK_GEMM_TILED": "1"}],
                         ids=["defaults", "every_switch_on"])
def test_whole_model_stream_in_the_host_build(qk, emu, tmp_path, monkeypatch, switches, switches_back_to_defaults):
    """The engine on a small whole model (one gated-DeltaNet layer, one attention layer, a MoE block each)
    through the host-side build: two slots' greedy streams -- prompts prefilled in a pass, then serial steps
    from a replayed graph -- equal the restated state machine driving the CPU oracle of the whole model,
    call by call."""
    import os
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
    import qk_oracle_engine as OE
    for k_, v_ in {"QK_ONE_ROW": "lane", "QK_DENSE_REG": "0", "QK_FUSED_NORM": "0", "QK_ATTN_BLOCK": "0", "QK_DN_FUSED": "0", "QK_GEMM_TILED": "0", **switches}.items():
        monkeypatch.setenv(k_, v_)   # qk_open reads the switches that are set
    vocab = 96
    model = qk.engine.FullModel(9, kinds="RA", vocab=vocab, n_expert=8, n_ff=256, n_used=2, eos=vocab + 5)
    path = model.write(str(tmp_path / "m.gguf"))
    rng = np.random.default_rng(2)
    prompts = {1: [int(t) for t in rng.integers(0, vocab, 7)], 0: [int(t) for t in rng.integers(0, vocab, 1)]}
    with qk.engine.Engine(path, n_slots=2, n_ctx=64, chunk=3) as eng:
        ref = OE.SlotMachine(OE.FullModelOracle(model, 2, 64), vocab, vocab + 5, 2, 64, 3)
        for call in range(4):
            if call == 0:
                assert eng.slot_start(1, prompts[1], 5) == ref.slot_start(1, prompts[1], 5) == 0
            if call == 1:
                assert eng.slot_start(0, prompts[0], 4) == ref.slot_start(0, prompts[0], 4) == 0
            got, want = eng.step_chunk(), ref.step_chunk()
            assert got == want, (call, got, want)
        assert not any(sl["active"] for sl in ref.slots)


@pytest.mark.parametrize("down,n", [("iq4_xs", 16), ("q6_k", 40)])
def test_expert_major_moe_inside_its_tensors(qk, orc, emu, down, n):
    """The expert-major path (more than ten rows: routing with selection in the last workgroup, the
    matrix-core gate/up and down kernels, the fold) on guarded tensors and a guarded workspace, 16 rows
    (the fused launches) and 40 rows (the shared expert on its own launches), against the oracle."""
    hl = qk.synth.HostLayer(seed=31 + n, n_ff=256, n_expert=8, n_used=2, down_type=type_id(qk, down))
    x = np.random.default_rng(n).standard_normal((n, 2048)).astype(np.float32)
    ids = moe_case(qk, orc, emu, hl, x)
    assert ids.shape == (n, 2) and set(np.unique(ids)) <= set(range(8))
    qk.moe_workspace_status()   # the cleared workspace raised no flag


@pytest.mark.parametrize("down,n,E,k,F", [("iq4_xs", 16, 8, 2, 256), ("q6_k", 40, 8, 2, 256), ("iq4_xs", 70, 4, 2, 512), ("q6_k", 12, 16, 8, 1024),
                                          ("iq4_xs", 20, 2, 1, 256)])
def test_row_split_expert_kernels_inside_their_tensors(qk, orc, emu, down, n, E, k, F):
    """The routed experts' projections with the waves splitting the weight rows (the "moe_rows" switch): 12 to 70
    rows, so that experts hold from a few pairs to several tiles of 16 (70 rows x 2 picks on 4 experts: three
    tiles, the last one partial), n_ff of two to eight blocks of 128 rows, the LAST expert among the picks and the
    tensors ending at guard pages; work items of four, two and one block of rows (the host-side build's "device" has
    four CUs, so eight resident workgroups decide); against the oracle, and the same ids and (to rounding of the sums)
    the same outputs as the K-split kernels."""
    hl = qk.synth.HostLayer(seed=31 + n, n_ff=F, n_expert=E, n_used=k, down_type=type_id(qk, down))
    x = rows_that_pick_the_last_expert(hl, n, seed=n)
    base = moe_case(qk, orc, emu, hl, x)
    with qk.option("moe_rows", 1):
        ids = moe_case(qk, orc, emu, hl, x)
    assert np.array_equal(ids, base) and all(E - 1 in row for row in ids)
    qk.moe_workspace_status()


@pytest.mark.parametrize("M,K,N", [(48, 2048, 20), (33, 512, 9), (16, 4096, 128)])
def test_q8_0_gemm_inside_its_tensors(qk, orc, emu, M, K, N):
    """The prefill GEMM (cooperative matrix-core stream, weights read once for all rows) on a tensor that ends
    at the guard page, against the oracle's double-precision product."""
    W = qk.synth.tensor_host(qk.Q8_0, M, K, seed=M + N)
    X = np.random.default_rng(N).standard_normal((N, K)).astype(np.float32)
    Y = emu.zeros((N, M), np.float32)
    qk.gemm_q8_0(emu.tensor(W.reshape(-1)), emu.tensor(X), M, K, out=Y)
    want = orc.gemm_q8_0(W, X, M, K)
    assert orc.rel_maxabs_err(Y.numpy(), want) <= 1e-3


@pytest.mark.parametrize("name", QUANT)
@pytest.mark.parametrize("M,K,N", [(32, 256, 64), (50, 512, 130), (17, 2048, 128), (96, 768, 200)])
def test_tiled_gemm_inside_its_tensors(qk, orc, emu, name, M, K, N):
    """The product for 64 and more activation rows with every weight tile decoded once per 128 rows (the
    "gemm_tiled" switch), all four block formats: weight row counts that leave the last 32-row block partial,
    activation row counts that leave waves idle or half full, row lengths whose fragments start anywhere
    inside a 16-byte piece, the tensor ending at the guard page; against the oracle's double-precision rows
    and against the cooperative stream (the default)."""
    t = type_id(qk, name)
    if (M * qk.row_bytes(t, K)) % 16:
        pytest.skip("the tensor does not end on a 16-byte boundary: neither matrix-core kernel takes it")
    W = qk.synth.tensor_host(t, M, K, seed=M + N)
    X = np.random.default_rng(N).standard_normal((N, K)).astype(np.float32)
    Wd, Xd = emu.tensor(W.reshape(-1)), emu.tensor(X)
    Y0, Y1 = emu.zeros((N, M), np.float32), emu.zeros((N, M), np.float32)
    qk.gemv(t, Wd, Xd, M, K, out=Y0)
    with qk.option("gemm_tiled", 1):
        qk.gemv(t, Wd, Xd, M, K, out=Y1)
    want = np.stack([orc.gemv(t, W, X[n], M, K) for n in range(N)])
    assert orc.rel_maxabs_err(Y1.numpy(), want) <= 1e-3
    assert orc.rel_maxabs_err(Y1.numpy(), Y0.numpy()) <= 1e-5   # both keep operands exact to 2^-22: rounding of the sums only
    assert not np.array_equal(Y0.numpy(), np.zeros_like(Y0.numpy()))


def test_tiled_gemm_is_the_q8_0_prefill_product(qk, orc, emu):
    """qkk_gemm_q8_0 with the switch: the reference's acceptance bar (max error below 2e-3 of the result's
    rms, src/main.cpp:5659-5662) and the per-element bar; fewer than 64 rows keep the cooperative stream."""
    M, K, N = 64, 1024, 128
    W = qk.synth.tensor_host(qk.Q8_0, M, K, seed=9)
    X = np.random.default_rng(1).standard_normal((N, K)).astype(np.float32)
    Wd, Xd = emu.tensor(W.reshape(-1)), emu.tensor(X)
    with qk.option("gemm_tiled", 1):
        Y = emu.zeros((N, M), np.float32)
        qk.gemm_q8_0(Wd, Xd, M, K, out=Y)
        Ys = emu.zeros((40, M), np.float32)
        qk.gemm_q8_0(Wd, emu.tensor(X[:40]), M, K, out=Ys)
    want = orc.gemm_q8_0(W, X, M, K)
    err = np.abs(Y.numpy().astype(np.float64) - want)
    assert err.max() < 2e-3 * np.sqrt(np.mean(want ** 2)) and orc.rel_maxabs_err(Y.numpy(), want) <= 1e-3
    assert orc.rel_maxabs_err(Ys.numpy(), want[:40]) <= 1e-3


def _oracle_module(name):
    import importlib
    import os
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
    return importlib.import_module(name)


def test_attention_decode_inside_its_tensors(qk, emu):
    """The attention decode step (prep + position ranges + fold) for two slots whose caches end at the guard
    page, the second slot at the cache's last position, against the CPU mirror."""
    OA = _oracle_module("qk_oracle_attn")
    DH, NROT, HQ, HKV, tmax, positions = 256, 64, 16, 2, 96, [5, 95]
    rng = np.random.default_rng(1)
    kc, vc = np.zeros((2, HKV, tmax, DH), np.float32), np.zeros((2, HKV, tmax, DH), np.float32)
    for s, p in enumerate(positions):
        kc[s, :, :p], vc[s, :, :p] = rng.standard_normal((HKV, p, DH)), rng.standard_normal((HKV, p, DH))
    qfull = (rng.standard_normal((2, HQ, 2 * DH)) * 2).astype(np.float32)
    kin, vin = rng.standard_normal((2, HKV, DH)).astype(np.float32), rng.standard_normal((2, HKV, DH)).astype(np.float32)
    qn, kn = (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32), (1 + 0.2 * rng.standard_normal(DH)).astype(np.float32)
    rope = OA.rope_table(tmax, NROT)
    kd, vd, qfd = emu.tensor(kc), emu.tensor(vc), emu.tensor(qfull)
    pos = emu.tensor(np.array(positions, dtype=np.int32))
    qh = qk.attn_prep(qfd, emu.tensor(kin), emu.tensor(vin), emu.tensor(qn), emu.tensor(kn), emu.tensor(rope), pos, kd, vd, NROT,
                      qhat=emu.zeros((2, HQ, DH), np.float32))
    att = qk.attn_decode(qh, kd, vd, qfd, pos, emu.workspace(qk.attn_workspace_bytes(2, HQ)),
                         att=emu.zeros((2, HQ, DH), np.float32)).numpy()
    for s, p in enumerate(positions):
        want = OA.attend(OA.prep(qfull[s], kin[s], vin[s], qn, kn, rope, p, kc[s], vc[s], NROT), kc[s], vc[s], qfull[s], p)
        assert float(np.max(np.abs(att[s] - want)) / np.max(np.abs(want))) <= 1e-3, s


@pytest.mark.parametrize("fused", [False, True])
def test_deltanet_step_inside_its_tensors(qk, emu, fused):
    """The gated-DeltaNet decode step for two slots -- as the two launches and as the one launch -- on guarded
    window, state and weight tensors, against the CPU mirror."""
    OD = _oracle_module("qk_oracle_deltanet")
    DS, HK, HV, NE = 128, 16, 32, 2048
    CH, QK = (2 * HK + HV) * DS, 2 * HK * DS
    rng = np.random.default_rng(3)
    r = lambda *shape, scale=1.0: (rng.standard_normal(shape) * scale).astype(np.float32)
    alpha_w, beta_w, dt_bias = r(HV, NE, scale=0.03), r(HV, NE, scale=0.03), r(HV)
    a_vec, ker, norm_w = (-np.abs(r(HV)) - 0.05).astype(np.float32), r(CH, 4, scale=0.5), (1 + 0.1 * r(DS)).astype(np.float32)
    st, S = r(2, CH, 3), r(2, HV, DS, DS, scale=0.1)
    x, qkv, z = r(2, NE), r(2, CH), r(2, HV * DS)
    std, Sd = emu.tensor(st), emu.tensor(np.ascontiguousarray(S.transpose(0, 1, 3, 2)))
    w = [emu.tensor(a) for a in (alpha_w, beta_w, dt_bias, a_vec)]
    if fused:
        att = qk.dn_step_fused(emu.tensor(x), *w, std, emu.tensor(qkv), emu.tensor(ker), Sd, emu.tensor(norm_w), emu.tensor(z), HK, HV)
    else:
        gb, conv = qk.dn_ab_conv(emu.tensor(x), *w, std, emu.tensor(qkv), emu.tensor(ker), QK)
        att = qk.dn_step(conv, gb, Sd, emu.tensor(norm_w), emu.tensor(z), HK, HV)
    for s in range(2):
        g, b = OD.ab(x[s], alpha_w, beta_w, dt_bias, a_vec)
        want = OD.step(OD.conv(st[s].copy(), qkv[s], ker, DS, QK), g, b, S[s].copy(), norm_w, z[s], HK, HV)
        assert float(np.max(np.abs(att.numpy()[s] - want)) / np.max(np.abs(want))) <= 1e-3, s


SITES = ["iq3_grid", "iq3_sign", "iq4_pair", "iq4_float", "iq3_grid_word"]


def _lds_lookup_cycles(qk, emu, run):
    """Runs `run()` with the host-side build's LDS bank model on and returns, per marked lookup site,
    (wave instructions, modelled cycles per instruction, conflict-free cycles per instruction)."""
    import ctypes as C
    L = emu_util.emu_lib(qk)
    L.emu_lds_probe_read.argtypes = [C.c_int, C.POINTER(C.c_uint64)]
    L.emu_lds_probe_enable(1)
    try:
        run()
    finally:
        L.emu_lds_probe_enable(0)
    out = {}
    for site, name in enumerate(SITES):
        v = (C.c_uint64 * 3)()
        L.emu_lds_probe_read(site, v)
        if v[0]:
            out[name] = (int(v[0]), v[1] / v[0], v[2] / v[0])
    return out


def _model_cycles(entries, entry_bytes, copies, rng, trials=400):
    """The same bank model for a table of `entries` entries in `copies` copies, copy r confined to its own
    64 / copies banks and read by the lanes with lane mod copies = r: mean cycles per wave instruction of 64
    random lookups."""
    per_pass = {4: 64, 8: 32, 16: 16}[entry_bytes]
    dw, banks_per_copy = entry_bytes // 4, 64 // copies
    slots = max(1, banks_per_copy // dw)          # entries of one copy per 256-byte row
    total = 0
    for _ in range(trials):
        e = rng.integers(0, entries, 64)
        for l0 in range(0, 64, per_pass):
            seen = {}
            for lane in range(l0, l0 + per_pass):
                r = lane % copies
                row, slot = divmod(int(e[lane]), slots)
                for d in range(dw):
                    bank = r * banks_per_copy + (slot * dw + d) % banks_per_copy
                    seen.setdefault(bank, set()).add((row, d))
            total += max(len(v) for v in seen.values())
    return total / trials


def test_lds_bank_model_of_the_table_lookups(qk, orc, emu, capsys):
    """A PROXY for the device's LDS, not a measurement (64 banks of four bytes; a pass of 64 / 32 / 16 lanes for
    4 / 8 / 16-byte reads costs the largest number of distinct dwords any bank is asked for).  Counted on the GEMVs
    in the host-side build, per wave instruction:
      * the streamed IQ3_XXS product reads 8-byte codebook entries at about three times, and 16-byte sign entries at
        nearly three times, their conflict-free cost (device counters on the same loop: 58 % of the LDS cycles were
        bank conflicts); the streamed IQ4_XS pair table at three to four times;
      * the per-lane IQ4_XS product reads a 16-entry float codebook, whose entries lie in 16 different banks: no
        conflicts at all, twice the lookups -- one reason why that form measured faster for IQ4_XS;
      * copies of a table in bank groups of their own do not help until every lane of a pass has a group to itself:
        8 copies of the codebook still cost nearly three passes, because a wave instruction waits for its worst bank;
        only 32 copies (64 KB for 256 entries of 8 bytes) are conflict-free -- more LDS than the streaming loop can
        give up without losing the occupancy that hides its latency."""
    M, K = 64, 2048
    x = np.random.default_rng(4).standard_normal((1, K)).astype(np.float32)
    got = {}
    for name, form in (("iq3_xxs", 1), ("iq4_xs", 1), ("iq3_xxs", 0), ("iq4_xs", 0)):
        t = type_id(qk, name)
        W = qk.synth.tensor_host(t, M, K, seed=3)
        Wd, Xd, Yd = emu.tensor(W.reshape(-1)), emu.tensor(x), emu.zeros((1, M), np.float32)
        with qk.option("one_row", form):
            got[name, form] = _lds_lookup_cycles(qk, emu, lambda: qk.gemv(t, Wd, Xd, M, K, out=Yd))
        assert orc.rel_maxabs_err(Yd.numpy()[0], orc.gemv(t, W, x[0], M, K)) <= 1e-3
    with capsys.disabled():
        print(f"\n[lds model] (instructions, cycles each, conflict-free cycles each): {got}", flush=True)
    n, c, i = got["iq3_xxs", 1]["iq3_grid"]
    assert n == M * 8 and i == 2 and 2.5 <= c / i <= 4.0          # 8 lookups per 32 weights, 64 rows of one wave each
    n, c, i = got["iq3_xxs", 1]["iq3_sign"]
    assert n == M * 4 and i == 4 and 2.0 <= c / i <= 4.0
    n, c, i = got["iq4_xs", 1]["iq4_pair"]
    assert n == M * 16 and i == 1 and 2.5 <= c / i <= 5.0
    n, c, i = got["iq4_xs", 0]["iq4_float"]
    assert n == M * 32 and c == i == 1                             # 16 entries in 16 banks: never a conflict
    n, c, i = got["iq3_xxs", 0]["iq3_grid_word"]
    assert n == M * 8 and i == 1 and 2.5 <= c / i <= 5.0
    # what copies per bank group would buy, in the same model
    rng = np.random.default_rng(0)
    one, eight, thirty_two = (_model_cycles(256, 8, r, rng) for r in (1, 8, 32))
    assert abs(one - got["iq3_xxs", 1]["iq3_grid"][1]) < 0.5        # the model in Python agrees with the counted kernel
    assert eight > 0.85 * one and thirty_two == 2.0


@pytest.mark.parametrize("E,k", [(8, 8), (100, 8), (256, 8), (256, 16), (300, 10), (512, 16), (64, 1)])
def test_selectors_agree_with_the_oracle_on_exact_logits(qk, orc, emu, E, k):
    """The router's logits made exact (the activation row is the first unit vector, so logit e is the first
    element of router row e): ties in clusters, NaN and infinite logits, fewer finite logits than picks, all
    logits non-finite.  Ids and weights of the one-wave selector (per-lane form, and the streamed form with
    "select_ranked" off) and of the rank-counting selector (the streamed form's default) against the oracle's
    restatement of the reference's rounds (shaders/moe_select.comp:28-34, 53-76): ids bit for bit in pick order."""
    hl = qk.synth.HostLayer(seed=E + k, n_ff=256, n_expert=E, n_used=k)
    rng = np.random.default_rng(E * 31 + k)
    x = np.zeros((1, 2048), np.float32)
    x[0, 0] = 1.0
    cases = []
    cases.append(rng.standard_normal(E))                                   # plain
    cases.append(np.round(rng.standard_normal(E) * 2) / 2)                 # many ties
    t = rng.standard_normal(E); t[rng.integers(0, E, max(1, E // 3))] = np.nan; t[rng.integers(0, E, 3)] = np.inf; cases.append(t)
    t = np.full(E, np.nan); t[rng.choice(E, min(E, max(1, k // 2)), replace=False)] = rng.standard_normal(min(E, max(1, k // 2))); cases.append(t)  # fewer finite than picks
    cases.append(np.full(E, np.nan))                                       # nothing finite
    cases.append(np.full(E, 0.25))                                         # all equal
    t = -np.abs(rng.standard_normal(E)); t[E - 1] = 0.0; t[0] = -0.0; cases.append(t)   # signed zeros tie
    import contextlib
    hl.gate_inp[:, :] = 0
    layer = emu_util.layer_in_pool(qk, emu, hl)           # once: the cases rewrite the router's first column in place
    router = layer.tensors["gate_inp"].numpy()
    ws = emu.workspace(qk.moe_workspace_bytes(layer, 1))
    X = emu.tensor(x)
    for ci, logits in enumerate(cases):
        router[:, 0] = logits.astype(np.float32)
        want = orc.select_f32(logits.astype(np.float32), k)
        got = {}
        for name, opts in (("lane", {"one_row": 0}), ("stream_rounds", {"one_row": 1, "select_ranked": 0}),
                           ("stream_ranked", {"one_row": 1, "select_ranked": 1})):
            sel = emu.zeros((1, 160), np.uint8)
            Y = emu.zeros((1, 2048), np.float32)
            with contextlib.ExitStack() as st:
                for o, v in opts.items():
                    st.enter_context(qk.option(o, v))
                qk.moe_decode(layer, X, ws, Y=Y, sel=sel, stages=3)   # route + select/gate/up
            raw = sel.numpy().reshape(-1)
            ids = raw[:64].view(np.uint32)[:k].tolist()
            w = raw[64:128].view(np.float32)[:k]
            got[name] = ids
            assert ids == list(want.ids[:k]), (ci, name, ids, list(want.ids[:k]))
            assert np.allclose(w, np.array(want.w[:k]), rtol=0, atol=1e-6, equal_nan=True), (ci, name, w, list(want.w[:k]))


def _snapshot(*arrays):
    return [np.ascontiguousarray(a.numpy()).view(np.uint8).copy() for a in arrays]


def _order_cases(qk, emu):
    """Small launches of every kernel family, each returning the bytes it produced."""
    K = 2048
    cases = {}
    for name in QUANT:
        t = type_id(qk, name)
        W = qk.synth.tensor_host(t, 67, K, seed=7)
        x1 = np.random.default_rng(1).standard_normal((1, K)).astype(np.float32)
        x5 = np.random.default_rng(5).standard_normal((5, K)).astype(np.float32)
        x70 = np.random.default_rng(70).standard_normal((70, K)).astype(np.float32)

        def gemv(x, W=W, t=t):
            Y = emu.zeros((x.shape[0], 67), np.float32)
            qk.gemv(t, emu.tensor(W.reshape(-1)), emu.tensor(x), 67, K, out=Y)
            return _snapshot(Y)
        cases[f"gemv {name} one row"] = lambda x1=x1, gemv=gemv: gemv(x1)
        cases[f"gemv {name} five rows"] = lambda x5=x5, gemv=gemv: gemv(x5)
        if name in ("q8_0", "iq3_xxs"):
            cases[f"gemv {name} seventy rows"] = lambda x70=x70, gemv=gemv: gemv(x70)
    Wf = np.random.default_rng(3).standard_normal((40, K)).astype(np.float16)
    xf = np.random.default_rng(4).standard_normal((1, K)).astype(np.float32)

    def dense():
        Y = emu.zeros((1, 40), np.float32)
        qk.gemv(qk.F16, emu.tensor(Wf.reshape(-1)), emu.tensor(xf), 40, K, out=Y)
        return _snapshot(Y)
    cases["gemv f16"] = dense
    for down, E, k, F in (("iq4_xs", 8, 2, 256), ("q6_k", 16, 4, 512)):
        hl = qk.synth.HostLayer(seed=E, n_ff=F, n_expert=E, n_used=k, down_type=type_id(qk, down))
        for n in (1, 3, 12, 40):
            x = np.random.default_rng(n).standard_normal((n, K)).astype(np.float32)

            def moe(hl=hl, x=x, n=n):
                layer = emu_util.layer_in_pool(qk, emu, hl)
                ws = emu.workspace(qk.moe_workspace_bytes(layer, n))
                sel, Y = emu.zeros((n, 160), np.uint8), emu.zeros((n, K), np.float32)
                qk.moe_decode(layer, emu.tensor(x), ws, Y=Y, sel=sel)
                return _snapshot(Y, sel)
            cases[f"moe {down} {n} rows"] = moe
    Wh = qk.synth.tensor_host(qk.Q6_K, 300, K, seed=300)
    for b in (1, 3):
        xh = np.random.default_rng(b).standard_normal((b, K)).astype(np.float32)

        def head(xh=xh, b=b):
            ws = emu.workspace(qk.head_workspace_bytes(300, b))
            tok, logits = qk.head_argmax(emu.tensor(Wh.reshape(-1)), emu.tensor(xh), 300, K, ws, want_logits=True)
            return _snapshot(tok, logits)
        cases[f"head {b} rows"] = head
    return cases


FORMS = [{}, {"one_row": 1, "dense_reg": 1}, {"one_row": 1, "select_ranked": 0}, {"gemm_tiled": 1, "moe_rows": 1, "head_rows": 1}]


@pytest.mark.parametrize("form_switches", FORMS, ids=["defaults", "streamed", "streamed-rounds", "tiled-rows"])
def test_results_do_not_depend_on_the_order_of_the_threads(qk, emu, switches_back_to_defaults, form_switches):
    """Between two barriers the host-side build runs the threads of a workgroup one after the other.  Two accesses
    to LDS (or to a workspace) by different threads that need a barrier between them and have none are seen
    writer-first under one order and reader-first under another, so every family of kernels, in every form, has to
    give the same bits with the threads visited in ascending order, in descending order and in two random orders
    drawn anew at every sweep.  (What this cannot see: orderings inside a wave that the hardware's lockstep
    provides and the device compiler must keep.)"""
    L = emu_util.emu_lib(qk)
    for name_, v in form_switches.items():
        qk.set_option(name_, v)
    cases = _order_cases(qk, emu)
    try:
        L.emu_set_schedule(0, 1)
        want = {k_: run() for k_, run in cases.items()}
        for mode, seed in ((1, 1), (2, 11), (2, 12)):
            L.emu_set_schedule(mode, seed)
            for k_, run in cases.items():
                got = run()
                assert all(np.array_equal(a, b) for a, b in zip(got, want[k_])), (k_, mode, seed)
    finally:
        L.emu_set_schedule(0, 1)


def test_mixers_and_engine_under_a_random_thread_order(qk, emu, tmp_path, monkeypatch, switches_back_to_defaults):
    """The attention and gated-DeltaNet kernels (both forms each) and the engine's captured steps with every switch
    on, once more with the threads of a workgroup visited in a random order and waves held back at random: the same
    checks against the CPU mirrors and the oracle's state machine as in ascending order."""
    L = emu_util.emu_lib(qk)
    L.emu_set_schedule(2, 21)
    try:
        test_attention_blocks_inside_their_tensors(qk, emu, 8, 2, 45, 19)
        test_attention_decode_inside_its_tensors(qk, emu)
        for fused in (False, True):
            test_deltanet_step_inside_its_tensors(qk, emu, fused)
        every = {"QK_ONE_ROW": "stream", "QK_DENSE_REG": "1", "QK_FUSED_NORM": "1", "QK_ATTN_BLOCK": "1", "QK_DN_FUSED": "1",
                 "QK_GEMM_TILED": "1", "QK_MOE_ROWS": "1", "QK_HEAD_ROWS": "1"}
        test_whole_model_stream_in_the_host_build(qk, emu, tmp_path, monkeypatch, every, None)
    finally:
        L.emu_set_schedule(0, 1)
