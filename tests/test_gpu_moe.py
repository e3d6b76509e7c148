"""Fused MoE decode step through the C ABI against the oracle's restatement of the
reference's CPU MoE.  Selected expert ids must match exactly and in pick order; router
weights within 1e-4 (the reference's bar); outputs within 1e-3 relative max-abs."""
import numpy as np
import pytest

# every test runs on both forms of the one-row kernels (conftest.one_row_form)
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("one_row_form")]
TOL = 1e-3


def sel_fields(sel):
    raw = sel.cpu().numpy()
    ids = raw.view(np.uint32).reshape(-1, 40)[:, :16]
    w = raw.view(np.float32).reshape(-1, 40)[:, 16:32]
    wsh = raw.view(np.float32).reshape(-1, 40)[:, 32]
    return ids, w, wsh


def pick_inputs(orc, hl, n, seed, min_gap=2e-3):
    """n activation rows whose top-k margin is comfortably above fp32 dot-product noise."""
    rng = np.random.default_rng(seed)
    rows, refs = [], []
    gi64 = hl.gate_inp.astype(np.float64)
    while len(rows) < n:
        x = rng.standard_normal(hl.n_embd).astype(np.float32)
        top = np.sort(gi64 @ x.astype(np.float64))[::-1][:hl.n_used + 1]
        if hl.n_used < hl.n_expert and np.min(-np.diff(top)) <= min_gap:
            continue   # cheap pre-check of the margins before the full CPU reference
        r = orc.moe_ref(hl, x)
        picked = sorted(r["sel"].w[:hl.n_used], reverse=True)
        # margins between consecutive picks decide the ORDER, the gap decides the SET
        lw = np.log(np.array(picked))
        order_margin = np.min(-np.diff(lw)) if hl.n_used > 1 else np.inf
        if r["sel"].gap > min_gap and order_margin > min_gap:
            rows.append(x)
            refs.append(r)
    return np.stack(rows), refs


@pytest.fixture(scope="module")
def layer_iq4(qk):
    return qk.synth.HostLayer(seed=100, down_type=qk.IQ4_XS)


@pytest.fixture(scope="module")
def layer_q6k(qk):
    return qk.synth.HostLayer(seed=200, down_type=qk.Q6_K)


def check(qk, orc, dev, hl, X, refs, stages=None):
    import torch
    layer = hl.to_device(dev)
    n = X.shape[0]
    ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
    Y, sel = qk.moe_decode(layer, torch.from_numpy(X).to(dev), ws, stages=stages)
    torch.cuda.synchronize()
    assert np.all(sel.cpu().numpy().view(np.uint32).reshape(-1, 40)[:, 33:] == 0)   # padding untouched
    Y = Y.cpu().numpy()
    ids, w, wsh = sel_fields(sel)
    k = hl.n_used
    for s in range(n):
        r = refs[s]
        assert list(ids[s, :k]) == list(r["sel"].ids[:k]), f"slot {s}"
        assert np.max(np.abs(w[s, :k] - np.array(r["sel"].w[:k]))) <= 1e-4
        assert abs(wsh[s] - r["sel"].w_shared) <= 1e-4
        assert orc.rel_maxabs_err(Y[s], r["y"]) <= TOL, f"slot {s}"
        assert orc.max_rel_err(Y[s], r["y"]) <= 1e-2
    return layer, ws, Y, sel


def test_moe_decode_bs1_iq4_down(qk, orc, dev, layer_iq4):
    print("[case] moe bs=1 E=256 k=8 IQ4_XS down", flush=True)
    X, refs = pick_inputs(orc, layer_iq4, 1, seed=1)
    check(qk, orc, dev, layer_iq4, X, refs)


def test_moe_decode_bs1_three_launch_form(qk, orc, dev, layer_iq4, layer_q6k):
    print("[case] moe bs=1 via qkk_moe_decode_stages(ALL)", flush=True)
    for hl in (layer_iq4, layer_q6k):
        X, refs = pick_inputs(orc, hl, 1, seed=11)
        check(qk, orc, dev, hl, X, refs, stages=7)


def test_moe_decode_bs1_q6k_down(qk, orc, dev, layer_q6k):
    print("[case] moe bs=1 E=256 k=8 Q6_K down", flush=True)
    X, refs = pick_inputs(orc, layer_q6k, 1, seed=12)
    check(qk, orc, dev, layer_q6k, X, refs)


def test_moe_decode_bs1_many_steps_one_workspace(qk, orc, dev, layer_iq4):
    """Back-to-back steps on one workspace: no state may leak from one step into the next."""
    import torch
    print("[case] moe bs=1 x 50 steps on one workspace", flush=True)
    X, refs = pick_inputs(orc, layer_iq4, 5, seed=13)
    layer = layer_iq4.to_device(dev)
    ws = torch.zeros(qk.moe_workspace_bytes(layer, 1), dtype=torch.uint8, device=dev)
    Xd = torch.from_numpy(X).to(dev)
    for it in range(50):
        i = it % 5
        Y, sel = qk.moe_decode(layer, Xd[i:i + 1], ws)
        if it >= 45:
            torch.cuda.synchronize()
            ids, _, _ = sel_fields(sel)
            assert list(ids[0, :8]) == list(refs[i]["sel"].ids[:8])
            assert orc.rel_maxabs_err(Y.cpu().numpy()[0], refs[i]["y"]) <= TOL
    torch.cuda.synchronize()
    assert int(ws[:256].view(torch.int32).abs().sum()) == 0   # arrival counters are back at zero


def test_moe_decode_bs16_q6k_down(qk, orc, dev, layer_q6k):
    print("[case] moe bs=16 E=256 k=8 Q6_K down", flush=True)
    X, refs = pick_inputs(orc, layer_q6k, 16, seed=2)
    check(qk, orc, dev, layer_q6k, X, refs)


def test_moe_decode_bs16_with_the_waves_splitting_the_rows(qk, orc, dev, unrun_form, layer_q6k, layer_iq4):
    """Sixteen rows through the row-split expert kernels (the "moe_rows" switch): against the oracle, both
    down formats, and twice on one workspace with identical bits."""
    import torch
    print("[case] moe bs=16, row-split experts", flush=True)
    with qk.option("moe_rows", 1):
        for hl, seed in ((layer_q6k, 2), (layer_iq4, 5)):
            X, refs = pick_inputs(orc, hl, 16, seed=seed)
            layer, ws, Y, sel = check(qk, orc, dev, hl, X, refs)
            Y2, sel2 = qk.moe_decode(layer, torch.from_numpy(X).to(dev), ws)
            torch.cuda.synchronize()
            assert np.array_equal(Y2.cpu().numpy().view(np.uint32), Y.view(np.uint32)) and torch.equal(sel2, sel)


def test_moe_decode_bs3_iq4_down_repeatable(qk, orc, dev, layer_iq4):
    import torch
    print("[case] moe bs=3 repeat on one workspace", flush=True)
    X, refs = pick_inputs(orc, layer_iq4, 3, seed=3)
    layer, ws, Y, sel = check(qk, orc, dev, layer_iq4, X, refs)
    # same workspace, second and third call: bit-identical output (the race canary)
    for _ in range(2):
        Y2, sel2 = qk.moe_decode(layer, torch.from_numpy(X).to(dev), ws)
        torch.cuda.synchronize()
        assert np.array_equal(Y2.cpu().numpy().view(np.uint32), Y.view(np.uint32))
        assert torch.equal(sel2, sel)


def test_moe_identical_slots_share_experts(qk, orc, dev, layer_q6k):
    print("[case] moe bs=4 identical rows", flush=True)
    X, refs = pick_inputs(orc, layer_q6k, 1, seed=4)
    X4 = np.repeat(X, 4, axis=0)
    _, _, Y, _ = check(qk, orc, dev, layer_q6k, X4, refs * 4)
    for s in range(1, 4):
        assert np.array_equal(Y[s].view(np.uint32), Y[0].view(np.uint32))


@pytest.mark.parametrize("E,k,F,down", [(8, 2, 256, "iq4"), (32, 8, 512, "q6k"), (64, 10, 512, "iq4"),
                                         (512, 16, 512, "iq4"), (16, 16, 256, "q6k"), (4, 1, 1024, "iq4")])
def test_moe_decode_other_shapes(qk, orc, dev, E, k, F, down):
    print(f"[case] moe E={E} k={k} F={F} down={down}", flush=True)
    hl = qk.synth.HostLayer(seed=300 + E + k, n_ff=F, n_expert=E, n_used=k,
                            down_type=qk.IQ4_XS if down == "iq4" else qk.Q6_K)
    X, refs = pick_inputs(orc, hl, 2, seed=5, min_gap=(2e-3 if k < E else -1.0))
    check(qk, orc, dev, hl, X, refs)


def test_moe_nan_activations_keep_ids_in_range(qk, dev, layer_iq4):
    import torch
    print("[case] moe NaN activations", flush=True)
    layer = layer_iq4.to_device(dev)
    X = torch.full((2, 2048), float("nan"), device=dev)
    X[1] = float("inf")
    ws = torch.zeros(qk.moe_workspace_bytes(layer, 2), dtype=torch.uint8, device=dev)
    Y, sel = qk.moe_decode(layer, X, ws)
    torch.cuda.synchronize()
    ids, _, _ = sel_fields(sel)
    assert np.all(ids[:, :8] < 256)


@pytest.mark.parametrize("n", [1, 3])
def test_moe_tied_logits_pick_the_lower_id(qk, orc, dev, n):
    """Two experts with identical router rows have identical logits: when both are picked the lower
    id comes first, when one is picked it is the lower one (reference shaders/moe_select.comp:53-59)."""
    import torch
    print(f"[case] moe tied logits, {n} rows", flush=True)
    hl = qk.synth.HostLayer(seed=77, n_expert=16, n_used=4, n_ff=256)
    rng = np.random.default_rng(5)
    for trial in range(6):
        x = rng.standard_normal((n, 2048)).astype(np.float32)
        order = np.argsort(-(hl.gate_inp.astype(np.float64) @ x[0].astype(np.float64)))
        # trial even: duplicate the top row into a higher id (both picked); odd: duplicate the 4th pick (one picked)
        src = int(order[0] if trial % 2 == 0 else order[3])
        dst = int(max(e for e in range(16) if e != src))
        hl.gate_inp[dst] = hl.gate_inp[src]
        layer = hl.to_device(dev)
        ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
        Y, sel = qk.moe_decode(layer, torch.from_numpy(x).to(dev), ws)
        torch.cuda.synchronize()
        ids, _, _ = sel_fields(sel)
        got = [int(i) for i in ids[0, :4]]
        lo, hi = min(src, dst), max(src, dst)
        assert lo in got, (trial, got)
        if hi in got:
            assert got.index(lo) + 1 == got.index(hi), (trial, got)
        r = orc.moe_ref(hl, x[0])
        assert got == list(r["sel"].ids[:4]) or r["sel"].gap < 1e-3, (trial, got, list(r["sel"].ids[:4]))


def test_moe_argument_errors(qk, dev, layer_iq4):
    import torch
    layer = layer_iq4.to_device(dev)
    X = torch.zeros((1, 2048), device=dev)
    small = torch.zeros(256, dtype=torch.uint8, device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.moe_decode(layer, X, small)
    assert e.value.code == -5


def test_moe_n_embd_4096_rows(qk, orc, dev):
    """n_embd = 4096: up to ROWWISE_MAX rows run (each through the one-row launches); more rows need
    the expert-major path, which is built for n_embd = 2048, and are refused with a shape error."""
    import torch
    hl = qk.synth.HostLayer(seed=55, n_embd=4096, n_ff=256, n_expert=4, n_used=2)
    layer = hl.to_device(dev)
    X = np.random.default_rng(3).standard_normal((3, 4096)).astype(np.float32)
    ws = torch.zeros(qk.moe_workspace_bytes(layer, 3), dtype=torch.uint8, device=dev)
    Y, sel = qk.moe_decode(layer, torch.from_numpy(X).to(dev), ws)
    torch.cuda.synchronize()
    ids, _, _ = sel_fields(sel)
    for t in range(3):
        r = orc.moe_ref(hl, X[t])
        assert sorted(ids[t, :2]) == sorted(r["sel"].ids[:2])
        assert orc.rel_maxabs_err(Y.cpu().numpy()[t], r["y"]) <= TOL
    X5 = torch.zeros((qk.ROWWISE_MAX + 1, 4096), device=dev)
    ws5 = torch.zeros(qk.moe_workspace_bytes(layer, qk.ROWWISE_MAX + 1), dtype=torch.uint8, device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.moe_decode(layer, X5, ws5)
    assert e.value.code == -2 and "2048" in str(e.value)


def test_moe_decode_bs17_two_shared_tiles(qk, orc, dev, layer_iq4):
    """17 rows: the shared expert needs a second, one-row tile; workspace reused for a smaller call."""
    import torch
    print("[case] moe bs=17 then bs=2 on one workspace", flush=True)
    X, refs = pick_inputs(orc, layer_iq4, 17, seed=31)
    layer, ws, Y, sel = check(qk, orc, dev, layer_iq4, X, refs)
    Y2, sel2 = qk.moe_decode(layer, torch.from_numpy(X[:2]).to(dev), ws)
    torch.cuda.synchronize()
    for s in range(2):
        assert orc.rel_maxabs_err(Y2.cpu().numpy()[s], refs[s]["y"]) <= TOL


@pytest.mark.parametrize("n", [3, 40])
def test_moe_stale_workspace_stays_in_bounds(qk, orc, dev, layer_iq4, n):
    """Gate/up and down run on a workspace that no routing launch has written (arbitrary bytes, then
    small integers that look like indices but fit nothing): the numbers mean nothing, but every word the
    kernels take from the workspace is clamped to the tensors' ranges, so the launches complete.  The
    same workspace, cleared, then gives the right step."""
    import torch
    print(f"[case] moe stale workspace, {n} rows", flush=True)
    X, refs = pick_inputs(orc, layer_iq4, n, seed=40 + n)
    layer = layer_iq4.to_device(dev)
    nbytes = qk.moe_workspace_bytes(layer, n)
    Xd = torch.from_numpy(X).to(dev)
    g = torch.Generator(device=dev)
    g.manual_seed(n)
    fills = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=dev, generator=g),
             torch.randint(0, 64, (nbytes // 4,), dtype=torch.int32, device=dev, generator=g).view(torch.uint8)]
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    for fill in fills:
        ws.copy_(fill)
        qk.moe_decode(layer, Xd, ws, stages=6)
        torch.cuda.synchronize()
    ws.zero_()
    Y, sel = qk.moe_decode(layer, Xd, ws)
    torch.cuda.synchronize()
    ids, _, _ = sel_fields(sel)
    Y = Y.cpu().numpy()
    for s in range(n):
        assert list(ids[s, :8]) == list(refs[s]["sel"].ids[:8]), f"slot {s}"
        assert orc.rel_maxabs_err(Y[s], refs[s]["y"]) <= TOL, f"slot {s}"


@pytest.mark.parametrize("n", [16, 40])
def test_dirty_workspace_header_is_an_error(qk, dev, layer_iq4, n):
    """A workspace whose header was never cleared: the routing launch of the expert-major path sees the
    words behind the arrival counter and qkk_moe_workspace_status reports QKK_EINVAL, once; a cleared
    workspace leaves the status clean.  Only the routing launch runs on the dirty workspace."""
    import torch
    print(f"[case] dirty workspace header, {n} rows", flush=True)
    layer = layer_iq4.to_device(dev)
    x = torch.randn((n, 2048), device=dev)
    try:
        qk.moe_workspace_status()                   # whatever earlier tests left is taken here
    except qk.capi.QkError:
        pass
    ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
    qk.moe_decode(layer, x, ws, stages=1)
    qk.moe_workspace_status()                       # clean: no error
    ws[4:256] = 0x5A                                # the counter itself is zero, the 63 words behind it are not
    qk.moe_decode(layer, x, ws, stages=1)
    with pytest.raises(qk.capi.QkError) as e:
        qk.moe_workspace_status()
    assert e.value.code == -1 and "header" in str(e.value)
    qk.moe_workspace_status()                       # reported once, then clean again
    ws.zero_()
    qk.moe_decode(layer, x, ws, stages=1)
    qk.moe_workspace_status()


def test_moe_layer_loaded_from_gguf(qk, orc, dev, tmp_path):
    """The reference's per-layer check on a model file (`qk moe <layer>`, src/main.cpp:920-1254): the
    layer's tensors come out of a GGUF file through the library's reader, the step runs on them,
    and the result is held against the CPU restatement on the same bytes.  The file is synthetic
    (no model file is available): same tensor names, types, shapes and metadata keys."""
    import torch
    print("[case] moe layer from a GGUF file", flush=True)
    hl = qk.synth.HostLayer(seed=900, n_expert=16, n_used=4, down_type=qk.Q6_K)
    path = tmp_path / "model.gguf"
    qk.gguf.write(path, {"general.architecture": "qwen3next", "qwen3next.expert_used_count": 4},
                  qk.gguf.layer_tensors(hl, 5))
    with qk.gguf.File(path) as f:
        layer = f.moe_layer(5, dev)
    assert (layer.n_embd, layer.n_ff, layer.n_expert, layer.n_used, layer.down_type) == (2048, 512, 16, 4, qk.Q6_K)
    for n in (1, 6):
        X, refs = pick_inputs(orc, hl, n, seed=60 + n)
        ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
        Y, sel = qk.moe_decode(layer, torch.from_numpy(X).to(dev), ws)
        torch.cuda.synchronize()
        ids, w, _ = sel_fields(sel)
        Y = Y.cpu().numpy()
        for s in range(n):
            assert list(ids[s, :4]) == list(refs[s]["sel"].ids[:4])
            assert np.max(np.abs(w[s, :4] - np.array(refs[s]["sel"].w[:4]))) <= 1e-4
            assert orc.rel_maxabs_err(Y[s], refs[s]["y"]) <= TOL


@pytest.mark.parametrize("n", [1, 2, 16, 40])
def test_moe_decode_tail(qk, orc, dev, layer_iq4, n):
    """Step + residual + next layer's RMS norm in one call against the oracle's step followed by its
    norm (reference src/main.cpp:4379-4402); the plain step on the same rows gives the same picks,
    and S - resid is that step's output up to fp32 rounding of the sum."""
    import torch
    print(f"[case] moe step with layer tail, {n} rows", flush=True)
    X, refs = pick_inputs(orc, layer_iq4, n, seed=70 + n)
    rng = np.random.default_rng(n)
    resid = rng.standard_normal((n, 2048)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 2048).astype(np.float32)
    y = np.stack([r["y"] for r in refs])
    want_s, want_xn = orc.add_rms(resid, w, 1e-6, b=y, want_sum=True)
    layer = layer_iq4.to_device(dev)
    ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
    Xd, Rd, Wd = (torch.from_numpy(a).to(dev) for a in (X, resid, w))
    S, Xn, sel = qk.moe_decode_tail(layer, Xd, Rd, Wd, ws)
    torch.cuda.synchronize()
    ids, _, _ = sel_fields(sel)
    for s in range(n):
        assert list(ids[s, :8]) == list(refs[s]["sel"].ids[:8])
    scale_y = np.max(np.abs(y))
    assert np.max(np.abs(S.cpu().numpy() - want_s)) <= TOL * scale_y
    assert orc.rel_maxabs_err(Xn.cpu().numpy(), want_xn) <= TOL
    # in place: the residual buffer receives S; same bits as out of place
    S2, Xn2, _ = qk.moe_decode_tail(layer, Xd, Rd, Wd, ws, S=Rd)
    torch.cuda.synchronize()
    assert S2.data_ptr() == Rd.data_ptr() and torch.equal(S2, S) and torch.equal(Xn2, Xn)
    with pytest.raises(qk.QkError):
        qk.moe_decode_tail(layer, Xd, Rd, Wd, ws, Xn=Xd)


@pytest.mark.parametrize("which", ["iq4", "q6k"])
def test_moe_layer_rows_one_row(qk, orc, dev, layer_iq4, layer_q6k, which):
    """One row's whole MoE block in place -- norm inside the router and gate/up launches, residual
    added by the down launch -- against the oracle's norm, step and sum
    (reference src/main.cpp:4376-4402)."""
    import torch
    hl = layer_iq4 if which == "iq4" else layer_q6k
    print(f"[case] moe layer row, down {which}", flush=True)
    layer = hl.to_device(dev)
    ws = torch.zeros(qk.moe_workspace_bytes(layer, 1), dtype=torch.uint8, device=dev)
    rng = np.random.default_rng(17)
    w = rng.uniform(0.5, 1.5, 2048).astype(np.float32)
    Wd = torch.from_numpy(w).to(dev)
    done = 0
    for trial in range(40):
        # a residual row far from unit scale: the norm, not the input, must bring it to O(1)
        s0 = (rng.standard_normal(2048) * rng.choice([0.03, 1.0, 40.0])).astype(np.float32)
        xn = orc.add_rms(s0, w, 1e-6)
        r = orc.moe_ref(hl, xn)
        lw = np.log(np.array(sorted(r["sel"].w[:8], reverse=True)))
        if r["sel"].gap <= 2e-3 or np.min(-np.diff(lw)) <= 2e-3:
            continue
        Sd = torch.from_numpy(s0).to(dev).reshape(1, 2048)
        S, sel = qk.moe_layer_rows(layer, Sd, Wd, ws)
        torch.cuda.synchronize()
        assert S.data_ptr() == Sd.data_ptr()
        ids, wts, wsh = sel_fields(sel)
        assert list(ids[0, :8]) == list(r["sel"].ids[:8])
        assert np.max(np.abs(wts[0, :8] - np.array(r["sel"].w[:8]))) <= 1e-4
        got = S.cpu().numpy()[0]
        assert np.max(np.abs((got - s0) - r["y"])) <= TOL * np.max(np.abs(r["y"])) + 2e-7 * np.max(np.abs(s0))
        # the same bits as the plain step on the normalised row plus the residual, up to the
        # place where the scale is applied (after the dot products instead of before)
        Y, _ = qk.moe_decode(layer, torch.from_numpy(xn).to(dev).reshape(1, 2048), ws)
        torch.cuda.synchronize()
        assert orc.rel_maxabs_err(got - s0, Y.cpu().numpy()[0]) <= 1e-4
        done += 1
        if done == 4:
            break
    assert done == 4
    with pytest.raises(qk.QkError):
        qk.moe_layer_rows(layer, Sd, None, ws)


@pytest.mark.parametrize("rows", [1, 3, 10])
def test_moe_layer_rows_with_a_mixer_output_on_top(qk, dev, layer_iq4, layer_q6k, rows):
    """qkk_moe_layer_rows_add: the first launch adds the mixer's rows to the residual while it loads
    and stores the sum for the other two.  Bit for bit qkk_moe_layer_rows on rows added beforehand
    (which the oracle pins above); T holds the sum."""
    import torch
    print(f"[case] moe layer rows + mixer output, rows={rows}", flush=True)
    for hl in (layer_iq4, layer_q6k):
        layer = hl.to_device(dev)
        ws = torch.zeros(qk.moe_workspace_bytes(layer, rows), dtype=torch.uint8, device=dev)
        g = torch.Generator(device="cpu").manual_seed(rows)
        S0 = (torch.randn(rows, 2048, generator=g) * 3).to(dev)
        mix = torch.randn(rows, 2048, generator=g).to(dev)
        W = (0.5 + torch.rand(2048, generator=g)).to(dev)
        want, sel_w = qk.moe_layer_rows(layer, (S0 + mix).clone(), W, ws)
        want, sel_w = want.clone(), sel_w.clone()
        S, T = S0.clone(), torch.full_like(S0, float("nan"))
        got, sel = qk.moe_layer_rows(layer, S, W, ws, mix=mix, T=T)
        torch.cuda.synchronize()
        assert torch.equal(T, S0 + mix)
        assert torch.equal(got, want) and torch.equal(sel, sel_w)
    with pytest.raises(qk.QkError):   # T must be a buffer of its own
        qk.moe_layer_rows(layer, S, W, ws, mix=mix, T=S)
    with pytest.raises(qk.QkError):   # more rows than the row-wise launches take
        big = torch.zeros(11, 2048, device=dev)
        qk.moe_layer_rows(layer, big, W, torch.zeros(qk.moe_workspace_bytes(layer, 11), dtype=torch.uint8, device=dev),
                          mix=big.clone(), T=big.clone())


def test_rows_up_to_the_rowwise_limit_do_not_depend_on_company(qk, dev, layer_iq4):
    """Up to ROWWISE_MAX rows every row runs the one-row launches: the same row gives the same bits
    alone, among other rows and at another position; one row more takes the expert-major path and
    agrees to the tolerance.  The same for the block with the norm in front."""
    import torch
    layer = layer_iq4.to_device(dev)
    nmax = qk.ROWWISE_MAX
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    X = torch.randn((nmax + 1, 2048), device=dev, generator=g)
    W = torch.rand(2048, device=dev, generator=g) + 0.5
    ws = torch.zeros(qk.moe_workspace_bytes(layer, nmax + 1), dtype=torch.uint8, device=dev)
    alone = torch.cat([qk.moe_decode(layer, X[i:i + 1].contiguous(), ws)[0] for i in range(nmax + 1)])
    Y, sel = qk.moe_decode(layer, X[:nmax].contiguous(), ws)
    assert torch.equal(Y, alone[:nmax])
    perm = torch.tensor([3, 0, 2], device=dev)
    Yp, _ = qk.moe_decode(layer, X[perm].contiguous(), ws)
    assert torch.equal(Yp, alone[perm])
    Yg, selg = qk.moe_decode(layer, X.contiguous(), ws)         # one row more: expert-major path
    torch.cuda.synchronize()
    scale = float(alone.abs().max())
    assert float((Yg - alone).abs().max()) <= TOL * scale
    assert np.array_equal(sel_fields(selg)[0][:nmax, :8], sel_fields(sel)[0][:, :8])
    # the block with the norm in front
    one = torch.cat([qk.moe_layer_rows(layer, X[i:i + 1].clone(), W, ws)[0] for i in range(nmax)])
    S, _ = qk.moe_layer_rows(layer, X[:nmax].clone(), W, ws)
    torch.cuda.synchronize()
    assert torch.equal(S, one)
    with pytest.raises(qk.QkError) as e:
        qk.moe_layer_rows(layer, X.clone(), W, ws)
    assert e.value.code == -2


@pytest.mark.parametrize("n", [16, 40])
def test_expert_major_rows_do_not_depend_on_company(qk, dev, layer_q6k, n):
    """The expert-major path (more than ROWWISE_MAX rows) groups the rows' picks by expert, sixteen pairs to
    a matrix-core tile -- but a row's sums never mix with its tile companions' and the picks are folded in
    pick order, so a row's result does not depend on which rows it is batched with or where it stands:
    the rows permuted give the outputs permuted, and a subset of the rows (still above the limit) gives
    the subset of the outputs, bit for bit."""
    import torch
    print(f"[case] expert-major rows and their company, {n} rows", flush=True)
    layer = layer_q6k.to_device(dev)
    g = torch.Generator(device=dev)
    g.manual_seed(n)
    X = torch.randn((n, 2048), device=dev, generator=g)
    ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
    Y, sel = qk.moe_decode(layer, X, ws)
    Y, sel = Y.clone(), sel.clone()
    perm = torch.randperm(n, device=dev, generator=g)
    Yp, selp = qk.moe_decode(layer, X[perm].contiguous(), ws)
    torch.cuda.synchronize()
    assert torch.equal(selp, sel[perm]) and torch.equal(Yp, Y[perm])
    m = qk.ROWWISE_MAX + 1
    Ys, sels = qk.moe_decode(layer, X[n - m:].contiguous(), ws)   # the last eleven rows alone
    torch.cuda.synchronize()
    assert torch.equal(sels, sel[n - m:]) and torch.equal(Ys, Y[n - m:])


def test_one_workspace_serves_changing_row_counts(qk, dev, layer_q6k):
    """An engine keeps one workspace and its step's row count changes from call to call (both
    paths, whose workspace areas lie at offsets that depend on the row count): every call must give
    the bits it gives on a freshly cleared workspace."""
    import torch
    layer = layer_q6k.to_device(dev)
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    X = torch.randn((16, 2048), device=dev, generator=g)
    shared = torch.zeros(qk.moe_workspace_bytes(layer, 16), dtype=torch.uint8, device=dev)
    for n in (16, 11, 3, 12, 1, 10, 16, 2, 13):
        fresh = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
        want, wsel = qk.moe_decode(layer, X[:n].contiguous(), fresh)
        got, gsel = qk.moe_decode(layer, X[:n].contiguous(), shared)
        torch.cuda.synchronize()
        assert torch.equal(got, want) and torch.equal(gsel, wsel), n


def test_group_pairs_matches_oracle(qk, orc, dev):
    import torch
    print("[case] group pairs", flush=True)
    rng = np.random.default_rng(6)
    for n_tokens, E, k in [(16, 256, 8), (128, 256, 8), (3, 8, 2), (512, 256, 8), (1, 512, 16)]:
        sel = np.zeros((n_tokens, 40), dtype=np.uint32)
        for t in range(n_tokens):
            sel[t, :k] = rng.choice(E, size=k, replace=False)
        sel[0, 0] = E + 3
        sb = sel.view(np.uint8).reshape(n_tokens, 160)
        off, pairs = qk.moe_group_pairs(torch.from_numpy(sb.copy()).to(dev), n_tokens, E, k)
        woff, wpairs = orc.group_pairs(sb, n_tokens, E, k)
        assert np.array_equal(off.cpu().numpy().view(np.uint32), woff)
        assert np.array_equal(pairs.cpu().numpy().view(np.uint32), wpairs)
