"""Batched-prefill entry points against the oracle: the MoE step over a chunk of tokens
(per token identical to the decode step: exact expert ids in pick order, outputs within 1e-3
relative max-abs) and the Q8_0 dense projection GEMM (reference bar for fp16-input tiles:
max error < 2e-3 * rms, src/main.cpp:5659-5662)."""
import numpy as np
import pytest

from test_gpu_moe import pick_inputs, sel_fields

pytestmark = pytest.mark.gpu


def prefill_case(qk, orc, dev, hl, n_tokens, seed):
    import torch
    X, refs = pick_inputs(orc, hl, n_tokens, seed=seed)
    layer = hl.to_device(dev)
    ws = torch.zeros(qk.moe_prefill_workspace_bytes(layer, n_tokens), dtype=torch.uint8, device=dev)
    Y, sel = qk.moe_prefill(layer, torch.from_numpy(X).to(dev), ws)
    torch.cuda.synchronize()
    Y = Y.cpu().numpy()
    ids, w, wsh = sel_fields(sel)
    k = hl.n_used
    worst = 0.0
    for t in range(n_tokens):
        r = refs[t]
        assert list(ids[t, :k]) == list(r["sel"].ids[:k]), f"token {t}"
        assert np.max(np.abs(w[t, :k] - np.array(r["sel"].w[:k]))) <= 1e-4
        assert abs(wsh[t] - r["sel"].w_shared) <= 1e-4
        worst = max(worst, orc.rel_maxabs_err(Y[t], r["y"]))
    assert worst <= 1e-3, worst
    # second call on the same workspace: identical bits
    Y2, _ = qk.moe_prefill(layer, torch.from_numpy(X).to(dev), ws)
    torch.cuda.synchronize()
    assert np.array_equal(Y2.cpu().numpy().view(np.uint32), Y.view(np.uint32))


def test_moe_prefill_128_tokens_iq4_down(qk, orc, dev):
    print("[case] moe prefill 128 tokens IQ4_XS down", flush=True)
    hl = qk.synth.HostLayer(seed=100, down_type=qk.IQ4_XS)
    prefill_case(qk, orc, dev, hl, 128, seed=21)


def test_moe_prefill_40_tokens_q6k_down(qk, orc, dev):
    print("[case] moe prefill 40 tokens Q6_K down", flush=True)
    hl = qk.synth.HostLayer(seed=200, down_type=qk.Q6_K)
    prefill_case(qk, orc, dev, hl, 40, seed=22)


def test_moe_prefill_small_layer_many_pairs_per_expert(qk, orc, dev):
    print("[case] moe prefill 96 tokens on 16 experts", flush=True)
    hl = qk.synth.HostLayer(seed=300, n_expert=16, n_used=4, down_type=qk.IQ4_XS)
    prefill_case(qk, orc, dev, hl, 96, seed=23)


@pytest.mark.parametrize("down,n,E,k", [("iq4", 128, 256, 8), ("q6k", 40, 256, 8), ("iq4", 96, 16, 4)])
def test_moe_prefill_with_the_waves_splitting_the_rows(qk, orc, dev, unrun_form, down, n, E, k):
    """The "moe_rows" switch: the routed experts' gate/up and down projections with a wave owning 16 weight
    rows for all of K and the pairs' activations shared through LDS.  The oracle's ids, weights and outputs
    per token, and the ids of the default (K-split) kernels; experts with a few pairs (256 experts) and with
    several tiles of 16 (16 experts)."""
    import torch
    print(f"[case] moe prefill, row-split experts: {n} tokens, {E} experts, {down} down", flush=True)
    hl = qk.synth.HostLayer(seed=400 + n, n_expert=E, n_used=k, down_type=qk.IQ4_XS if down == "iq4" else qk.Q6_K)
    with qk.option("moe_rows", 1):
        prefill_case(qk, orc, dev, hl, n, seed=24)
        X, _ = pick_inputs(orc, hl, n, seed=24)
        layer = hl.to_device(dev)
        ws = torch.zeros(qk.moe_prefill_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
        _, sel_rows = qk.moe_prefill(layer, torch.from_numpy(X).to(dev), ws)
        sel_rows = sel_rows.clone()
    _, sel_k = qk.moe_prefill(layer, torch.from_numpy(X).to(dev), ws)
    torch.cuda.synchronize()
    assert torch.equal(sel_rows, sel_k)


def test_moe_step_in_hip_graph_matches_eager(qk, dev):
    """The many-row step forks the shared expert onto a side stream of the library and joins it back
    with events: captured into a HIP graph it must replay to the eager result every time, with
    eager work of the program between the replays; likewise the few-row step (no fork)."""
    import torch
    print("[case] moe step captured in a HIP graph, 40 and 5 rows", flush=True)
    hl = qk.synth.HostLayer(seed=400, n_expert=32, n_used=4, down_type=qk.IQ4_XS)
    layer = hl.to_device(dev)
    for n in (40, 5):
        rng = np.random.default_rng(50 + n)
        Xs = [torch.from_numpy(rng.standard_normal((n, 2048)).astype(np.float32)).to(dev) for _ in range(3)]
        ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
        eager = []
        for X in Xs:
            Y, sel = qk.moe_decode(layer, X, ws)
            torch.cuda.synchronize()
            eager.append((Y.clone(), sel.clone()))
        Xg = Xs[0].clone()
        Yg = torch.empty_like(Xg)
        selg = torch.zeros((n, 160), dtype=torch.uint8, device=dev)
        side = torch.cuda.Stream()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            qk.moe_decode(layer, Xg, ws, Yg, selg)
        torch.cuda.synchronize()
        for rep in range(6):
            i = rep % 3
            Xg.copy_(Xs[i])
            scratch = (Xs[i] * 2).sum()      # unrelated eager work between replays
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(Yg, eager[i][0]), (n, rep)
            assert torch.equal(selg, eager[i][1]), (n, rep)
            assert torch.isfinite(scratch)


@pytest.mark.parametrize("M,K,N", [(8192, 2048, 128), (100, 96, 5), (64, 32, 33), (130, 2048, 200), (4096, 4096, 48),
                                   (300, 256, 40), (96, 512, 64), (1000, 1024, 17), (17, 2048, 8), (2048, 2048, 7),
                                   (7, 64, 1), (1024, 512, 16)])
def test_gemm_q8_0(qk, orc, dev, M, K, N):
    import torch
    print(f"[case] gemm q8_0 M={M} K={K} N={N}", flush=True)
    W = qk.synth.tensor_host(qk.Q8_0, M, K, seed=7, d_scale=1e-2)
    X = np.random.default_rng(8).uniform(-1, 1, (N, K)).astype(np.float32)
    Y = qk.gemm_q8_0(torch.from_numpy(W).to(dev), torch.from_numpy(X).to(dev), M, K).cpu().numpy()
    want = orc.gemm_q8_0(W, X, M, K)
    assert Y.shape == want.shape == (N, M)
    assert orc.max_err_over_rms(Y, want) < 2e-3      # the reference's bar for fp16-input tiles
    assert orc.rel_maxabs_err(Y, want) <= 1e-3


@pytest.mark.parametrize("name,M,K,N", [("q8_0", 8192, 2048, 128), ("q8_0", 4096, 4096, 200), ("q6_k", 2048, 2048, 128), ("iq4_xs", 2048, 512, 300),
                                        ("iq3_xxs", 1000, 2048, 64), ("q8_0", 50, 256, 1024)])
def test_gemm_with_every_weight_tile_decoded_once(qk, orc, dev, unrun_form, name, M, K, N):
    """The "gemm_tiled" switch: 64 and more activation rows through the kernel that owns 32 weight rows and
    128 activation rows per workgroup, against the oracle's double-precision product (the reference's bar for
    its half-precision tiles, src/main.cpp:5659-5662, and the per-element bar) and against the cooperative
    stream; the BASELINE shape of the prefill chunk first."""
    import torch
    print(f"[case] tiled gemm {name} M={M} K={K} N={N}", flush=True)
    t = {"q8_0": qk.Q8_0, "q6_k": qk.Q6_K, "iq4_xs": qk.IQ4_XS, "iq3_xxs": qk.IQ3_XXS}[name]
    W = qk.synth.tensor_host(t, M, K, seed=7)
    X = np.random.default_rng(8).uniform(-1, 1, (N, K)).astype(np.float32)
    Wd, Xd = torch.from_numpy(W).to(dev), torch.from_numpy(X).to(dev)
    base = qk.gemv(t, Wd, Xd, M, K).cpu().numpy()
    with qk.option("gemm_tiled", 1):
        Y = (qk.gemm_q8_0(Wd, Xd, M, K) if t == qk.Q8_0 else qk.gemv(t, Wd, Xd, M, K)).cpu().numpy()
    rows = range(N) if N * M <= 1 << 18 else list(range(0, N, max(1, N // 24))) + [N - 1]   # the oracle is a scalar loop
    want = np.stack([orc.gemv(t, W, X[n], M, K) for n in rows])
    assert orc.max_err_over_rms(Y[list(rows)], want) < 2e-3
    assert orc.rel_maxabs_err(Y[list(rows)], want) <= 1e-3
    assert orc.rel_maxabs_err(Y, base) <= 1e-5


def test_gemm_q8_0_matches_gemv_rows(qk, dev):
    """The GEMM and the GEMV read the same blocks: row by row they agree to fp16-weight rounding."""
    import torch
    M, K, N = 512, 2048, 16
    W = torch.from_numpy(qk.synth.tensor_host(qk.Q8_0, M, K, seed=9)).to(dev)
    X = torch.randn((N, K), device=dev)
    a = qk.gemm_q8_0(W, X, M, K)
    b = qk.gemv(qk.Q8_0, W, X, M, K)
    assert torch.max(torch.abs(a - b)) <= 1e-3 * torch.max(torch.abs(b))


def test_gemm_argument_errors(qk, dev):
    import torch
    W = torch.zeros(34 * 4, dtype=torch.uint8, device=dev)
    X = torch.zeros((2, 40), device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.gemm_q8_0(W, X, 1, 40)
    assert e.value.code == -2
