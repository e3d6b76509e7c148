"""LM head (Q6_K) with fused greedy sampling: the token id must equal the oracle's argmax of
the double-accumulated logits; logits within 1e-3 relative max-abs."""
import numpy as np
import pytest

# every test runs on both forms of the one-row kernels (conftest.one_row_form)
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("one_row_form")]


def head_case(qk, orc, dev, V, K, batch, seed, want_logits=True):
    import torch
    print(f"[case] head V={V} K={K} batch={batch}", flush=True)
    W = qk.synth.tensor_host(qk.Q6_K, V, K, seed)
    x = np.random.default_rng(seed + 1).standard_normal((batch, K)).astype(np.float32)
    ws = torch.zeros(qk.head_workspace_bytes(V, batch), dtype=torch.uint8, device=dev)
    Wd, xd = torch.from_numpy(W).to(dev), torch.from_numpy(x).to(dev)
    tok, logits = qk.head_argmax(Wd, xd, V, K, ws, want_logits=want_logits)
    torch.cuda.synchronize()
    ref_logits = orc.gemv(orc.Q6_K, W, x, V, K)
    want = [orc.argmax(ref_logits[b]) for b in range(batch)]
    # the comparison is only meaningful when the winner's margin exceeds fp32 noise
    for b in range(batch):
        srt = np.sort(ref_logits[b])
        assert srt[-1] - srt[-2] > 1e-5 * abs(srt[-1]), "ambiguous fixture: pick another seed"
    assert list(tok.cpu().numpy()) == want
    if want_logits:
        assert orc.rel_maxabs_err(logits.cpu().numpy(), ref_logits) <= 1e-3
    # second call on the same workspace (counters must have been rearmed), no logits
    tok2, _ = qk.head_argmax(Wd, xd, V, K, ws, want_logits=False)
    assert list(tok2.cpu().numpy()) == want
    return tok


def test_head_full_vocab_bs1(qk, orc, dev):
    head_case(qk, orc, dev, 151936, 2048, 1, seed=10)


def test_head_full_vocab_bs16(qk, orc, dev):
    head_case(qk, orc, dev, 151936, 2048, 16, seed=11)


@pytest.mark.parametrize("V,K,batch", [(1000, 2048, 2), (4097, 2048, 1), (3, 2048, 1), (777, 4096, 3), (4097, 2048, 16),
                                           (33, 2048, 5), (16, 2048, 9)])
def test_head_ragged(qk, orc, dev, V, K, batch):
    head_case(qk, orc, dev, V, K, batch, seed=12 + V)


@pytest.mark.parametrize("V,batch", [(151936, 16), (151936, 2), (4097, 16), (128, 5), (33, 9)])
def test_head_with_the_waves_splitting_the_rows(qk, orc, dev, unrun_form, V, batch):
    """The "head_rows" switch: 2..16 rows with a wave owning 16 vocabulary rows for all of K."""
    with qk.option("head_rows", 1):
        head_case(qk, orc, dev, V, 2048, batch, seed=40 + batch)


@pytest.mark.parametrize("V", [151936, 4097, 3])
def test_head_with_the_norm_in_front(qk, orc, dev, unrun_form, V):
    """qkk_head_argmax_norm: the output norm inside the head's launch, against the oracle's norm (double)
    followed by its GEMV and argmax."""
    import torch
    print(f"[case] head with norm V={V}", flush=True)
    K = 2048
    W = qk.synth.tensor_host(qk.Q6_K, V, K, 40 + V % 7)
    rng = np.random.default_rng(V)
    x = (rng.standard_normal((1, K)) * 2.0).astype(np.float32)
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    ws = torch.zeros(qk.head_workspace_bytes(V, 1), dtype=torch.uint8, device=dev)
    up = lambda a: torch.from_numpy(a).to(dev)
    Wd, xd, wd = up(W), up(x), up(w)
    tok, logits = qk.head_argmax_norm(Wd, xd, wd, V, K, ws, want_logits=True)
    torch.cuda.synchronize()
    ref = orc.gemv(orc.Q6_K, W, orc.add_rms(x[0], w, 1e-6), V, K)
    srt = np.sort(ref)
    if V > 1:
        assert srt[-1] - srt[-2] > 1e-5 * abs(srt[-1]), "ambiguous fixture: pick another seed"
    assert int(tok.cpu()[0]) == orc.argmax(ref)
    assert orc.rel_maxabs_err(logits.cpu().numpy()[0], ref) <= 1e-3
    tok2, _ = qk.head_argmax_norm(Wd, xd, wd, V, K, ws)      # the counters were rearmed
    assert int(tok2.cpu()[0]) == int(tok.cpu()[0])


def test_head_full_vocab_scaling_is_exact(qk, dev):
    """At the full vocabulary (151,936 x 2048): doubling the activation row doubles every logit exactly
    (a power of two changes no rounding on the fp32 path) and leaves the token unchanged; so does the
    row given twice in a batch of one call each."""
    import torch
    print("[case] head properties at the full vocabulary", flush=True)
    V, K = 151936, 2048
    W = qk.synth.blocks_device(qk.Q6_K, V * (K // 256), 21, dev).reshape(-1)
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    x = torch.randn((1, K), device=dev, generator=g)
    ws = torch.zeros(qk.head_workspace_bytes(V, 1), dtype=torch.uint8, device=dev)
    tok, logits = qk.head_argmax(W, x, V, K, ws, want_logits=True)
    tok2, logits2 = qk.head_argmax(W, (2 * x).contiguous(), V, K, ws, want_logits=True)
    torch.cuda.synchronize()
    assert torch.equal(logits2, 2 * logits) and int(tok2[0]) == int(tok[0])
    assert int(tok[0]) == int(torch.argmax(logits[0]))


def test_head_ties_pick_lowest_id(qk, dev):
    import torch
    print("[case] head ties", flush=True)
    V, K = 5000, 2048
    W = qk.synth.tensor_host(qk.Q6_K, V, K, 13).reshape(V, -1).copy()
    x = np.random.default_rng(14).standard_normal((1, K)).astype(np.float32)
    ws = torch.zeros(qk.head_workspace_bytes(V, 1), dtype=torch.uint8, device=dev)
    tok, logits = qk.head_argmax(torch.from_numpy(W.reshape(-1)).to(dev), torch.from_numpy(x).to(dev), V, K, ws, True)
    best = int(tok[0])
    # copy the winning row to three other places: identical logits, the lowest id must win
    for r in (4999, 17, 2500):
        W[r] = W[best]
    tok, _ = qk.head_argmax(torch.from_numpy(W.reshape(-1)).to(dev), torch.from_numpy(x).to(dev), V, K, ws)
    assert int(tok[0]) == min(best, 17)


def test_argmax_standalone(qk, orc, dev):
    import torch
    rng = np.random.default_rng(15)
    v = rng.standard_normal((4, 151936)).astype(np.float32)
    v[1, [5, 100000]] = 9.0
    v[2, :] = -np.inf
    v[3, 0] = np.nan
    tok = qk.argmax(torch.from_numpy(v).to(dev)).cpu().numpy()
    assert tok[0] == orc.argmax(v[0]) and tok[1] == 5 and tok[2] == 0
    assert tok[3] == int(np.nanargmax(v[3]))   # a NaN never wins on the device (argmax1.comp:27)
