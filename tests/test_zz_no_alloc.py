"""qkk_moe_decode_static -- the fused MoE step on the library's own static device workspace, for
callers that cannot allocate -- through the C ABI against qkk_moe_decode on a caller-owned
workspace.  Both run the same kernels, so the bar is bit-exact: expert ids, router weights and
outputs.  Two calls in a row share the array, the second with fewer rows (what the first left in
the array must not reach the second's results); the sizes cover the expert-major path (16 rows),
the row-wise path (3 rows) and the one-row launches.  The first case also holds the static entry
point against the oracle.  Collected last: a failure here must not hide the other GPU tests."""
import numpy as np
import pytest

# every test runs on both forms of the one-row kernels (conftest.one_row_form)
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("one_row_form")]


def run_pair(qk, dev, layer, X):
    """(Y, sel) of the existing entry point and of the static one on the same rows."""
    import torch
    n = X.shape[0]
    Xd = torch.from_numpy(X).to(dev)
    ws = torch.zeros(qk.moe_workspace_bytes(layer, n), dtype=torch.uint8, device=dev)
    Y0, sel0 = qk.moe_decode(layer, Xd, ws)
    Y1 = torch.full_like(Y0, float("nan"))
    sel1 = torch.zeros((n, 160), dtype=torch.uint8, device=dev)
    qk.moe_decode_static(layer, Xd, Y1, sel1)
    torch.cuda.synchronize()
    return Y0.cpu().numpy(), sel0.cpu().numpy(), Y1.cpu().numpy(), sel1.cpu().numpy()


@pytest.mark.parametrize("down", ["iq4_xs", "q6_k"])
def test_static_workspace_matches_caller_workspace(qk, orc, dev, down):
    hl = qk.synth.HostLayer(seed=321, down_type=qk.IQ4_XS if down == "iq4_xs" else qk.Q6_K)
    layer = hl.to_device(dev)
    rng = np.random.default_rng(5)
    for n in (16, 3, 12, 1):   # each call after the first finds the previous call's contents in the array
        print(f"[case] qkk_moe_decode_static {down} rows={n}", flush=True)
        X = rng.standard_normal((n, hl.n_embd)).astype(np.float32)
        Y0, sel0, Y1, sel1 = run_pair(qk, dev, layer, X)
        assert np.array_equal(sel0, sel1), f"router records differ at {n} rows"
        assert np.array_equal(Y0.view(np.uint32), Y1.view(np.uint32)), f"outputs differ at {n} rows"
        if n == 1:   # and the oracle agrees with what both produced
            r = orc.moe_ref(hl, X[0])
            ids = sel1.view(np.uint32).reshape(-1, 40)[0, :hl.n_used]
            if r["sel"].gap > 2e-3:
                assert sorted(ids) == sorted(r["sel"].ids[:hl.n_used])
                assert orc.rel_maxabs_err(Y1[0], r["y"]) <= 1e-3


def test_static_workspace_limits(qk, dev):
    import torch
    hl = qk.synth.HostLayer(seed=9, n_expert=32)
    layer = hl.to_device(dev)
    n = qk.MOE_STATIC_MAX_SLOTS + 1
    X = torch.zeros((n, hl.n_embd), device=dev)
    Y = torch.zeros_like(X)
    sel = torch.zeros((n, 160), dtype=torch.uint8, device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.moe_decode_static(layer, X, Y, sel)
    assert e.value.code == -2 and "outside 1..16" in str(e.value)
    # a layer shape whose workspace does not fit the array is refused, not truncated
    wide = qk.synth.HostLayer(seed=10, n_expert=16, n_used=16, n_embd=4096, n_ff=1024)
    lw = wide.to_device(dev)
    assert qk.moe_workspace_bytes(lw, 16) > qk.MOE_STATIC_BYTES
    X = torch.zeros((16, 4096), device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.moe_decode_static(lw, X, torch.zeros_like(X), torch.zeros((16, 160), dtype=torch.uint8, device=dev))
    assert e.value.code == -5
