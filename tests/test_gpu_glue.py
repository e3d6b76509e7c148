"""Layer glue through the C ABI against the oracle: residual sums bit-exact (fp32 adds in the
shaders' order), normalised rows within 1e-5 relative max-abs (the device sums squares in fp32,
the CPU checker in double, reference src/main.cpp:1685-1690), embedding rows bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rel(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))


@pytest.mark.parametrize("rows,n", [(1, 2048), (16, 2048), (3, 4096), (2, 8192), (5, 100), (1, 7), (4, 12288),
                                    (128, 2048)])
def test_norm_family(qk, orc, dev, rows, n):
    import torch
    print(f"[case] norms rows={rows} n={n}", flush=True)
    rng = np.random.default_rng(rows * 131 + n)
    a, b, c = (rng.standard_normal((rows, n)).astype(np.float32) * np.float32(s) for s in (1.0, 0.5, 3.0))
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    eps = 1e-6
    A, B, Cc, W = (torch.from_numpy(x).to(dev) for x in (a, b, c, w))

    xn = qk.rmsnorm(A, W, eps).cpu().numpy()
    assert rel(xn, orc.add_rms(a, w, eps)) <= TOL

    y, xn = qk.add_rmsnorm(A, B, W, eps)
    ws, wxn = orc.add_rms(a, w, eps, b=b, want_sum=True)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert rel(xn.cpu().numpy(), wxn) <= TOL

    s, xn = qk.add_rms3(A, B, Cc, W, eps)
    ws, wxn = orc.add_rms(a, w, eps, b=b, c=c, want_sum=True)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert rel(xn.cpu().numpy(), wxn) <= TOL

    v = qk.vec_add(A, B).cpu().numpy()
    assert np.array_equal(v.view(np.uint32), (a + b).view(np.uint32))


def test_norms_in_place_and_unaligned(qk, orc, dev):
    """The residual row may be updated in place (y = a, xn = b); rows that do not start on 16 bytes
    take the scalar kernel: same results."""
    import torch
    print("[case] norms in place / unaligned", flush=True)
    rng = np.random.default_rng(77)
    rows, n = 3, 2048
    a, b = rng.standard_normal((2, rows, n)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    ws, wxn = orc.add_rms(a, w, 1e-6, b=b, want_sum=True)
    A, B, W = (torch.from_numpy(x).to(dev) for x in (a, b, w))
    qk.add_rmsnorm(A, B, W, 1e-6, y=A, xn=B)
    assert np.array_equal(A.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert rel(B.cpu().numpy(), wxn) <= TOL
    # unaligned: views that start one float into a larger buffer
    buf = torch.zeros(3 * rows * n + 3, device=dev)
    A2 = buf[1:1 + rows * n].view(rows, n)
    A2.copy_(torch.from_numpy(a))
    Bd = torch.from_numpy(b).to(dev)
    y, xn = qk.add_rmsnorm(A2, Bd, W, 1e-6)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert rel(xn.cpu().numpy(), wxn) <= TOL
    qk.add_rmsnorm(A2, Bd, W, 1e-6, y=A2, xn=Bd)   # scalar kernel, in place
    assert np.array_equal(A2.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert rel(Bd.cpu().numpy(), wxn) <= TOL


def test_norm_is_deterministic_and_handles_zero_rows(qk, dev):
    import torch
    x = torch.randn((16, 2048), device=dev)
    w = torch.rand(2048, device=dev) + 0.5
    a, b = qk.rmsnorm(x, w), qk.rmsnorm(x, w)
    assert torch.equal(a, b)
    z = qk.rmsnorm(torch.zeros((2, 2048), device=dev), w, 1e-6)
    assert torch.equal(z, torch.zeros_like(z))


@pytest.mark.parametrize("name,t", [("q6_k", 14), ("q8_0", 8), ("iq4_xs", 23), ("iq3_xxs", 18)])
def test_embed_bitwise(qk, orc, dev, name, t):
    import torch
    print(f"[case] embed {name}", flush=True)
    V, K = 300, 2048
    W = qk.synth.tensor_host(t, V, K, seed=21)
    rng = np.random.default_rng(4)
    ids = rng.integers(0, V, 40).astype(np.uint32)
    ids[5] = V - 1
    Wd = torch.from_numpy(W).to(dev)
    idd = torch.from_numpy(ids.view(np.int32)).to(dev)
    for idx, per_req, rows in ((0, 1, 40), (5, 0, 3), (2, 7, 6), (39, 1, 1)):
        got = qk.embed(t, Wd, V, K, idd, rows, idx=idx, per_req=per_req).cpu().numpy()
        want = orc.embed(t, W, V, K, ids, idx, per_req, rows)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (idx, per_req, rows)


def test_embed_out_of_vocabulary_id_reads_the_last_row(qk, orc, dev):
    import torch
    V, K = 10, 256
    W = qk.synth.tensor_host(qk.Q6_K, V, K, seed=2)
    ids = torch.tensor([3, 1000000, -1], dtype=torch.int32, device=dev)
    got = qk.embed(qk.Q6_K, torch.from_numpy(W).to(dev), V, K, ids, 3).cpu().numpy()
    want = orc.embed(qk.Q6_K, W, V, K, np.array([3, V - 1, V - 1], dtype=np.uint32), 0, 1, 3)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_glue_argument_errors(qk, dev):
    import torch
    x = torch.zeros((2, 64), device=dev)
    w = torch.zeros(64, device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.rmsnorm(x, w, eps=-1.0)
    assert e.value.code == -1
    ids = torch.zeros(4, dtype=torch.int32, device=dev)
    W = torch.zeros(34 * 2 * 8, dtype=torch.uint8, device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.embed(qk.Q8_0, W, 8, 64, ids, 3, idx=2, per_req=1)      # ids[2 + 2] is one past the end
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:
        qk.embed(qk.F16, W, 8, 64, ids, 1)
    assert e.value.code == -3
