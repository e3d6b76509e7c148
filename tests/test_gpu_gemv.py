"""Quantised GEMVs through the C ABI against the oracle (dequantise row, dot in double).
Bar: max|got-ref| / max|ref| <= 1e-3 (accumulation order differs); the reference's own
scale-aware metric (<= 1e-2) is checked as well."""
import numpy as np
import pytest

# every test runs on both forms of the one-row kernels (conftest.one_row_form)
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("one_row_form")]

TYPES = {"q8_0": 8, "q6_k": 14, "iq4_xs": 23, "iq3_xxs": 18, "f16": 1, "f32": 0}
TOL = 1e-3


def run_case(qk, orc, dev, name, M, K, batch, seed=42):
    import torch
    print(f"[case] gemv {name} M={M} K={K} batch={batch} seed={seed}", flush=True)
    t = TYPES[name]
    W = qk.synth.tensor_host(t, M, K, seed)
    x = np.random.default_rng(seed + 1).standard_normal((batch, K)).astype(np.float32)
    got = qk.gemv(t, torch.from_numpy(W).to(dev), torch.from_numpy(x).to(dev), M, K).cpu().numpy()
    want = orc.gemv(t, W, x, M, K)
    assert got.shape == want.shape
    assert orc.rel_maxabs_err(got, want) <= TOL
    assert orc.max_rel_err(got, want) <= 1e-2
    return got


@pytest.mark.parametrize("name", ["q8_0", "q6_k", "iq4_xs", "iq3_xxs"])
@pytest.mark.parametrize("M,K,batch", [(8192, 2048, 1), (1000, 2048, 3), (515, 4096, 2), (2048, 512, 1),
                                       (333, 512, 2), (64, 8192, 1), (37, 1024, 1), (50, 256, 1),
                                       (21, 768, 2), (9, 2304, 1), (1, 2048, 1)])
def test_gemv_quantised(qk, orc, dev, name, M, K, batch):
    run_case(qk, orc, dev, name, M, K, batch)


@pytest.mark.parametrize("name", ["q8_0", "q6_k", "iq4_xs", "iq3_xxs"])
@pytest.mark.parametrize("M,K,batch", [(8192, 2048, 16), (1000, 2048, 5), (130, 1024, 16), (96, 512, 4),
                                       (77, 512, 3), (48, 256, 32), (2048, 2048, 40), (33, 2048, 17),
                                       (2048, 4096, 16), (100, 4096, 5), (33, 4096, 40)])
def test_gemv_quantised_several_rows(qk, orc, dev, name, M, K, batch):
    """batch >= 3 takes the matrix-core path where the shape allows (K = 256..2048, or 4096 in two
    passes over the rows' halves, and the tensor ending on a 16-byte boundary), one pass per row
    otherwise: same bar either way."""
    run_case(qk, orc, dev, name, M, K, batch, seed=77)


@pytest.mark.parametrize("M,K", [(8192, 2048), (4096, 2048), (2048, 4096), (512, 2048), (12288, 2048), (9216, 2048)])
@pytest.mark.parametrize("batch", [1, 16])
def test_gemv_q8_0_engine_shapes(qk, orc, dev, M, K, batch):
    """The dense projections of a decode step at the shapes the reference dispatches them
    (src/main.cpp:4310-4335, 4195-4196), for one slot and for sixteen; 12288 and 9216 rows are a
    layer's input projections back to back, as the engine runs them for one slot."""
    run_case(qk, orc, dev, "q8_0", M, K, batch, seed=5)


@pytest.mark.parametrize("name", ["q8_0", "q6_k", "iq4_xs", "iq3_xxs"])
@pytest.mark.parametrize("M,batch", [(12288, 1), (9216, 1), (515, 2), (3, 1)])
def test_gemv_with_the_norm_in_front(qk, orc, dev, unrun_form, name, M, batch):
    """qkk_gemv_norm: y = W . rmsnorm(x) * w with the norm inside the launch, against the oracle's norm
    (double) followed by its GEMV; 12288 and 9216 rows are a layer's input projections back to back."""
    import torch
    print(f"[case] gemv with norm {name} M={M} batch={batch}", flush=True)
    K, t = 2048, TYPES[name]
    W = qk.synth.tensor_host(t, M, K, 31)
    rng = np.random.default_rng(M)
    x = (rng.standard_normal((batch, K)) * 3.0).astype(np.float32)
    w = rng.uniform(0.5, 1.5, K).astype(np.float32)
    up = lambda a: torch.from_numpy(a).to(dev)
    got = qk.gemv_norm(t, up(W), up(x), up(w), M, K, eps=1e-6).cpu().numpy()
    xn = np.stack([orc.add_rms(x[b], w, 1e-6) for b in range(batch)])
    want = orc.gemv(t, W, xn, M, K)
    assert orc.rel_maxabs_err(got, want) <= TOL
    # the same numbers as the norm launch followed by the plain product, to rounding
    two = qk.gemv(t, up(W), qk.rmsnorm(up(x), up(w)), M, K).cpu().numpy()
    assert orc.rel_maxabs_err(got, two) <= 1e-5
    with pytest.raises(qk.QkError):
        qk.gemv_norm(t, up(W), up(x[:, :1024].copy()), up(w[:1024].copy()), M, 1024)


def test_gemv_two_pass_k_is_deterministic(qk, orc, dev):
    """K = 4096 for several rows adds the second half's sum to the first's in a fixed order."""
    a = run_case(qk, orc, dev, "q6_k", 784, 4096, 9, seed=12)
    b = run_case(qk, orc, dev, "q6_k", 784, 4096, 9, seed=12)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("M,K", [(64, 32), (33, 96), (10, 2080)])
def test_gemv_q8_0_short_rows(qk, orc, dev, M, K):
    run_case(qk, orc, dev, "q8_0", M, K, 1)


@pytest.mark.parametrize("name", ["f16", "f32"])
@pytest.mark.parametrize("M,K,batch", [(4096, 4096, 1), (257, 2048, 2), (256, 2048, 16), (5, 72, 1)])
def test_gemv_dense(qk, orc, dev, name, M, K, batch):
    run_case(qk, orc, dev, name, M, K, batch)


@pytest.mark.parametrize("name", ["q8_0", "q6_k", "iq4_xs", "iq3_xxs", "f16", "f32"])
@pytest.mark.parametrize("batch", [1, 16])
def test_gemv_full_size_scaling_and_linearity(qk, orc, dev, name, batch):
    """Size-independent properties at the benchmark's shape (8192 x 2048): doubling x doubles every sum
    -- exactly on the fp32 paths (a power of two changes no rounding; the formats that split x into two
    halves, and the several-row matrix-core path, round the low half differently: 1e-6 there) -- and
    W.(x1 + x2) = W.x1 + W.x2 to fp32 rounding."""
    import torch
    print(f"[case] gemv properties {name} batch={batch}", flush=True)
    M, K, t = 8192, 2048, TYPES[name]
    W = torch.from_numpy(qk.synth.tensor_host(t, M, K, 7)).to(dev)
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    x1, x2 = torch.randn((batch, K), device=dev, generator=g), torch.randn((batch, K), device=dev, generator=g)
    y1, y2 = qk.gemv(t, W, x1, M, K), qk.gemv(t, W, x2, M, K)
    y1d, y12 = qk.gemv(t, W, (2 * x1).contiguous(), M, K), qk.gemv(t, W, (x1 + x2).contiguous(), M, K)
    torch.cuda.synchronize()
    scale = float(y1.abs().max())
    exact = batch == 1 and name in ("q8_0", "q6_k", "f16", "f32")
    if exact:
        assert torch.equal(y1d, 2 * y1)
    else:
        assert float((y1d - 2 * y1).abs().max()) <= 1e-6 * scale
    assert float((y12 - (y1 + y2)).abs().max()) <= 2e-5 * scale


def test_gemv_is_deterministic(qk, orc, dev):
    a = run_case(qk, orc, dev, "iq3_xxs", 4096, 2048, 1, seed=9)
    b = run_case(qk, orc, dev, "iq3_xxs", 4096, 2048, 1, seed=9)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_gemv_zero_scales_give_zero(qk, dev):
    import torch
    W = qk.synth.tensor_host(qk.Q6_K, 64, 2048, 3).reshape(-1, 210).copy()
    W[:, 208:210] = 0
    x = torch.randn(2048, device=dev)
    y = qk.gemv(qk.Q6_K, torch.from_numpy(W.reshape(-1)).to(dev), x, 64, 2048)
    assert torch.all(y == 0)


def test_gemv_argument_errors(qk, dev):
    import torch
    W = torch.zeros(34 * 64, dtype=torch.uint8, device=dev)
    x = torch.zeros(2048, device=dev)
    with pytest.raises(qk.QkError) as e:
        qk.gemv(qk.Q6_K, W, x, 1, 100)
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:
        qk.gemv(77, W, x, 1, 2048)
    assert e.value.code == -3
    with pytest.raises(qk.QkError) as e:
        qk.gemv(qk.Q8_0, W[2:], x, 1, 32)   # misaligned tensor base
    assert e.value.code == -1
