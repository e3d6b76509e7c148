"""GPU dequantisation must be bit-identical to the reference's CPU dequantisation."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "dequant_golden.npz"))
FORMATS = [("q8_0", 8, 32), ("q6_k", 14, 256), ("iq4_xs", 23, 256), ("iq3_xxs", 18, 256)]


@pytest.mark.parametrize("name,t,be", FORMATS)
def test_dequant_matches_golden_bitwise(qk, dev, name, t, be):
    import torch
    print(f"[case] dequant golden {name}", flush=True)
    blocks, want = G[f"{name}_blocks"], G[f"{name}_values"]
    out = qk.dequant(t, torch.from_numpy(blocks.reshape(-1).copy()).to(dev), blocks.shape[0] * be)
    got = out.cpu().numpy().view(np.uint32).reshape(want.shape)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("name,t,be", FORMATS)
def test_dequant_matches_oracle_bitwise_random(qk, orc, dev, name, t, be):
    import torch
    print(f"[case] dequant random {name}", flush=True)
    nb = 20000
    blocks = qk.synth.blocks_host(t, nb, seed=314)
    want = orc.dequant(t, blocks, nb * be)
    got = qk.dequant(t, torch.from_numpy(blocks.reshape(-1)).to(dev), nb * be).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # arbitrary bytes with finite scales
    rng = np.random.default_rng(5)
    raw = rng.integers(0, 256, size=blocks.shape, dtype=np.uint8)
    raw[:, qk.synth.D_OFFSET[t] + 1] &= 0xFB
    want = orc.dequant(t, raw, nb * be)
    got = qk.dequant(t, torch.from_numpy(raw.reshape(-1)).to(dev), nb * be).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_f16_all_halves(qk, orc, dev):
    import torch
    h = np.arange(65536, dtype=np.uint16)
    got = qk.dequant(qk.F16, torch.from_numpy(h.view(np.uint8).copy()).to(dev), 65536).cpu().numpy()
    want = orc.dequant(orc.F16, h.view(np.uint8), 65536)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_rejects_partial_block(qk, dev):
    import torch
    w = torch.zeros(210, dtype=torch.uint8, device=dev)
    with pytest.raises(qk.QkError):
        qk.dequant(qk.Q6_K, w, 100)
