"""The oracle against the committed golden vectors (made from the reference's compiled
header by tests/golden/make_golden.py).  Runs where the reference tree is absent."""
import os

import numpy as np
import pytest

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "dequant_golden.npz"))
FORMATS = [("q8_0", 8, 32), ("q6_k", 14, 256), ("iq4_xs", 23, 256), ("iq3_xxs", 18, 256)]


@pytest.mark.parametrize("name,t,be", FORMATS)
def test_oracle_dequant_matches_golden(orc, name, t, be):
    blocks, want = G[f"{name}_blocks"], G[f"{name}_values"]
    got = orc.dequant(t, blocks, blocks.shape[0] * be).view(np.uint32).reshape(want.shape)
    assert np.array_equal(got, want)


def test_oracle_half_conversions_match_golden(orc):
    got = np.array([np.float32(orc.lib().qko_f16_to_f32(int(v))).view(np.uint32) for v in G["f16_bits"]],
                   dtype=np.uint32)
    assert np.array_equal(got, G["f16_values"])
    got = np.array([orc.lib().qko_f32_to_f16(float(v)) for v in G["f32_in"]], dtype=np.uint16)
    assert np.array_equal(got, G["f32_to_f16"])


def test_synth_scale_rounding_matches_golden(qk):
    assert np.array_equal(qk.synth.f32_to_f16_bits(G["f32_in"]), G["f32_to_f16"])
