"""Writes tests/golden/dequant_golden.npz: block bytes and the fp32 bit patterns the
REFERENCE's own dequantisation header produces for them.

Run in the build container (needs oracle/_ref/libqkref.so, i.e. `make -C oracle` with the
reference tree mounted):  python tests/golden/make_golden.py
The reference ships no numeric vectors for this path; these fixtures are made from its
compiled header so that they travel to machines where the reference tree is absent.
Contents per format F in {q8_0, q6_k, iq4_xs, iq3_xxs}:
  F_blocks  uint8 [n, block_bytes]   seeded random valid blocks + hand-made corner blocks
  F_values  uint32 [n, block_elems]  bit patterns of dequant_row_F(blocks)
plus f16_bits/f16_values (half -> float of the reference for a spread of halves) and
f32_in/f32_to_f16 (float -> half of the reference, including the flush below 2^-14).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import __graft_entry__ as entry  # noqa: E402

qk = entry.load_package()
orc = entry.load_oracle()
ref = orc.ref()
assert ref is not None, "build oracle/_ref first (make -C oracle)"

out = {}
for name, t, be in [("q8_0", qk.Q8_0, 32), ("q6_k", qk.Q6_K, 256), ("iq4_xs", qk.IQ4_XS, 256),
                    ("iq3_xxs", qk.IQ3_XXS, 256)]:
    nbytes = qk.capi.BLOCK[t][1]
    rng = np.random.default_rng(1000 + t)
    blocks = [qk.synth.blocks_host(t, 24, seed=2000 + t)]
    raw = rng.integers(0, 256, size=(24, nbytes), dtype=np.uint8)  # arbitrary bytes, finite scales
    off = qk.synth.D_OFFSET[t]
    raw[:, off + 1] &= 0xFB
    blocks.append(raw)
    corner = np.zeros((4, nbytes), dtype=np.uint8)
    corner[1, :] = 0xFF
    corner[1, off:off + 2] = np.frombuffer(np.float16(-0.125).tobytes(), dtype=np.uint8)
    corner[2, :] = 0x55
    corner[2, off:off + 2] = np.frombuffer(np.float16(6.1e-5).tobytes(), dtype=np.uint8)  # subnormal-adjacent
    corner[3, :] = 0xAA
    corner[3, off:off + 2] = np.frombuffer(np.uint16(0x0001).tobytes(), dtype=np.uint8)  # smallest subnormal
    blocks.append(corner)
    blocks = np.concatenate(blocks)
    vals = orc.dequant(t, blocks, blocks.shape[0] * be, use_ref=True)
    out[f"{name}_blocks"] = blocks
    out[f"{name}_values"] = vals.view(np.uint32).reshape(blocks.shape[0], be)

h = np.concatenate([np.arange(0, 65536, 37, dtype=np.uint32), [0, 1, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0x8000, 0xFBFF]])
h = h.astype(np.uint16)
out["f16_bits"] = h
out["f16_values"] = np.array([np.float32(ref.qkref_f16_to_f32(int(v))).view(np.uint32) for v in h], dtype=np.uint32)
rng = np.random.default_rng(77)
f = np.concatenate([rng.standard_normal(400).astype(np.float32) * np.float32(1e-3),
                    (2.0 ** rng.uniform(-20, 17, 400)).astype(np.float32),
                    np.array([0, 2.0 ** -14, 6.0e-5, 6.1035e-5, 65504, 65520, 1e9, -1e-9], dtype=np.float32)])
out["f32_in"] = f
out["f32_to_f16"] = np.array([ref.qkref_f32_to_f16(float(v)) for v in f], dtype=np.uint16)

path = os.path.join(HERE, "dequant_golden.npz")
np.savez_compressed(path, **out)
print("wrote", path, os.path.getsize(path), "bytes")
