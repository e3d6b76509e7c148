"""Seeded synthetic GGUF block streams and MoE layers.

The reference's self-checking modes build their inputs from mt19937 seeds 42/43 and
per-format field ranges (reference src/main.cpp:619-625, 665-670, 693-699, 722-728,
751-755); those are recipes, not vectors (libstdc++'s normal_distribution is not
portable), so this module follows the same recipes with numpy's PCG64 (host) or torch's
generator (device): every bit pattern of the quantised fields is valid, super-block scales
are |N(0,1)|*1e-3 rounded to half the way the reference rounds (values below 2^-14 flush
to zero, reference src/quants.h:42).
"""
import numpy as np

from .capi import BLOCK, F16, F32, IQ3_XXS, IQ4_XS, Q6_K, Q8_0

# byte offset of the f16 super-block scale inside a block
D_OFFSET = {Q8_0: 0, Q6_K: 208, IQ4_XS: 0, IQ3_XXS: 0}


def f32_to_f16_bits(v):
    """float32 array -> uint16 half bits, round-to-nearest-even, with the reference's
    flush of everything below 2^-14 to signed zero and overflow to infinity."""
    v = np.asarray(v, dtype=np.float32)
    with np.errstate(over="ignore"):
        h = v.astype(np.float16).view(np.uint16)
    small = np.abs(v) < np.float32(2.0 ** -14)
    sign = (v.view(np.uint32) >> 16).astype(np.uint16) & np.uint16(0x8000)
    h = np.where(small, sign, h)
    nan = np.isnan(v)
    h = np.where(nan, sign | np.uint16(0x7C00), h)
    return h.astype(np.uint16)


def blocks_host(type_, n_blocks, seed, d_scale=1e-3):
    """uint8 array [n_blocks, block_bytes] of random valid blocks."""
    rng = np.random.default_rng(seed)
    _, nbytes = BLOCK[type_]
    raw = rng.integers(0, 256, size=(n_blocks, nbytes), dtype=np.uint8)
    if type_ == Q8_0:
        raw[:, 2:] = rng.integers(-127, 128, size=(n_blocks, 32), dtype=np.int8).view(np.uint8)
    elif type_ == Q6_K:
        raw[:, 192:208] = rng.integers(-127, 128, size=(n_blocks, 16), dtype=np.int8).view(np.uint8)
    d = f32_to_f16_bits(np.abs(rng.standard_normal(n_blocks).astype(np.float32)) * np.float32(d_scale))
    off = D_OFFSET[type_]
    raw[:, off] = (d & 0xFF).astype(np.uint8)
    raw[:, off + 1] = (d >> 8).astype(np.uint8)
    return raw


def tensor_host(type_, rows, k, seed, d_scale=1e-3):
    """Row-major weight tensor [rows] x K as a flat uint8 array of GGUF blocks (or f16/f32)."""
    rng = np.random.default_rng(seed)
    if type_ == F32:
        return (rng.standard_normal((rows, k)).astype(np.float32)).view(np.uint8).reshape(-1)
    if type_ == F16:
        w = (rng.standard_normal((rows, k)).astype(np.float32) * np.float32(0.05))
        return f32_to_f16_bits(w).view(np.uint8).reshape(-1)
    be, _ = BLOCK[type_]
    assert k % be == 0
    return blocks_host(type_, rows * (k // be), seed, d_scale).reshape(-1)


def blocks_device(type_, n_blocks, seed, device="cuda", d_scale=1e-3):
    """Same recipe generated on the device with torch (for benchmark-sized tensors)."""
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    _, nbytes = BLOCK[type_]
    raw = torch.randint(0, 256, (n_blocks, nbytes), dtype=torch.uint8, device=device, generator=g)
    if type_ == Q8_0:
        q = torch.randint(-127, 128, (n_blocks, 32), dtype=torch.int8, device=device, generator=g)
        raw[:, 2:] = q.view(torch.uint8)
    elif type_ == Q6_K:
        q = torch.randint(-127, 128, (n_blocks, 16), dtype=torch.int8, device=device, generator=g)
        raw[:, 192:208] = q.view(torch.uint8)
    v = torch.randn(n_blocks, device=device, generator=g).abs() * d_scale
    h = v.to(torch.float16)
    h = torch.where(v < 2.0 ** -14, torch.zeros_like(h), h)
    hb = h.view(torch.int16).to(torch.int32) & 0xFFFF
    off = D_OFFSET[type_]
    raw[:, off] = (hb & 0xFF).to(torch.uint8)
    raw[:, off + 1] = (hb >> 8).to(torch.uint8)
    return raw


class HostLayer:
    """One synthetic MoE layer on the host (numpy), the reference model's shapes by default
    (2048 wide, 256 experts of 512, 8 used)."""

    def __init__(self, seed, n_embd=2048, n_ff=512, n_expert=256, n_used=8, down_type=IQ4_XS, gu_type=IQ3_XXS,
                 d_scale=1e-3):
        rng = np.random.default_rng(seed)
        H, F, E = n_embd, n_ff, n_expert
        self.n_embd, self.n_ff, self.n_expert, self.n_used = H, F, E, n_used
        self.gu_type, self.down_type = gu_type, down_type
        # router rows scaled so logits are O(1)
        self.gate_inp = (rng.standard_normal((E, H)).astype(np.float32) * np.float32(2.0 / np.sqrt(H)))
        self.gate_inp_shexp = (rng.standard_normal(H).astype(np.float32) * np.float32(1.0 / np.sqrt(H)))
        self.gate_exps = tensor_host(gu_type, E * F, H, seed + 1, d_scale)
        self.up_exps = tensor_host(gu_type, E * F, H, seed + 2, d_scale)
        self.down_exps = tensor_host(down_type, E * H, F, seed + 3, d_scale)
        self.gate_shexp = tensor_host(Q8_0, F, H, seed + 4, d_scale)
        self.up_shexp = tensor_host(Q8_0, F, H, seed + 5, d_scale)
        self.down_shexp = tensor_host(Q8_0, H, F, seed + 6, d_scale)

    NAMES = ("gate_inp", "gate_inp_shexp", "gate_exps", "up_exps", "down_exps", "gate_shexp", "up_shexp",
             "down_shexp")

    def to_device(self, device="cuda"):
        import torch
        from .capi import MoeLayer
        t = {n: torch.from_numpy(np.ascontiguousarray(getattr(self, n))).to(device) for n in self.NAMES}
        return MoeLayer(self.n_embd, self.n_ff, self.n_expert, self.n_used, self.down_type, gu_type=self.gu_type,
                        **t)


def device_layer(seed, n_embd=2048, n_ff=512, n_expert=256, n_used=8, down_type=IQ4_XS, device="cuda",
                 d_scale=1e-3, slab=None):
    """Synthetic MoE layer generated directly in device memory.  slab: a Slab the tensors are carved from
    (every layer of a ring in ONE device allocation) instead of an allocation per tensor."""
    import torch
    from .capi import MoeLayer
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    H, F, E = n_embd, n_ff, n_expert
    keep = (lambda x: slab.take(x)) if slab is not None else (lambda x: x)
    gi = keep(torch.randn((E, H), device=device, generator=g) * (2.0 / H ** 0.5))
    gis = keep(torch.randn(H, device=device, generator=g) * (1.0 / H ** 0.5))

    def t(type_, rows, k, s):
        return keep(blocks_device(type_, rows * (k // BLOCK[type_][0]), s, device, d_scale).reshape(-1))

    return MoeLayer(H, F, E, n_used, down_type, gi, gis, t(IQ3_XXS, E * F, H, seed + 1),
                    t(IQ3_XXS, E * F, H, seed + 2), t(down_type, E * H, F, seed + 3), t(Q8_0, F, H, seed + 4),
                    t(Q8_0, F, H, seed + 5), t(Q8_0, H, F, seed + 6))


def layer_bytes(n_embd=2048, n_ff=512, n_expert=256, down_type=IQ4_XS):
    """Bytes of one synthetic layer's tensors, each rounded up to 256."""
    from .capi import row_bytes
    H, F, E = n_embd, n_ff, n_expert
    sizes = [E * H * 4, H * 4, 2 * E * F * row_bytes(IQ3_XXS, H), E * H * row_bytes(down_type, F),
             2 * F * row_bytes(Q8_0, H), H * row_bytes(Q8_0, F)]
    return sum((b + 255) // 256 * 256 for b in sizes) + 4 * 256


class Slab:
    """One device allocation that tensors are copied into back to back (256-byte aligned): a ring of
    layers then lies in one mapping, as the tensors of a model file uploaded into one buffer would."""

    def __init__(self, nbytes, device="cuda"):
        import torch
        self.buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        self.at = 0

    def take(self, t):
        import torch
        raw = t.contiguous().view(torch.uint8).reshape(-1)
        n = raw.numel()
        if self.at + n > self.buf.numel():
            raise ValueError("Slab: full")
        view = self.buf[self.at:self.at + n]
        view.copy_(raw)
        self.at += (n + 255) // 256 * 256
        return view.view(t.dtype).reshape(t.shape)
