"""ctypes binding of the engine-level C ABI (include/qk.h) and the recipe for a synthetic model file
the engine can open: a token embedding, MoE-only layers and a Q6_K head, under the reference's
tensor names (reference src/main.cpp:3602-3604, 1270-1277, 2726)."""
import ctypes as C

import numpy as np

from . import capi, gguf, synth


class Config(C.Structure):
    """reference include/qk.h:20-24"""
    _fields_ = [("n_slots", C.c_uint32), ("n_ctx", C.c_uint32), ("chunk", C.c_uint32)]


def _lib():
    L = capi.lib()
    if not getattr(L, "_qk_engine_bound", False):   # per library object: the tests also load a host-side build
        vp, u32 = C.c_void_p, C.c_uint32
        L.qk_open.restype = vp
        L.qk_open.argtypes = [C.c_char_p, C.POINTER(Config), C.c_char_p, C.c_size_t]
        L.qk_close.restype = None
        L.qk_close.argtypes = [vp]
        for name in ("qk_n_vocab", "qk_n_ctx", "qk_n_slots", "qk_chunk", "qk_eos_token", "qk_bos_token",
                     "qk_layer_first", "qk_layer_end", "qk_n_layer", "qk_n_embd", "qk_state_n"):
            getattr(L, name).restype = u32
            getattr(L, name).argtypes = [vp]
        L.qk_slot_start.argtypes = [vp, u32, vp, u32, u32, u32]
        L.qk_slot_cancel.restype = None
        L.qk_slot_cancel.argtypes = [vp, u32]
        L.qk_step_chunk.argtypes = [vp, vp, vp, vp]
        L.qk_stage_run.argtypes = [vp, u32, vp, vp, u32, u32, vp, vp]
        L.qk_stage_topk.argtypes = [vp, u32, vp, vp]
        L.qk_state_save.argtypes = [vp, u32, u32, u32]
        L.qk_state_load.argtypes = [vp, u32, u32, u32]
        L._qk_engine_bound = True
    return L


class Engine:
    """One qk_engine.  Methods return what the C functions return (negative codes included); only
    qk_open failing raises, with the message the library wrote."""

    def __init__(self, path, n_slots=1, n_ctx=4096, chunk=8):
        L = _lib()
        err = C.create_string_buffer(512)
        cfg = Config(n_slots, n_ctx, chunk)
        self._h = L.qk_open(str(path).encode(), C.byref(cfg), err, len(err))
        if not self._h:
            raise capi.QkError(-1, err.value.decode())
        self.n_slots, self.n_ctx, self.chunk = L.qk_n_slots(self._h), L.qk_n_ctx(self._h), L.qk_chunk(self._h)
        self.vocab, self.eos, self.bos = L.qk_n_vocab(self._h), L.qk_eos_token(self._h), L.qk_bos_token(self._h)
        self.n_layer, self.n_embd = L.qk_n_layer(self._h), L.qk_n_embd(self._h)
        self._tok = (C.c_uint32 * (self.n_slots * self.chunk))()
        self._cnt = (C.c_uint32 * self.n_slots)()
        self._fin = C.c_uint32(0)

    def close(self):
        if self._h:
            _lib().qk_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def slot_start(self, slot, prompt, max_gen, snap_prefix=0):
        arr = (C.c_uint32 * max(1, len(prompt)))(*prompt)
        return _lib().qk_slot_start(self._h, slot, arr if len(prompt) else None, len(prompt), max_gen, snap_prefix)

    def slot_cancel(self, slot):
        _lib().qk_slot_cancel(self._h, slot)

    def step_chunk(self):
        """-> (return code, {slot: [tokens]}, finished mask)"""
        rc = _lib().qk_step_chunk(self._h, self._tok, self._cnt, C.byref(self._fin))
        out = {}
        if rc >= 0:
            for s in range(self.n_slots):
                out[s] = [self._tok[s * self.chunk + i] for i in range(self._cnt[s])]
        return rc, out, self._fin.value

    def stage_run(self, slot, toks, base=0):
        """-> (return code, greedy ids)"""
        n = len(toks)
        arr = (C.c_uint32 * max(1, n))(*toks)
        ids = (C.c_uint32 * max(1, n))()
        rc = _lib().qk_stage_run(self._h, slot, arr, None, n, base, None, ids)
        return rc, list(ids[:n])

    def stage_topk(self, k):
        ids = (C.c_uint32 * max(1, k))()
        vals = (C.c_float * max(1, k))()
        rc = _lib().qk_stage_topk(self._h, k, ids, vals)
        return rc, list(ids[:k]), list(vals[:k])

    def state_n(self):
        return _lib().qk_state_n(self._h)

    def state_save(self, slot, idx, n_tok=0):
        return _lib().qk_state_save(self._h, slot, idx, n_tok)

    def state_load(self, slot, idx, n_tok=0):
        return _lib().qk_state_load(self._h, slot, idx, n_tok)


class StackModel:
    """Synthetic MoE-only model on the host: the tensors of a file qk_open accepts."""

    def __init__(self, seed, n_layer=2, vocab=1024, n_expert=32, n_ff=512, n_used=8, down_types=None,
                 embd_type=capi.Q6_K, embd_scale=0.3, eos=7, bos=11, arch="qwen35moe"):
        # embedding rows of rms ~300 next to MoE outputs of rms ~300 (block scales |N(0,1)|*1e-3):
        # both the residual and every layer move the logits
        H = 2048
        rng = np.random.default_rng(seed)
        self.arch, self.vocab, self.eos, self.bos, self.n_used = arch, vocab, eos, bos, n_used
        self.embd_type = embd_type
        self.embd = synth.tensor_host(embd_type, vocab, H, seed + 101, embd_scale)
        self.head = synth.tensor_host(capi.Q6_K, vocab, H, seed + 102)
        self.out_norm = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
        down_types = down_types or [capi.IQ4_XS] * n_layer
        self.layers = [synth.HostLayer(seed + 1000 * (l + 1), H, n_ff, n_expert, n_used, down_types[l])
                       for l in range(n_layer)]
        self.post_norm = [(1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32) for _ in range(n_layer)]

    @staticmethod
    def interleave_ba(alpha, beta):
        """[hV, H] alpha and beta -> the fused [2 hV, H] rows: per key-head group g the rows 4g, 4g+1 are
        beta of the value heads 2g, 2g+1 and 4g+2, 4g+3 their alpha."""
        hv = alpha.shape[0]
        ba = np.empty((2 * hv,) + alpha.shape[1:], dtype=alpha.dtype)
        for r in range(2 * hv):
            grp, sub = r >> 2, r & 3
            ba[r] = (beta if sub < 2 else alpha)[grp * 2 + (sub & 1)]
        return ba

    @staticmethod
    def split_ba(rows):
        """The inverse of interleave_ba: fused rows -> (alpha, beta)."""
        hv = rows.shape[0] // 2
        alpha, beta = np.empty((hv,) + rows.shape[1:], rows.dtype), np.empty((hv,) + rows.shape[1:], rows.dtype)
        for r in range(2 * hv):
            grp, sub = r >> 2, r & 3
            (beta if sub < 2 else alpha)[grp * 2 + (sub & 1)] = rows[r]
        return alpha, beta

    def kvs(self):
        return {"general.architecture": self.arch, self.arch + ".block_count": len(self.layers),
                self.arch + ".expert_used_count": self.n_used, "tokenizer.ggml.eos_token_id": self.eos,
                "tokenizer.ggml.bos_token_id": self.bos}

    def tensors(self):
        H = 2048
        t = [("token_embd.weight", self.embd_type, (H, self.vocab), self.embd),
             ("output_norm.weight", capi.F32, (H,), self.out_norm),
             ("output.weight", capi.Q6_K, (H, self.vocab), self.head)]
        for l, hl in enumerate(self.layers):
            t += gguf.layer_tensors(hl, l)
            t.append((f"blk.{l}.post_attention_norm.weight", capi.F32, (H,), self.post_norm[l]))
        return t

    def write(self, path):
        gguf.write(path, self.kvs(), self.tensors())
        return path


class FullModel:
    """Synthetic whole model on the host: every layer a mixer (gated DeltaNet "R" or full attention
    "A", the reference's fixed head shapes) followed by a MoE block; the tensors of a file qk_open
    accepts, under the reference's names (reference src/main.cpp:3916-4010)."""

    DN = dict(ch=8192, d_in=4096, hv=32, ds=128, hk=16)
    FA = dict(dh=256, hq=16, hkv=2, n_rot=64)

    def __init__(self, seed, kinds="RRRA", vocab=512, n_expert=8, n_ff=256, n_used=4, eos=1000, bos=11, arch="qwen35moe",
                 distinct_moe=None, fused_ba=None):
        """fused_ba: None writes ssm_alpha / ssm_beta as two F32 tensors; capi.F32 writes the same numbers
        as one interleaved ssm_ba tensor (the qwen3next form, reference src/main.cpp:3931-3948); capi.Q8_0 /
        capi.IQ4_XS write a quantised ssm_ba of its own -- alpha and beta of such a model are the
        dequantised rows, which whoever needs them on the host computes (mix[l]["alpha"] is None)."""
        H = 2048
        self.fused_ba = fused_ba
        rng = np.random.default_rng(seed)
        f = lambda *shape, scale=1.0: (rng.standard_normal(shape) * scale).astype(np.float32)
        near1 = lambda n: (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)
        q8 = lambda rows, k, s, sc: synth.tensor_host(capi.Q8_0, rows, k, s, sc)
        self.arch, self.vocab, self.eos, self.bos, self.n_used, self.kinds = arch, vocab, eos, bos, n_used, kinds
        self.embd_type = capi.Q6_K
        self.embd = synth.tensor_host(capi.Q6_K, vocab, H, seed + 101, 1e-3)      # rows of rms ~1
        self.head = synth.tensor_host(capi.Q6_K, vocab, H, seed + 102)
        self.out_norm = near1(H)
        self.layers, self.post_norm, self.attn_norm, self.mix = [], [], [], []
        for l, kind in enumerate(kinds):
            s0 = seed + 1000 * (l + 1)
            # block scales chosen so that residual, mixer output and MoE output are all of order one
            if distinct_moe and l >= distinct_moe:   # large files: reuse the first layers' MoE weights (own copy in the file)
                self.layers.append(self.layers[l % distinct_moe])
            else:
                self.layers.append(synth.HostLayer(s0, H, n_ff, n_expert, n_used, capi.IQ4_XS if l % 2 == 0 else capi.Q6_K,
                                                   d_scale=1.5e-4))
            self.post_norm.append(near1(H))
            self.attn_norm.append(near1(H))
            if kind == "R":
                d = self.DN
                self.mix.append(dict(kind="R", qkv=q8(d["ch"], H, s0 + 11, 4e-4), gate=q8(d["d_in"], H, s0 + 12, 4e-4),
                                     out=q8(H, d["d_in"], s0 + 13, 3e-4), alpha=f(d["hv"], H, scale=0.03),
                                     beta=f(d["hv"], H, scale=0.03), dt=f(d["hv"]),
                                     a=(-np.abs(rng.standard_normal(d["hv"])) - 0.05).astype(np.float32),
                                     ker=f(d["ch"], 4, scale=0.5), norm=near1(d["ds"])))
                m = self.mix[-1]
                if fused_ba == capi.F32:
                    m["ba"] = self.interleave_ba(m["alpha"], m["beta"])
                elif fused_ba is not None:
                    m["ba"] = synth.tensor_host(fused_ba, 2 * d["hv"], H, s0 + 14, 4e-4 if fused_ba == capi.Q8_0 else 2.4e-5)   # rows of std ~0.03, like the split tensors
                    m["alpha"] = m["beta"] = None
            elif kind == "A":
                a = self.FA
                self.mix.append(dict(kind="A", q=q8(a["hq"] * 2 * a["dh"], H, s0 + 21, 4e-4), k=q8(a["hkv"] * a["dh"], H, s0 + 22, 4e-4),
                                     v=q8(a["hkv"] * a["dh"], H, s0 + 23, 4e-4), out=q8(H, a["hq"] * a["dh"], s0 + 24, 3e-4),
                                     qn=near1(a["dh"]), kn=near1(a["dh"])))
            else:
                raise ValueError(kind)

    @staticmethod
    def interleave_ba(alpha, beta):
        """[hV, H] alpha and beta -> the fused [2 hV, H] rows: per key-head group g the rows 4g, 4g+1 are
        beta of the value heads 2g, 2g+1 and 4g+2, 4g+3 their alpha."""
        hv = alpha.shape[0]
        ba = np.empty((2 * hv,) + alpha.shape[1:], dtype=alpha.dtype)
        for r in range(2 * hv):
            grp, sub = r >> 2, r & 3
            ba[r] = (beta if sub < 2 else alpha)[grp * 2 + (sub & 1)]
        return ba

    @staticmethod
    def split_ba(rows):
        """The inverse of interleave_ba: fused rows -> (alpha, beta)."""
        hv = rows.shape[0] // 2
        alpha, beta = np.empty((hv,) + rows.shape[1:], rows.dtype), np.empty((hv,) + rows.shape[1:], rows.dtype)
        for r in range(2 * hv):
            grp, sub = r >> 2, r & 3
            (beta if sub < 2 else alpha)[grp * 2 + (sub & 1)] = rows[r]
        return alpha, beta

    def kvs(self):
        return {"general.architecture": self.arch, self.arch + ".block_count": len(self.layers),
                self.arch + ".expert_used_count": self.n_used, "tokenizer.ggml.eos_token_id": self.eos,
                "tokenizer.ggml.bos_token_id": self.bos}

    def tensors(self):
        H, d, a = 2048, self.DN, self.FA
        t = [("token_embd.weight", self.embd_type, (H, self.vocab), self.embd),
             ("output_norm.weight", capi.F32, (H,), self.out_norm),
             ("output.weight", capi.Q6_K, (H, self.vocab), self.head)]
        for l, hl in enumerate(self.layers):
            p, m = f"blk.{l}.", self.mix[l]
            t += gguf.layer_tensors(hl, l)
            t += [(p + "post_attention_norm.weight", capi.F32, (H,), self.post_norm[l]),
                  (p + "attn_norm.weight", capi.F32, (H,), self.attn_norm[l])]
            if m["kind"] == "R":
                t += [(p + "attn_qkv.weight", capi.Q8_0, (H, d["ch"]), m["qkv"]), (p + "attn_gate.weight", capi.Q8_0, (H, d["d_in"]), m["gate"]),
                      (p + "ssm_out.weight", capi.Q8_0, (d["d_in"], H), m["out"]), (p + "ssm_dt.bias", capi.F32, (d["hv"],), m["dt"]),
                      (p + "ssm_a", capi.F32, (d["hv"],), m["a"]), (p + "ssm_conv1d.weight", capi.F32, (4, d["ch"]), m["ker"]),
                      (p + "ssm_norm.weight", capi.F32, (d["ds"],), m["norm"])]
                if "ba" in m:
                    t += [(p + "ssm_ba.weight", self.fused_ba, (H, 2 * d["hv"]), m["ba"])]
                else:
                    t += [(p + "ssm_alpha.weight", capi.F32, (H, d["hv"]), m["alpha"]),
                          (p + "ssm_beta.weight", capi.F32, (H, d["hv"]), m["beta"])]
            else:
                t += [(p + "attn_q.weight", capi.Q8_0, (H, a["hq"] * 2 * a["dh"]), m["q"]), (p + "attn_k.weight", capi.Q8_0, (H, a["hkv"] * a["dh"]), m["k"]),
                      (p + "attn_v.weight", capi.Q8_0, (H, a["hkv"] * a["dh"]), m["v"]), (p + "attn_output.weight", capi.Q8_0, (a["hq"] * a["dh"], H), m["out"]),
                      (p + "attn_q_norm.weight", capi.F32, (a["dh"],), m["qn"]), (p + "attn_k_norm.weight", capi.F32, (a["dh"],), m["kn"])]
        return t

    def write(self, path):
        gguf.write(path, self.kvs(), self.tensors())
        return path
