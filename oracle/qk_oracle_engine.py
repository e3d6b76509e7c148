"""CPU restatement of the reference engine's slot state machine and of the MoE-only model step.
TEST INFRASTRUCTURE ONLY: imported by tests/; the product never imports it.

  SlotMachine    qk_slot_start / qk_slot_cancel / qk_step_chunk as the reference runs them with
                 speculative decoding off and no cached prefix (reference src/main.cpp:5447-5532,
                 4462-4485, 4552-4646), over a model given as a function  (token, dispatch depth) -> next token.
  stack_next     that function for a model whose layers are MoE blocks only (the decode step of
                 reference src/main.cpp:4194-4419 with every mixer output zero), from the oracle's
                 embed / add_rms / moe_ref / gemv / argmax.
  Stub           binding of the reference's own stub engine (stub/qk_stub.c) built into
                 _ref/libqk_stub.so; tests pin SlotMachine against it where the two coincide.

Pinned by: the stub engine (same chunking, finished mask, max_gen ending and return values once
the stub's one extra silent prefill step is accounted for), and the closed form of a memoryless
model's stream (token j of a slot is f^(j+1)(last prompt token), emitted at the slot's step
serial_prefill_steps + j) in tests/test_engine_oracle.py."""
import ctypes as C
import os

import numpy as np

import qk_oracle_py as O

HERE = os.path.dirname(os.path.abspath(__file__))


class SlotMachine:
    """nxt: a function (token, dispatch depth) -> next token for a model without memory, or an object
    with reset(slot) and feed(slot, token, position, depth) -> next token for one with per-slot state
    (the positions [0, done) that qk_slot_start prefills are fed at the start, reference
    src/main.cpp:5470-5500; a step feeds prompt[cursor] at position cursor or the last sample at
    pos, :4563-4573)."""

    def __init__(self, nxt, vocab, eos, n_slots, n_ctx, chunk, max_b=128, no_batch=False):
        self.model = nxt if hasattr(nxt, "feed") else None
        self.nxt, self.vocab, self.eos = nxt, vocab, eos
        self.n_slots, self.n_ctx, self.chunk, self.max_b, self.no_batch = n_slots, n_ctx, chunk, max_b, no_batch
        self.slots = [dict(active=False) for _ in range(n_slots)]
        self.depths = []   # dispatch depth of every device step, for the tests

    # reference src/main.cpp:5447-5516
    def slot_start(self, slot, prompt, max_gen, snap_prefix=0):
        if slot >= self.n_slots:
            return -1
        if self.slots[slot]["active"]:
            return -2
        if prompt is None or len(prompt) < 1 or len(prompt) + max_gen > self.n_ctx:
            return -3
        if any(t >= self.vocab for t in prompt):
            return -4
        start, target, done = 0, len(prompt) - 1, 0

        def batch_to(limit):   # :5470-5477
            nonlocal done
            while limit > done and limit - done >= 16:
                done += min(self.max_b, limit - done)
        snap_at = snap_prefix if (start < snap_prefix < target) else 0   # :5487
        if not self.no_batch:
            if snap_at:
                batch_to(snap_at)
            batch_to(target)
        if self.model:
            self.model.reset(slot)
            for p in range(done):
                self.model.feed(slot, prompt[p], p, 1)
        self.slots[slot] = dict(active=True, prompt=list(prompt), cursor=done, pos=done, last=0, gen=0, max_gen=max_gen)
        return 0

    def slot_cancel(self, slot):   # :5519-5525
        if slot < self.n_slots:
            self.slots[slot]["active"] = False

    # reference src/main.cpp:4462-4467 and phase 3, :4552-4646
    def step_chunk(self):
        out = {s: [] for s in range(self.n_slots)}
        fin = 0
        active_at_entry = sum(1 for sl in self.slots if sl["active"])
        if not active_at_entry:
            return 0, out, 0
        for _ in range(self.chunk):
            n_act, max_z, need, fed, at = 0, 0, False, {}, {}
            for s, sl in enumerate(self.slots):
                if not sl["active"]:
                    continue
                n_act += 1
                max_z = s + 1
                if sl["cursor"] < len(sl["prompt"]):
                    fed[s], at[s] = sl["prompt"][sl["cursor"]], sl["cursor"]
                    need = True
                else:
                    fed[s], at[s] = sl["last"], sl["pos"]
                    if len(out[s]) < self.chunk:
                        need = True
            if not n_act or not need:
                break
            self.depths.append(max_z)
            for s, sl in enumerate(self.slots):
                if not sl["active"]:
                    continue
                sampled = self.model.feed(s, fed[s], at[s], max_z) if self.model else self.nxt(fed[s], max_z)
                prefilling = sl["cursor"] < len(sl["prompt"])
                if prefilling and sl["cursor"] + 1 < len(sl["prompt"]):
                    sl["cursor"] += 1
                    continue
                if prefilling:
                    sl["cursor"] = sl["pos"] = len(sl["prompt"])
                if sampled == self.eos:
                    if not prefilling:
                        sl["pos"] += 1
                    sl["active"] = False
                    fin |= 1 << s
                    continue
                out[s].append(sampled)
                sl["last"] = sampled
                sl["gen"] += 1
                if not prefilling:
                    sl["pos"] += 1
                if sl["pos"] >= self.n_ctx or sl["gen"] >= sl["max_gen"]:
                    sl["active"] = False
                    fin |= 1 << s
        return active_at_entry, out, fin


def stack_next(model, token, eps=1e-6, want_margin=False, threads=1):
    """Next greedy token of a MoE-only model (an object with embd, embd_type, vocab, layers,
    post_norm, out_norm, head, as qwen-kernel_amd's engine.StackModel) after `token`.  `threads`
    splits the row loops of the step over host threads (the same bits)."""
    H = 2048
    x = O.embed(model.embd_type, model.embd, model.vocab, H, np.array([token], dtype=np.uint32), 0, 1, 1)[0]
    for l, hl in enumerate(model.layers):
        xn = O.add_rms(x, model.post_norm[l], eps)
        y = O.moe_ref(hl, xn)["y"] if threads <= 1 else O.moe_ref_threads(hl, xn[None, :], threads)[0]
        x = (x + y).astype(np.float32)
    xn = O.add_rms(x, model.out_norm, eps)
    logits = O.gemv(O.Q6_K, model.head, xn, model.vocab, H, threads=threads)
    best = O.argmax(logits)
    if want_margin:
        srt = np.sort(logits.astype(np.float64))
        return best, float(srt[-1] - srt[-2]), float(np.abs(logits).max())
    return best


class _StubCfg(C.Structure):
    _fields_ = [("n_slots", C.c_uint32), ("n_ctx", C.c_uint32), ("chunk", C.c_uint32)]


class Stub:
    """The reference's stub engine; None-like (available() False) when _ref/libqk_stub.so is absent."""

    @staticmethod
    def available():
        return os.path.exists(os.path.join(HERE, "_ref", "libqk_stub.so"))

    def __init__(self, n_slots, n_ctx, chunk):
        L = C.CDLL(os.path.join(HERE, "_ref", "libqk_stub.so"))
        vp, u32 = C.c_void_p, C.c_uint32
        L.qk_open.restype = vp
        L.qk_open.argtypes = [C.c_char_p, C.POINTER(_StubCfg), C.c_char_p, C.c_size_t]
        L.qk_close.argtypes = [vp]
        L.qk_slot_start.argtypes = [vp, u32, vp, u32, u32, u32]
        L.qk_slot_cancel.argtypes = [vp, u32]
        L.qk_step_chunk.argtypes = [vp, vp, vp, vp]
        self.L, self.n_slots, self.chunk = L, n_slots, chunk
        err = C.create_string_buffer(128)
        self.h = L.qk_open(b"stub", C.byref(_StubCfg(n_slots, n_ctx, chunk)), err, 128)
        if not self.h:
            raise RuntimeError(err.value.decode())
        self._tok = (C.c_uint32 * (n_slots * chunk))()
        self._cnt = (C.c_uint32 * n_slots)()
        self._fin = C.c_uint32(0)

    def close(self):
        if self.h:
            self.L.qk_close(self.h)
            self.h = None

    def slot_start(self, slot, prompt, max_gen):
        arr = (C.c_uint32 * max(1, len(prompt)))(*prompt)
        return self.L.qk_slot_start(self.h, slot, arr, len(prompt), max_gen, 0)

    def slot_cancel(self, slot):
        self.L.qk_slot_cancel(self.h, slot)

    def step_chunk(self):
        rc = self.L.qk_step_chunk(self.h, self._tok, self._cnt, C.byref(self._fin))
        out = {s: [self._tok[s * self.chunk + i] for i in range(self._cnt[s])] for s in range(self.n_slots)}
        return rc, out, self._fin.value


class FullModelOracle:
    """The decode step of a whole model (mixer + MoE block per layer) with per-slot state, from the
    oracle's pieces, following the reference's recorded step (src/main.cpp:4194-4419): an object with
    the fields of qwen-kernel_amd's engine.FullModel.  feed() returns the greedy next token and
    records the top-2 logit gap and the largest logit of the step in .last_margin."""

    def __init__(self, model, n_slots, n_ctx, kdiv=0, eps=1e-6):
        import qk_oracle_attn as OA
        import qk_oracle_deltanet as OD
        self.OA, self.OD, self.m, self.n_ctx, self.kdiv, self.eps = OA, OD, model, n_ctx, kdiv, eps
        self.rope = OA.rope_table(n_ctx, model.FA["n_rot"])
        self.state = [None] * n_slots
        self.last_margin = None
        for s in range(n_slots):
            self.reset(s)

    def reset(self, slot):
        d, a = self.m.DN, self.m.FA
        st = []
        for mix in self.m.mix:
            if mix["kind"] == "R":
                st.append([np.zeros((d["ch"], 3), np.float32), np.zeros((d["hv"], d["ds"], d["ds"]), np.float32)])
            else:
                st.append([np.zeros((a["hkv"], self.n_ctx, a["dh"]), np.float32), np.zeros((a["hkv"], self.n_ctx, a["dh"]), np.float32)])
        self.state[slot] = st

    def feed(self, slot, token, pos, depth=1):
        m, d, a, eps, H = self.m, self.m.DN, self.m.FA, self.eps, 2048
        x = O.embed(m.embd_type, m.embd, m.vocab, H, np.array([token], dtype=np.uint32), 0, 1, 1)[0]
        for l, mix in enumerate(m.mix):
            st = self.state[slot][l]
            xn = O.add_rms(x, m.attn_norm[l], eps)
            if mix["kind"] == "R":
                qkv = O.gemv(O.Q8_0, mix["qkv"], xn, d["ch"], H)
                z = O.gemv(O.Q8_0, mix["gate"], xn, d["d_in"], H)
                g, b = self.OD.ab(xn, mix["alpha"], mix["beta"], mix["dt"], mix["a"])
                c = self.OD.conv(st[0], qkv, mix["ker"], d["ds"], 2 * d["hk"] * d["ds"], eps)
                att = self.OD.step(c, g, b, st[1], mix["norm"], z, d["hk"], d["hv"], kdiv=self.kdiv, eps=eps)
                mixed = O.gemv(O.Q8_0, mix["out"], att, H, d["d_in"])
            else:
                qfull = O.gemv(O.Q8_0, mix["q"], xn, a["hq"] * 2 * a["dh"], H).reshape(a["hq"], 2 * a["dh"])
                kin = O.gemv(O.Q8_0, mix["k"], xn, a["hkv"] * a["dh"], H).reshape(a["hkv"], a["dh"])
                vin = O.gemv(O.Q8_0, mix["v"], xn, a["hkv"] * a["dh"], H).reshape(a["hkv"], a["dh"])
                qhat = self.OA.prep(qfull, kin, vin, mix["qn"], mix["kn"], self.rope, pos, st[0], st[1], a["n_rot"], eps)
                att = self.OA.attend(qhat, st[0], st[1], qfull, pos).reshape(-1)
                mixed = O.gemv(O.Q8_0, mix["out"], att, H, a["hq"] * a["dh"])
            y = (x + mixed).astype(np.float32)
            xn2 = O.add_rms(y, m.post_norm[l], eps)
            x = (y + O.moe_ref(m.layers[l], xn2)["y"]).astype(np.float32)
        logits = O.gemv(O.Q6_K, m.head, O.add_rms(x, m.out_norm, eps), m.vocab, H)
        srt = np.sort(logits.astype(np.float64))
        self.last_margin = (float(srt[-1] - srt[-2]), float(np.abs(logits).max()))
        return O.argmax(logits)
