"""The slot state machine restated in oracle/qk_oracle_engine.py, pinned against the reference's own
stub engine (stub/qk_stub.c compiled into oracle/_ref/libqk_stub.so) and against the closed form of
a memoryless model's token stream; and qk_open's checks that need no device."""
import ctypes as C
import os
import random
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import qk_oracle_engine as OE  # noqa: E402


def lcg(tok, depth=0):   # the stub's model (reference stub/qk_stub.c:10)
    return (tok * 1103515245 + 12345) % 2 ** 32 % 248000


def run_script(machines, script, max_chunks=400):
    """Drives engines with the same calls; returns each one's trace of (rc, tokens, finished)."""
    traces = [[] for _ in machines]
    for call in range(max_chunks):
        for op in script.get(call, []):
            for m, tr, shift in machines:
                if op[0] == "start":
                    _, slot, prompt, max_gen = op
                    tr.append(("start", m.slot_start(slot, shift(prompt), max_gen)))
                else:
                    m.slot_cancel(op[1])
        for i, (m, tr, _) in enumerate(machines):
            traces[i].append(m.step_chunk())
        if call > max(script) and traces[0][-1][0] == 0:
            break
    return traces


@pytest.mark.skipif(not OE.Stub.available(), reason="oracle/_ref/libqk_stub.so not built")
@pytest.mark.parametrize("seed", range(6))
def test_slot_machine_matches_reference_stub(seed):
    """The stub stays silent for n_prompt steps and then iterates its model from the last prompt
    token; the engine's first token comes from the step that feeds the last prompt token.  With
    the last prompt token doubled and serial prefill the two are step for step the same machine."""
    rnd = random.Random(seed)
    n_slots, chunk, n_ctx = rnd.choice([1, 3, 4, 16]), rnd.choice([1, 2, 5, 8, 32]), 256
    script = {}
    for _ in range(rnd.randint(2, 10)):
        call = rnd.randint(0, 12)
        slot = rnd.randrange(n_slots + 1)   # one past the end too: -1
        if rnd.random() < 0.2:
            script.setdefault(call, []).append(("cancel", slot))
            continue
        prompt = [rnd.randrange(8, 248320) for _ in range(rnd.randint(1, 20))]
        script.setdefault(call, []).append(("start", slot, prompt, rnd.choice([0, 1, 3, 17, 60])))
    script.setdefault(0, []).append(("start", 0, [100, 200], 9))
    stub = OE.Stub(n_slots, n_ctx, chunk)
    # the doubled token makes the engine's prompt one longer: n_ctx + 1 keeps the -3 bound the same
    mine = OE.SlotMachine(lcg, 248320, 248046, n_slots, n_ctx + 1, chunk, no_batch=True)
    try:
        t_stub, t_mine = run_script([(stub, [], lambda p: p), (mine, [], lambda p: p + p[-1:])], script)
    finally:
        stub.close()
    assert len(t_stub) == len(t_mine)
    for a, b in zip(t_stub, t_mine):
        assert a == b


def closed_form(nxt, prompt, max_gen, eos):
    out, t = [], prompt[-1]
    while len(out) < max_gen:
        t = nxt(t, 1)
        if t == eos:
            return out, True
        out.append(t)
    return out, False


@pytest.mark.parametrize("seed", range(8))
def test_slot_machine_closed_form(seed):
    """A memoryless model's stream is the iterated map from the last prompt token, cut at EOS (not
    emitted) or max_gen; token j leaves at the slot's step (serial prefill steps + j), whatever
    the other slots do."""
    rnd = random.Random(100 + seed)
    vocab, eos = 97, 13
    table = [rnd.randrange(vocab) for _ in range(vocab)]
    n_slots, chunk, max_b = rnd.choice([1, 2, 5, 16]), rnd.choice([1, 3, 8]), rnd.choice([16, 32, 128])
    no_batch = bool(seed % 2)
    m = OE.SlotMachine(lambda t, z: table[t], vocab, eos, n_slots, 512, chunk, max_b=max_b, no_batch=no_batch)
    plans = {}
    for s in range(n_slots):
        prompt = [rnd.randrange(vocab) for _ in range(rnd.choice([1, 2, 15, 16, 17, 40, 150]))]
        plans[s] = dict(prompt=prompt, max_gen=rnd.choice([1, 5, 30]), at=rnd.randint(0, 3), snap=rnd.choice([0, 0, 20]))
    got = {s: [] for s in plans}
    first_call, fin_call = {}, {}
    for call in range(300):
        for s, p in plans.items():
            if p["at"] == call:
                assert m.slot_start(s, p["prompt"], p["max_gen"], p["snap"]) == 0
                assert m.slot_start(s, p["prompt"], p["max_gen"]) == -2
        rc, out, fin = m.step_chunk()
        assert rc == sum(1 for s, p in plans.items() if p["at"] <= call and s not in fin_call)
        for s in plans:
            assert len(out[s]) <= chunk
            if out[s] and s not in first_call:
                first_call[s] = call
            got[s] += out[s]
            if fin >> s & 1:
                assert s not in fin_call
                fin_call[s] = call
        if len(fin_call) == len(plans):
            break
    for s, p in plans.items():
        want, hit_eos = closed_form(lambda t, z: table[t], p["prompt"], p["max_gen"], eos)
        assert got[s] == want
        # serial prefill steps: what the batch rule leaves of the first n_prompt - 1 positions
        target, done = len(p["prompt"]) - 1, 0
        if not no_batch:
            for limit in ([p["snap"]] if 0 < p["snap"] < target else []) + [target]:
                while limit > done and limit - done >= 16:
                    done += min(max_b, limit - done)
        silent = target - done
        assert 0 <= silent < 16 or no_batch
        if want:
            assert first_call[s] == p["at"] + silent // chunk
        steps = silent + len(want) + (1 if hit_eos else 0)   # the EOS step emits nothing
        assert fin_call[s] == p["at"] + (steps - 1) // chunk


# ---- qk_open: everything it checks before it touches a device ---------------------------------

class Cfg(C.Structure):
    _fields_ = [("n_slots", C.c_uint32), ("n_ctx", C.c_uint32), ("chunk", C.c_uint32)]


def try_open(qk, path, cfg=(2, 256, 4)):
    L = qk.lib()
    L.qk_open.restype = C.c_void_p
    L.qk_open.argtypes = [C.c_char_p, C.c_void_p, C.c_char_p, C.c_size_t]
    L.qk_close.argtypes = [C.c_void_p]
    err = C.create_string_buffer(512)
    h = L.qk_open(str(path).encode(), C.byref(Cfg(*cfg)), err, 512)
    if h:
        L.qk_close(h)
    return bool(h), err.value.decode()


@pytest.fixture(scope="module")
def tiny(qk):
    return qk.engine.StackModel(3, n_layer=2, vocab=256, n_expert=8, n_ff=256, n_used=8)


def test_open_rejects_what_the_reference_rejects(qk, tiny, tmp_path, monkeypatch):
    monkeypatch.delenv("QK_LAYERS", raising=False)
    p = tmp_path / "m.gguf"
    (tmp_path / "junk.gguf").write_bytes(b"not a gguf file at all")
    assert try_open(qk, tmp_path / "junk.gguf") == (False, "qk_open: cannot open GGUF")

    def variant(kvs=None, drop=(), add=(), retype=None):
        k = tiny.kvs()
        k.update(kvs or {})
        t = [x for x in tiny.tensors() if x[0] not in drop] + list(add)
        if retype:
            t = [(n, retype[n], ne, d) if n in retype else (n, ty, ne, d) for n, ty, ne, d in t]
        qk.gguf.write(str(p), k, t)
        return try_open(qk, p)

    assert variant(kvs={"qwen35moe.block_count": 0}) == (False, "qk_open: bad block_count")
    assert variant(kvs={"qwen35moe.block_count": 257}) == (False, "qk_open: bad block_count")
    assert variant(kvs={"qwen35moe.expert_used_count": 17}) == (False, "qk_open: expert_used_count > 16 unsupported")
    for name in ("token_embd.weight", "output_norm.weight", "output.weight"):
        assert variant(drop=(name,)) == (False, "qk_open: missing/unexpected embd/head tensors")
    ok, msg = variant(drop=("blk.1.ffn_up_exps.weight",))
    assert not ok and "ffn_up_exps" in msg
    assert variant(drop=("blk.1.post_attention_norm.weight",)) == \
        (False, "qk_open: missing/unexpected post_attention_norm tensor")
    # mixer tensors on some layers only, or without the tensor that tells the kind of mixer
    stray = lambda name: variant(add=[(name, qk.F32, (2048, 4), np.zeros(8192, np.float32))])
    assert stray("blk.0.attn_q.weight") == (False, "qk_open: layers with and without mixers in one file")
    assert stray("blk.1.ssm_a") == (False, "qk_open: layers with and without mixers in one file")
    for name in ("blk.1.attn_qkv.weight", "blk.0.ssm_out.weight"):
        assert stray(name) == (False, "qk_open: a layer has mixer tensors but neither ssm_a nor attn_q")
    monkeypatch.setenv("QK_LAYERS", "2:1")
    assert variant() == (False, "qk_open: bad QK_LAYERS (want a:b with 0 <= a < b <= 2)")
    monkeypatch.setenv("QK_LAYERS", "1:2")
    ok, msg = variant()
    assert not ok and "pipeline stages" in msg
    monkeypatch.setenv("QK_LAYERS", "0:2")   # the whole model: not a split


def test_open_needs_a_device(qk, tiny, tmp_path, monkeypatch):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    monkeypatch.delenv("QK_LAYERS", raising=False)
    p = tiny.write(str(tmp_path / "m.gguf"))
    ok, msg = try_open(qk, p)
    assert not ok and "no HIP device" in msg
