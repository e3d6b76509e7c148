"""The engine ABI (include/qk.h) on the GPU: qk_open on a synthetic MoE-only GGUF, then the slot
state machine and the stage calls, against
  - the state machine restated in oracle/qk_oracle_engine.py (pinned against the reference's stub
    engine in tests/test_engine_oracle.py), driven by the model's next-token map;
  - that map computed by the same kernels through the operator-level ABI, one launch at a time
    (bit-identical ids expected: same kernels, same inputs);
  - the CPU oracle's model step for every token of the vocabulary (greedy ids equal wherever the oracle's
    top-2 logit gap exceeds 2e-3 of the largest logit, the GEMV/MoE tolerance of 1e-3 on either side)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import qk_oracle_engine as OE  # noqa: E402

pytestmark = pytest.mark.gpu

H = 2048
VOCAB = int(os.environ.get("QK_TEST_VOCAB", "1024"))   # a smaller vocabulary (a multiple of 16, above 100) for slow runs


def walk(nxt, start, n, depth=1):
    out, t = [], start
    for _ in range(n):
        t = nxt(t, depth)
        out.append(t)
    return out


@pytest.fixture(scope="module")
def world(qk, dev, tmp_path_factory):
    """The model file, the model's next-token maps computed by the kernels, and the maps' check."""
    import torch
    model = qk.engine.StackModel(21, n_layer=2, vocab=VOCAB, n_expert=32, n_ff=512, n_used=8,
                                 down_types=[qk.IQ4_XS, qk.Q6_K])
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    embd, head, onorm = up(model.embd), up(model.head), up(model.out_norm)
    layers = [hl.to_device(dev) for hl in model.layers]
    pnorm = [up(w) for w in model.post_norm]
    ws = torch.zeros(max(qk.moe_workspace_bytes(L, 16) for L in layers), dtype=torch.uint8, device=dev)
    hws = torch.zeros(qk.head_workspace_bytes(VOCAB, 16), dtype=torch.uint8, device=dev)

    def step(ids, want_logits=False):   # one device step over len(ids) rows, as the engine chains it
        t = torch.tensor(ids, dtype=torch.int32, device=dev)
        x = qk.embed(model.embd_type, embd, VOCAB, H, t, len(ids))
        if len(ids) <= qk.ROWWISE_MAX:   # few rows: the norm rides inside each layer's launches
            for l, L in enumerate(layers):
                qk.moe_layer_rows(L, x, pnorm[l], ws)
            xn = qk.rmsnorm(x, onorm)
        else:
            xn = qk.rmsnorm(x, pnorm[0])
            for l, L in enumerate(layers):
                x, xn, _ = qk.moe_decode_tail(L, xn, x, pnorm[l + 1] if l + 1 < len(layers) else onorm, ws, S=x)
        tok, logits = qk.head_argmax(head, xn, VOCAB, H, hws, want_logits=want_logits)
        torch.cuda.synchronize()
        return (tok.cpu().tolist(), logits.cpu().numpy()) if want_logits else tok.cpu().tolist()

    print("[engine] next-token maps", flush=True)
    nxt1 = [step([t])[0] for t in range(VOCAB)]                      # one row: one-row kernels, one-row head
    nxtf = sum((step(list(range(t, t + 8))) for t in range(0, VOCAB, 8)), [])     # few rows: one-row MoE kernels, several-row head
    nxtn = sum((step(list(range(t, t + 16))) for t in range(0, VOCAB, 16)), [])   # many rows: expert-major MoE, several-row head
    # the end-of-sequence id goes into the file's metadata: take one that a stream reaches as its
    # 4th sample (the next-token maps do not depend on it)
    t0 = next(t for t in range(VOCAB) if len(set(walk(lambda u, z: nxt1[u], t, 4) + [t])) == 5)
    model.eos = walk(lambda u, z: nxt1[u], t0, 4)[3]
    path = model.write(str(tmp_path_factory.mktemp("engine") / "stack.gguf"))
    return dict(model=model, path=path, nxt1=nxt1, nxtf=nxtf, nxtn=nxtn, step=step, eos=model.eos, eos_prompt=t0,
                nxt=lambda t, z: nxt1[t] if z == 1 else nxtf[t] if z <= qk.ROWWISE_MAX else nxtn[t])


def test_next_token_maps(world, orc):
    nxt1, nxtn, model = world["nxt1"], world["nxtn"], world["model"]
    assert len(set(nxt1)) > VOCAB // 8            # a real map, not a constant
    nxtf = world["nxtf"]
    # few rows: the rows' company and position do not matter
    few = np.random.default_rng(2).permutation(VOCAB)[:15].tolist()
    for i in range(0, 15, 5):
        assert world["step"](few[i:i + 5]) == [nxtf[t] for t in few[i:i + 5]]
    # rows do not influence each other: another grouping of the same tokens gives the same ids
    perm = np.random.default_rng(1).permutation(VOCAB)[:48].tolist()
    for i in range(0, 48, 12):
        assert world["step"](perm[i:i + 12]) == [nxtn[t] for t in perm[i:i + 12]]
    # against the CPU oracle, EVERY token: all three kernel families give the oracle's id wherever its two
    # best logits lie further apart than both sides' tolerance (1e-3 of the largest logit each); a token on
    # which the families disagree with each other must therefore be such a near-tie
    threads = max(1, min(16, len(os.sched_getaffinity(0))))
    checked, ties = 0, []
    for t in range(VOCAB):
        want, gap, top = OE.stack_next(model, t, want_margin=True, threads=threads)
        if gap > 2e-3 * top:
            assert nxt1[t] == want and nxtf[t] == want and nxtn[t] == want, (t, gap, top, nxt1[t], nxtf[t], nxtn[t], want)
            checked += 1
        else:
            ties.append(t)
    print(f"[info] {checked} of {VOCAB} tokens decided by more than the tolerance; near-ties at {ties[:10]}", flush=True)
    assert checked >= VOCAB * 9 // 10   # about 2 % of random logit rows have their two best this close
    # every layer moves the result: without the last layer most next tokens change
    import copy
    short = copy.copy(model)
    short.layers, short.post_norm = model.layers[:1], model.post_norm[:1]
    changed = sum(OE.stack_next(short, t) != nxt1[t] for t in range(0, VOCAB, VOCAB // 16))
    assert changed >= 8, changed   # of sixteen samples


def drive(eng, ref, script, n_calls):
    """The same calls on the engine and on the restated state machine; every return must agree."""
    for call in range(n_calls):
        for op in script.get(call, []):
            if op[0] == "start":
                _, slot, prompt, max_gen, snap = op
                assert eng.slot_start(slot, prompt, max_gen, snap) == ref.slot_start(slot, prompt, max_gen, snap), op
            else:
                eng.slot_cancel(op[1])
                ref.slot_cancel(op[1])
        got, want = eng.step_chunk(), ref.step_chunk()
        assert got == want, (call, got, want)


def test_single_slot_stream(qk, world):
    nxt, EOS = world["nxt"], world["eos"]
    with qk.engine.Engine(world["path"], n_slots=1, n_ctx=128, chunk=4) as eng:
        assert (eng.vocab, eng.eos, eng.bos, eng.n_layer, eng.n_embd) == (VOCAB, EOS, 11, 2, H)
        assert (eng.n_slots, eng.n_ctx, eng.chunk, eng.state_n()) == (1, 128, 4, 3)
        ref = OE.SlotMachine(nxt, VOCAB, EOS, 1, 128, 4)
        assert eng.step_chunk() == (0, {0: []}, 0)
        # argument checks (reference src/main.cpp:5449-5453)
        assert eng.slot_start(1, [5], 4) == -1
        assert eng.slot_start(0, [], 4) == -3
        assert eng.slot_start(0, [5] * 100, 29) == -3
        assert eng.slot_start(0, [5, VOCAB], 4) == -4
        assert (eng.state_save(0, 2), eng.state_load(0, 2), eng.state_save(0, 3), eng.state_load(1, 0)) == (0, 0, -1, -1)
        start = next(t for t in range(100, VOCAB) if EOS not in walk(nxt, t, 12))
        drive(eng, ref, {0: [("start", 0, [3, 9, min(400, VOCAB - 1), start], 10, 0)],
                         1: [("start", 0, [1], 1, 0)]},     # busy: -2 on both
              6)
        assert not ref.slots[0]["active"]
        # the stream is the iterated map; a second request reuses the slot
        ref.depths.clear()
        drive(eng, ref, {0: [("start", 0, [world["eos_prompt"]], 50, 0)]}, 3)
        assert len(ref.depths) == 4 and not ref.slots[0]["active"]   # EOS as the 4th sample: 3 tokens, then finished


def test_slots_staggered_against_the_state_machine(qk, world, monkeypatch):
    nxt, EOS = world["nxt"], world["eos"]
    monkeypatch.setenv("QK_MAXB", "16")
    rng = np.random.default_rng(5)
    P = lambda n: [int(t) for t in rng.integers(8, VOCAB, n)]
    with qk.engine.Engine(world["path"], n_slots=6, n_ctx=256, chunk=5) as eng:
        ref = OE.SlotMachine(nxt, VOCAB, EOS, 6, 256, 5, max_b=16)
        script = {0: [("start", 2, P(3), 14, 0), ("start", 0, P(40), 7, 0)],        # 40: two batches of 16, 7 serial
                  1: [("start", 5, P(21), 30, 18), ("start", 2, P(2), 3, 0)],       # history boundary at 18; busy
                  2: [("cancel", 0), ("start", 1, P(1), 9, 0)],
                  3: [("start", 0, P(17), 2, 0), ("cancel", 4)],
                  6: [("start", 3, P(33), 12, 40), ("start", 6, P(3), 3, 0)],       # boundary beyond the prompt; bad slot
                  5: [("cancel", 5)],                                                # mid-stream
                  10: [("start", 0, P(2), 6, 0)]}                                    # alone: depth 1
        drive(eng, ref, script, 16)
        assert not any(sl["active"] for sl in ref.slots)
        assert 1 in ref.depths and max(ref.depths) == 6      # one-row and several-row steps both ran
        assert eng.step_chunk() == (0, {s: [] for s in range(6)}, 0)


def test_twelve_slots_take_the_expert_major_path(qk, world):
    nxt, EOS = world["nxt"], world["eos"]
    with qk.engine.Engine(world["path"], n_slots=12, n_ctx=64, chunk=3) as eng:
        ref = OE.SlotMachine(nxt, VOCAB, EOS, 12, 64, 3)
        script = {0: [("start", s, [20 + 7 * s], 5 + s % 3, 0) for s in range(12)]}
        drive(eng, ref, script, 5)
        assert ref.depths[0] == 12 and not any(sl["active"] for sl in ref.slots)


@pytest.mark.parametrize("seed", [1, 2])
def test_random_request_traffic(qk, world, seed):
    """Sixteen slots, requests arriving, finishing and being cancelled at random for a few hundred
    chunks: every return of the engine against the restated state machine."""
    import random
    nxt, EOS = world["nxt"], world["eos"]
    rnd = random.Random(seed)
    with qk.engine.Engine(world["path"], n_slots=16, n_ctx=96, chunk=4) as eng:
        ref = OE.SlotMachine(nxt, VOCAB, EOS, 16, 96, 4)
        script = {}
        for call in range(120):
            ops = []
            for _ in range(rnd.choice([0, 0, 1, 1, 2, 5])):
                slot = rnd.randrange(16)
                if rnd.random() < 0.15:
                    ops.append(("cancel", slot))
                else:
                    prompt = [rnd.randrange(VOCAB) for _ in range(rnd.choice([1, 2, 5, 18, 40]))]
                    ops.append(("start", slot, prompt, rnd.choice([1, 4, 9, 30, 60]), rnd.choice([0, 0, 17])))
            script[call] = ops
        drive(eng, ref, script, 150)
        assert len(set(ref.depths)) >= 8 and max(ref.depths) > qk.ROWWISE_MAX and min(ref.depths) <= 4


def test_serial_prefill_and_eager_launches_give_the_same_streams(qk, world, monkeypatch):
    """QK_NO_BATCH consumes every prompt token in a serial step; QK_NO_GRAPH launches the step's
    kernels one by one instead of replaying the captured graph.  Neither changes a token."""
    nxt, EOS = world["nxt"], world["eos"]
    rng = np.random.default_rng(9)
    prompts = [[int(t) for t in rng.integers(8, VOCAB, n)] for n in (19, 2, 6)]
    streams = {}
    for mode in ("graph", "eager"):
        if mode == "eager":
            monkeypatch.setenv("QK_NO_GRAPH", "1")
        monkeypatch.setenv("QK_NO_BATCH", "1")
        with qk.engine.Engine(world["path"], n_slots=3, n_ctx=128, chunk=8) as eng:
            ref = OE.SlotMachine(nxt, VOCAB, EOS, 3, 128, 8, no_batch=True)
            got = {s: [] for s in range(3)}
            for s, p in enumerate(prompts):
                assert eng.slot_start(s, p, 20) == 0 and ref.slot_start(s, p, 20) == 0
            for _ in range(8):
                a, b = eng.step_chunk(), ref.step_chunk()
                assert a == b
                for s in range(3):
                    got[s] += a[1][s]
            streams[mode] = got
    assert streams["graph"] == streams["eager"]
    assert sum(len(v) for v in streams["graph"].values()) > 20   # the streams ran on (an end id early in a stream shortens it)


def test_stage_run_and_topk(qk, world):
    nxt1, nxtn = world["nxt1"], world["nxtn"]
    with qk.engine.Engine(world["path"], n_slots=2, n_ctx=64, chunk=2) as eng:
        assert eng.stage_topk(4)[0] == -2                       # no run yet
        assert eng.stage_run(2, [1], 0)[0] == -1                # bad slot
        assert eng.stage_run(0, [1] * 10, 60)[0] == -1          # beyond n_ctx
        toks = [int(t) for t in np.random.default_rng(3).integers(0, VOCAB, 40)]
        rc, ids = eng.stage_run(1, toks, 8)                     # 16 + 16 + 8 rows
        assert rc == 0 and ids == [nxtn[t] for t in toks[:32]] + [world["nxtf"][t] for t in toks[32:]]
        rc, top_ids, top_vals = eng.stage_topk(5)
        assert rc == 0 and len(set(top_ids)) == 5
        assert all(a >= b for a, b in zip(top_vals, top_vals[1:]))
        # against the logits of the same position from the several-row head (1e-3 of the largest logit)
        _, logits = world["step"]([toks[-1], toks[-1]], want_logits=True)
        tol = 1e-3 * float(np.abs(logits[0]).max())
        np.testing.assert_allclose(top_vals, logits[0][top_ids], rtol=0, atol=tol)
        kth = np.sort(logits[0])[::-1][:5]
        np.testing.assert_allclose(top_vals, kth, rtol=0, atol=2 * tol)
        assert logits[0][ids[-1]] >= top_vals[0] - 2 * tol        # the greedy id leads the list up to a near-tie
        rc, ids = eng.stage_run(0, [toks[0]], 0)                # one row: the one-row kernels
        assert rc == 0 and ids == [nxt1[toks[0]]]
        assert eng.stage_topk(0)[0] == -1 and eng.stage_topk(257)[0] == -1
