"""qk_open on a synthetic whole-model GGUF (gated-DeltaNet and full-attention layers, each followed
by a MoE block): the engine's token streams against the restated state machine driving the CPU
oracle of the whole model (oracle/qk_oracle_engine.py FullModelOracle: the reference's recorded step,
src/main.cpp:4194-4419, from the oracles of its parts).  Greedy tokens are compared exactly: the
kernels agree with the oracle to 1e-3, so a step whose two best logits lie closer than that could
legitimately differ; the seeds used here have no such step among those that decide a token (the
narrowest gap seen is printed)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import qk_oracle_engine as OE  # noqa: E402

pytestmark = pytest.mark.gpu

VOCAB = 384


class Checked:
    """The oracle model behind the state machine, recording the narrowest margin it saw."""

    def __init__(self, model, n_slots, n_ctx):
        self.o = OE.FullModelOracle(model, n_slots, n_ctx)
        self.narrowest = np.inf

    def reset(self, slot):
        self.o.reset(slot)

    def feed(self, slot, token, pos, depth):
        t = self.o.feed(slot, token, pos, depth)
        gap, top = self.o.last_margin
        self.narrowest = min(self.narrowest, gap / top)
        return t


@pytest.fixture(scope="module")
def full(qk, dev, tmp_path_factory):
    model = qk.engine.FullModel(17, kinds="RRAR", vocab=VOCAB, eos=VOCAB + 5)
    path = model.write(str(tmp_path_factory.mktemp("full") / "model.gguf"))
    return model, path


def drive(eng, ref, script, n_calls):
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


def test_whole_model_streams(qk, full):
    """Three slots with different prompt lengths (serial prefill, a prefilled prompt, a one-token
    prompt), a slot reused after it finished, one cancelled: the recurrent state and the KV rows of a
    slot belong to it alone and are cleared when the next request takes the slot."""
    model, path = full
    print("[case] whole model, three slots", flush=True)
    rng = np.random.default_rng(4)
    P = lambda n: [int(t) for t in rng.integers(0, VOCAB, n)]
    with qk.engine.Engine(path, n_slots=3, n_ctx=96, chunk=3) as eng:
        assert (eng.vocab, eng.n_layer, eng.eos) == (VOCAB, 4, VOCAB + 5)
        chk = Checked(model, 3, 96)
        ref = OE.SlotMachine(chk, VOCAB, VOCAB + 5, 3, 96, 3)
        script = {0: [("start", 1, P(5), 7, 0)],
                  1: [("start", 0, P(20), 5, 0), ("start", 2, P(1), 9, 0)],   # 20 tokens: 19 prefilled at the start
                  3: [("cancel", 2)],
                  4: [("start", 2, P(3), 4, 0)],                               # slot 2 again, fresh state
                  6: [("start", 1, P(2), 3, 0)]}                               # slot 1 again after it finished
        drive(eng, ref, script, 10)
        assert not any(sl["active"] for sl in ref.slots)
        print(f"[info] narrowest top-2 gap / largest logit over all steps fed: {chk.narrowest:.2e}", flush=True)


def test_whole_model_eager_launches_and_serial_prefill(qk, full, dev, monkeypatch, switches_back_to_defaults):
    """QK_NO_GRAPH launches the kernels one by one; QK_NO_BATCH feeds every prompt token in a serial
    step instead of at the start; QK_MAXB moves the border between prefilled and serially fed positions,
    QK_PREFILL_ROWS sets the rows per prefill pass; QK_DN_FUSED, QK_FUSED_NORM, QK_ATTN_BLOCK and QK_ONE_ROW
    choose between kernel forms of the same step (on a device only once those forms have had their first
    run there): the same streams."""
    from conftest import SWITCH_ENV_DEFAULTS, unrun_forms_allowed
    model, path = full
    print("[case] whole model, eager / serial prefill", flush=True)
    prompt = [int(t) for t in np.random.default_rng(6).integers(0, VOCAB, 18)]
    streams = []
    cases = [{}, {"QK_NO_GRAPH": "1"}, {"QK_NO_BATCH": "1"}, {"QK_MAXB": "16"},
             {"QK_PREFILL_ROWS": "16"}]    # QK_MAXB 16: 16 positions prefilled, one serial step more; rows 16: two passes
    if unrun_forms_allowed(dev):
        cases += [{"QK_DN_FUSED": "1"},         # the gated-DeltaNet step as one launch: the same bits
                  {"QK_ONE_ROW": "stream", "QK_DENSE_REG": "1"},   # block rows streamed through LDS
                  {"QK_ONE_ROW": "stream", "QK_FUSED_NORM": "1"},  # no norm launches: the same sums scaled later
                  {"QK_ATTN_BLOCK": "1"},       # the prompt's attention sixteen rows at a time
                  {"QK_GEMM_TILED": "1"},       # (passes of 64 rows and more only: here the same kernels)
                  {"QK_MOE_ROWS": "1"}]         # the prompt's 17 positions through the row-split expert kernels
    for env in cases:
        for k in ("QK_NO_GRAPH", "QK_NO_BATCH", "QK_MAXB", "QK_PREFILL_ROWS"):
            monkeypatch.delenv(k, raising=False)
        for k, v in {**SWITCH_ENV_DEFAULTS, **env}.items():   # qk_open applies the switches that are set
            monkeypatch.setenv(k, v)
        with qk.engine.Engine(path, n_slots=2, n_ctx=64, chunk=8) as eng:
            assert eng.slot_start(1, prompt, 6) == 0
            got = []
            for _ in range(4):
                rc, out, fin = eng.step_chunk()
                got += out[1]
            streams.append(got)
    assert len(streams[0]) == 6 and all(st == streams[0] for st in streams)


def test_whole_model_stage_run_and_snapshots(qk, full):
    """qk_stage_run feeds a slot's positions in order; a snapshot taken after a prefix brings the slot
    back to it (qk_state_save / qk_state_load), so the continuation repeats."""
    model, path = full
    print("[case] whole model, stage run and snapshots", flush=True)
    toks = [int(t) for t in np.random.default_rng(9).integers(0, VOCAB, 9)]
    with qk.engine.Engine(path, n_slots=2, n_ctx=64, chunk=2) as eng:
        o = OE.FullModelOracle(model, 1, 64)
        want = [o.feed(0, t, p) for p, t in enumerate(toks)]
        rc, ids = eng.stage_run(1, toks[:6], 0)
        assert rc == 0 and ids == want[:6]
        assert eng.state_save(1, 2, 6) == 0
        rc, tail = eng.stage_run(1, toks[6:], 6)
        assert rc == 0 and tail == want[6:]
        rc, top_ids, top_vals = eng.stage_topk(3)
        assert rc == 0 and top_ids[0] == tail[-1] and top_vals[0] >= top_vals[1] >= top_vals[2]
        # other tokens move the state on; loading the snapshot restores the prefix's state
        rc, other = eng.stage_run(1, [7, 8, 9], 6)
        assert rc == 0
        assert eng.state_load(1, 2, 6) == 0
        rc, again = eng.stage_run(1, toks[6:], 6)
        assert rc == 0 and again == tail
        assert eng.state_save(1, 3, 0) == -1 and eng.state_load(2, 0, 0) == -1


@pytest.mark.parametrize("tiled", [False, True], ids=["defaults", "gemm_tiled"])
def test_whole_model_long_prompt_and_long_stage_run(qk, full, dev, monkeypatch, switches_back_to_defaults, tiled):
    """A prompt longer than one prefill pass (64 positions here go through the projections and the
    MoE blocks together, the mixers through their sequence kernels), then two more passes, then the
    serial steps: the same stream as the oracle fed one token at a time.  qk_stage_run over 40
    positions returns the oracle's id after every one of them.  With the "gemm_tiled" switch the passes
    of 64 rows run their dense projections through the kernel that decodes a weight tile once per 128 rows."""
    from conftest import UNRUN, unrun_forms_allowed
    if tiled and not unrun_forms_allowed(dev):
        pytest.skip(UNRUN)
    model, path = full
    monkeypatch.setenv("QK_GEMM_TILED", "1" if tiled else "0")
    monkeypatch.setenv("QK_PREFILL_ROWS", "64")
    print("[case] whole model, 150-token prompt and a 40-position stage run", flush=True)
    rng = np.random.default_rng(21)
    prompt = [int(t) for t in rng.integers(0, VOCAB, 150)]
    with qk.engine.Engine(path, n_slots=2, n_ctx=192, chunk=4) as eng:
        chk = Checked(model, 2, 192)
        ref = OE.SlotMachine(chk, VOCAB, VOCAB + 5, 2, 192, 4)
        drive(eng, ref, {0: [("start", 1, prompt, 6, 0)], 1: [("start", 0, prompt[:40], 3, 0)]}, 3)
        assert not any(sl["active"] for sl in ref.slots)
        print(f"[info] narrowest top-2 gap / largest logit: {chk.narrowest:.2e}", flush=True)
        o = OE.FullModelOracle(model, 1, 192)
        want = [o.feed(0, t, p) for p, t in enumerate(prompt[:40])]
        rc, ids = eng.stage_run(0, prompt[:40], 0)
        assert rc == 0 and ids == want


def test_whole_model_stream_alone_and_among_fifteen_neighbours(qk, full):
    """The same request on slot 0 alone (dispatch depth 1: the one-row kernels) and with fifteen busy
    neighbours (depth 16: projections, MoE block and head on the matrix cores).  The kernel families sum
    in different orders, so the greedy streams may part -- but only at a step whose two best logits nearly
    tie: the streams must agree up to the first difference, and there qk_stage_topk over the common prefix
    must show the two ids as its two best, closer together than 2e-3 of the largest logit."""
    model, path = full
    print("[case] whole model, one stream alone and among fifteen neighbours", flush=True)
    rng = np.random.default_rng(77)
    P = lambda n: [int(t) for t in rng.integers(0, VOCAB, n)]
    prompt, n_gen = P(6), 10

    def stream_of_slot_0(eng):
        got = []
        for _ in range(40):
            rc, out, fin = eng.step_chunk()
            assert rc >= 0
            got += out[0]
            if fin & 1:
                return got
        raise AssertionError("slot 0 did not finish")

    with qk.engine.Engine(path, n_slots=16, n_ctx=64, chunk=4) as eng:
        assert eng.slot_start(0, prompt, n_gen) == 0
        alone = stream_of_slot_0(eng)
        for s in range(1, 16):
            assert eng.slot_start(s, P(2 + s % 5), 40) == 0
        assert eng.slot_start(0, prompt, n_gen) == 0
        crowd = stream_of_slot_0(eng)
        for s in range(1, 16):
            eng.slot_cancel(s)
        assert len(alone) == len(crowd) == n_gen   # the end id lies outside the vocabulary: both run to max_gen
        j = next((i for i, (a, b) in enumerate(zip(alone, crowd)) if a != b), None)
        print(f"[info] alone {alone}\n[info] crowd {crowd}\n[info] first difference at {j}", flush=True)
        if j is not None:
            rc, _ = eng.stage_run(0, prompt + alone[:j], 0)
            assert rc == 0
            rc, top_ids, top_vals = eng.stage_topk(3)
            assert rc == 0 and {alone[j], crowd[j]} == set(top_ids[:2]), (j, alone[j], crowd[j], top_ids, top_vals)
            assert top_vals[0] - top_vals[1] <= 2e-3 * max(abs(v) for v in top_vals), (j, top_ids, top_vals)


@pytest.mark.parametrize("ba", ["f32", "q8_0", "iq4_xs"])
def test_whole_model_fused_ssm_ba(qk, orc, dev, ba, tmp_path):
    """A file that holds the decay / write-strength weights of its gated-DeltaNet layers as ONE interleaved
    tensor ssm_ba (the qwen3next form, reference src/main.cpp:3931-3948): per key-head group the rows 4g,
    4g+1 are beta, 4g+2, 4g+3 alpha.  F32: the very numbers of the split form, so the engine gives the
    split file's ids; Q8_0 / IQ4_XS: the oracle's model takes the oracle's dequantised rows."""
    type_ = {"f32": qk.F32, "q8_0": qk.Q8_0, "iq4_xs": qk.IQ4_XS}[ba]
    print(f"[case] whole model, fused ssm_ba as {ba}", flush=True)
    FM = qk.engine.FullModel
    model = FM(23, kinds="RAR", vocab=VOCAB, eos=VOCAB + 5, fused_ba=type_)
    for m in model.mix:
        if m["kind"] == "R" and m["alpha"] is None:
            rows = orc.dequant(type_, m["ba"], 64 * 2048).reshape(64, 2048)
            m["alpha"], m["beta"] = FM.split_ba(rows)
    toks = [int(t) for t in np.random.default_rng(8).integers(0, VOCAB, 8)]
    o = OE.FullModelOracle(model, 1, 64)
    want = [o.feed(0, t, p) for p, t in enumerate(toks)]
    with qk.engine.Engine(model.write(str(tmp_path / "fused.gguf")), n_slots=1, n_ctx=64, chunk=2) as eng:
        rc, ids = eng.stage_run(0, toks, 0)
        assert rc == 0 and ids == want
    if ba == "f32":
        split = FM(23, kinds="RAR", vocab=VOCAB, eos=VOCAB + 5)
        assert all(np.array_equal(a["alpha"], b["alpha"]) and np.array_equal(a["beta"], b["beta"])
                   for a, b in zip(model.mix, split.mix) if a["kind"] == "R")
        with qk.engine.Engine(split.write(str(tmp_path / "split.gguf")), n_slots=1, n_ctx=64, chunk=2) as eng:
            assert eng.stage_run(0, toks, 0) == (0, ids)


def test_whole_model_pass_size_does_not_change_the_ids(qk, full, monkeypatch):
    """600 positions through qk_stage_run in one pass (the default of 1,024 rows), in passes of 64 and
    of 16 rows: the same greedy ids.  The oracle is too slow for passes this long, so the large
    pass is held against the small ones, which the oracle pins above.  The kernels' sums run in
    another order for another row count, so a position whose two best logits nearly tie may differ
    -- and only such a position: qk_stage_run feeds the given tokens, so an id that differs does not
    move the states, and for every position whose ids differ the run is repeated up to that position
    and qk_stage_topk must show the two ids as its two best, closer together than 2e-3 of the
    largest logit (the 1e-3 tolerance of either pass)."""
    model, path = full
    n_pos = int(os.environ.get("QK_TEST_POSITIONS", "600"))   # fewer for slow runs
    print(f"[case] whole model, {n_pos} positions in passes of 1024 / 64 / 16 rows", flush=True)
    toks = [int(t) for t in np.random.default_rng(33).integers(0, VOCAB, n_pos)]
    ids = {}
    for rows in ("1024", "64", "16"):
        monkeypatch.setenv("QK_PREFILL_ROWS", rows)
        with qk.engine.Engine(path, n_slots=1, n_ctx=640, chunk=2) as eng:
            rc, got = eng.stage_run(0, toks, 0)
            assert rc == 0 and len(got) == n_pos
            ids[rows] = got
    differing = sorted({i for other in ("64", "16") for i in range(n_pos) if ids["1024"][i] != ids[other][i]})
    print(f"[info] positions whose ids differ between passes of 1024 / 64 / 16 rows: {differing}", flush=True)
    assert len(differing) <= 12   # near-ties are rare; more than this is a defect whatever the margins say
    monkeypatch.setenv("QK_PREFILL_ROWS", "64")
    with qk.engine.Engine(path, n_slots=1, n_ctx=640, chunk=2) as eng:
        for i in differing:
            rc, got = eng.stage_run(0, toks[:i + 1], 0)
            assert rc == 0 and got == ids["64"][:i + 1]
            rc, top_ids, top_vals = eng.stage_topk(3)
            assert rc == 0
            seen = {ids[r][i] for r in ("1024", "64", "16")}
            assert seen == set(top_ids[:2]), (i, seen, top_ids, top_vals)
            assert top_vals[0] - top_vals[1] <= 2e-3 * max(abs(v) for v in top_vals), (i, top_ids, top_vals)
