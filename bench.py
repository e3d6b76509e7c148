#!/usr/bin/env python3
"""Benchmark of the quantized-weight decode hot path on one MI355X.

Headline workload (config.workload = "moe_decode_bs1"): one fused Qwen3-MoE decode layer,
hidden 2048, 256 experts, top-8, IQ3_XXS gate/up, IQ4_XS down, Q8_0 shared expert, bs=1.
A "step" is one call of qkk_moe_decode().  Steps run over a ring of distinct synthetic
layers whose total size exceeds the 256 MB last-level cache (as the 40 layers of a real
decode do), captured in a HIP graph; inputs are resident in HBM before the timed region.
`value` is algorithmic bytes per step / step time, in GB/s.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--ring R]
                  [--extras/--no-extras] [--cpu/--no-cpu]

Prints ONE JSON line.  --gpus above 1 is refused: this build drives one GPU.  The default run is three
parts -- the headline workload and the side measurements (`extras`) in a child process each, the CPU baseline
in this one -- so no side measurement can take the headline with it; with --no-extras, or any other
--workload, everything runs in this process (the form to put behind `rocprofv3 ... --`).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0   # dense fp16 matrix peak
MIN_REPLAYS = 20   # graph replays timed at least, whatever --steps says (steps timed = replays x ring, reported)
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by what the same
# counters read for a plain 256 MiB copy (profiles/); None where no counter run of the CURRENT kernel
# has been recorded (a figure of an earlier version of a kernel is not carried over).
TRAFFIC = {"moe_gateup_fused_kernel": 85845150,   # profiles/moe_decode_bs16_hbm_traffic.txt (103 distinct experts)
           "moe_gateup_kernel": 6722843}          # profiles/moe_decode_bs1_hbm_traffic.txt: the per-lane form (the default)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gpu_time_ms(fn, reps):
    """Mean milliseconds of fn() over reps calls, HIP events on the current stream."""
    import torch
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


class Graphed:
    """A list of launches captured once into a HIP graph on a side stream."""

    def __init__(self, launches):
        import torch
        self.n = len(launches)
        self.stream = torch.cuda.Stream()
        # the tensors were filled (and the workspace cleared) on the current stream: without this
        # the warm-up below can start on memory those launches have not written yet
        self.stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(self.stream):
            for f in launches:  # eager warm-up (also first-touch of every buffer)
                f()
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=self.stream):
            for f in launches:
                f()
        torch.cuda.synchronize()

    def replay(self):
        self.graph.replay()


def run_ring(launches, steps, warmup):
    """Times `steps` launches (a multiple of the ring) bracketed by synchronize.  Returns
    (ms_per_step by the host clock over the whole region, MEDIAN ms_per_step over the graph replays by HIP
    events on the launch stream, steps timed).  At least MIN_REPLAYS replays are timed."""
    import torch
    g = Graphed(launches)
    reps = max(MIN_REPLAYS, steps // g.n)   # never a single replay: a driver's small --steps still times twenty
    for _ in range(max(1, warmup // g.n)):
        g.replay()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    t0 = time.perf_counter()
    marks[0].record()   # replays and events both go to torch's current stream
    for r in range(reps):
        g.replay()
        marks[r + 1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per = sorted(marks[r].elapsed_time(marks[r + 1]) for r in range(reps))
    n = reps * g.n
    return (t1 - t0) * 1e3 / n, per[reps // 2] / g.n, n


# ---- workloads -------------------------------------------------------------------------------

def moe_workload(qk, n_slots, down_type, ring, steps, warmup, seed=1234, slab=False):
    """slab: the ring's tensors in ONE device allocation instead of one per tensor (same bytes, same
    addresses' spread): separates what the step pays for address translation over many mappings."""
    import torch
    dev = "cuda:0"
    pool = qk.synth.Slab(ring * qk.synth.layer_bytes(down_type=down_type), dev) if slab else None
    layers = [qk.synth.device_layer(seed + 16 * i, down_type=down_type, device=dev, slab=pool) for i in range(ring)]
    if slab:
        torch.cuda.empty_cache()   # the generators' own allocations go back to the driver
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    X = torch.randn((ring, n_slots, 2048), device=dev, generator=g)
    Y = torch.empty_like(X)
    sel = torch.zeros((ring, n_slots, 160), dtype=torch.uint8, device=dev)
    ws = torch.zeros(qk.moe_workspace_bytes(layers[0], n_slots), dtype=torch.uint8, device=dev)

    def step(i, stages=None):
        return lambda: qk.moe_decode(layers[i], X[i], ws, Y[i], sel[i], stages=stages)

    wall, ev, n = run_ring([step(i) for i in range(ring)], steps, warmup)
    # distinct experts touched per step (bs=1: n_used)
    ids = sel.cpu().numpy().view("uint32").reshape(ring, n_slots, 40)[:, :, :8]
    distinct = [len(set(ids[i].reshape(-1).tolist())) for i in range(ring)]
    u = sum(distinct) / len(distinct)
    L = layers[0]
    act = n_slots * (2048 * 4 * 2 + 160)  # x in, y out, sel out
    bytes_step = L.active_bytes(u) + act
    # per-stage kernel time: the same ring, one stage per launch
    stage_ms = {}
    for name, mask in (("route", 1), ("gateup", 2), ("down", 4)):
        _, sev, _ = run_ring([step(i, mask) for i in range(ring)], max(ring * 5, steps // 2), ring)
        stage_ms[name] = sev
    H, F = 2048, 512
    gu_bytes = u * 2 * F * qk.row_bytes(qk.IQ3_XXS, H) + n_slots * (H * 4 + 9 * F * 4)
    if 2 <= n_slots <= 32:   # few rows: the same launch streams the shared expert's gate and up rows
        gu_bytes += 2 * F * qk.row_bytes(qk.Q8_0, H) * ((n_slots + 15) // 16)
    return dict(ms_wall=wall, ms_event=ev, steps=n, bytes_step=bytes_step, distinct_experts=u, stage_ms=stage_ms,
                gateup_bytes=gu_bytes, ring=ring, ring_bytes=ring * L.active_bytes(L.n_expert))


def moe_tail_workload(qk, n_slots, down_type, ring, steps, warmup, seed=1234, layer_row=False):
    """The step with the layer tail behind it (qkk_moe_decode_tail): residual add and the next
    layer's RMS norm.  Same ring and inputs as moe_workload; returns microseconds per step.
    layer_row: the one-row block with the norm in front instead (qkk_moe_layer_rows, in place on R)."""
    import torch
    dev = "cuda:0"
    layers = [qk.synth.device_layer(seed + 16 * i, down_type=down_type, device=dev) for i in range(ring)]
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    X = torch.randn((ring, n_slots, 2048), device=dev, generator=g)
    R = torch.randn((ring, n_slots, 2048), device=dev, generator=g)
    W = torch.rand((ring, 2048), device=dev, generator=g) + 0.5
    S, Xn = torch.empty_like(X), torch.empty_like(X)
    sel = torch.zeros((ring, n_slots, 160), dtype=torch.uint8, device=dev)
    ws = torch.zeros(qk.moe_workspace_bytes(layers[0], n_slots), dtype=torch.uint8, device=dev)
    if layer_row:
        _, ev, _ = run_ring([(lambda i=i: qk.moe_layer_rows(layers[i], R[i], W[i], ws, sel=sel[i])) for i in range(ring)],
                            steps, warmup)
        return ev * 1e3
    _, ev, _ = run_ring([(lambda i=i: qk.moe_decode_tail(layers[i], X[i], R[i], W[i], ws, S=S[i], Xn=Xn[i], sel=sel[i]))
                         for i in range(ring)], steps, warmup)
    return ev * 1e3


def norm_workload(qk, rows, steps, warmup):
    """add_rmsnorm on `rows` rows of 2048 (ring of 64 distinct row sets)."""
    import torch
    dev = "cuda:0"
    ring = 64
    A, B = torch.randn((2, ring, rows, 2048), device=dev)
    W = torch.rand(2048, device=dev) + 0.5
    Y, Xn = torch.empty_like(A), torch.empty_like(A)
    _, ev, _ = run_ring([(lambda i=i: qk.add_rmsnorm(A[i], B[i], W, y=Y[i], xn=Xn[i])) for i in range(ring)], steps, warmup)
    return ev * 1e3


def gemv_workload(qk, type_, M, K, batch, steps, warmup, seed=99, ring=None):
    import torch
    dev = "cuda:0"
    rb = qk.row_bytes(type_, K)
    ring = ring or max(2, int(320e6 // (M * rb)) + 1)
    be = qk.capi.BLOCK[type_][0]
    if type_ == qk.F16:
        Ws = [(torch.randn(M * K, device=dev) * 0.05).to(torch.float16) for _ in range(ring)]
    else:
        Ws = [qk.synth.blocks_device(type_, M * (K // be), seed + i, dev).reshape(-1) for i in range(ring)]
    X = torch.randn((ring, batch, K), device=dev)
    Y = torch.empty((ring, batch, M), device=dev)
    wall, ev, n = run_ring([(lambda i=i: qk.gemv(type_, Ws[i], X[i], M, K, out=Y[i])) for i in range(ring)],
                           steps, warmup)
    return dict(ms_wall=wall, ms_event=ev, steps=n, bytes_step=M * rb + batch * (K + M) * 4, ring=ring)


def head_workload(qk, V, K, batch, steps, warmup, seed=77):
    import torch
    dev = "cuda:0"
    ring = 2
    Ws = [qk.synth.blocks_device(qk.Q6_K, V * (K // 256), seed + i, dev).reshape(-1) for i in range(ring)]
    X = torch.randn((ring, batch, K), device=dev)
    ws = torch.zeros(qk.head_workspace_bytes(V, batch), dtype=torch.uint8, device=dev)
    toks = []

    def step(i):
        def f():
            toks.append(qk.head_argmax(Ws[i], X[i], V, K, ws)[0])
        return f

    # head_argmax allocates its small token tensor: do that outside the capture
    import ctypes as C
    tok = torch.zeros((ring, batch), dtype=torch.int32, device=dev)
    L = qk.lib()

    def raw(i):
        def f():
            rc = L.qkk_head_argmax(C.c_void_p(Ws[i].data_ptr()), C.c_void_p(X[i].data_ptr()),
                                   C.c_void_p(tok[i].data_ptr()), None, V, K, batch, C.c_void_p(ws.data_ptr()),
                                   ws.numel(), C.c_void_p(torch.cuda.current_stream().cuda_stream))
            assert rc == 0, L.qkk_last_error()
        return f

    wall, ev, n = run_ring([raw(i) for i in range(ring)], steps, warmup)
    return dict(ms_wall=wall, ms_event=ev, steps=n, bytes_step=V * qk.row_bytes(qk.Q6_K, K) + batch * (K * 4 + 4),
                ring=ring)


def gemm_workload(qk, M, K, N, steps, warmup, seed=55):
    import torch
    dev = "cuda:0"
    ring = max(2, int(320e6 // (M * K // 32 * 34)) + 1)
    Ws = [qk.synth.blocks_device(qk.Q8_0, M * K // 32, seed + i, dev).reshape(-1) for i in range(ring)]
    X = torch.rand((ring, N, K), device=dev) * 2 - 1
    Y = torch.empty((ring, N, M), device=dev)
    wall, ev, n = run_ring([(lambda i=i: qk.gemm_q8_0(Ws[i], X[i], M, K, out=Y[i])) for i in range(ring)],
                           steps, warmup)
    return dict(ms_event=ev, flops=2.0 * M * K * N, bytes_step=M * K // 32 * 34 + N * K * 4 + N * M * 4)


def prefill_moe_workload(qk, n_tokens, steps, warmup, seed=4242):
    import torch
    dev = "cuda:0"
    ring = 2
    layers = [qk.synth.device_layer(seed + 16 * i, down_type=qk.IQ4_XS, device=dev) for i in range(ring)]
    X = torch.randn((ring, n_tokens, 2048), device=dev)
    Y = torch.empty_like(X)
    sel = torch.zeros((ring, n_tokens, 160), dtype=torch.uint8, device=dev)
    ws = torch.zeros(qk.moe_prefill_workspace_bytes(layers[0], n_tokens), dtype=torch.uint8, device=dev)
    wall, ev, n = run_ring([(lambda i=i: qk.moe_prefill(layers[i], X[i], ws, Y[i], sel[i])) for i in range(ring)],
                           steps, warmup)
    ids = sel.cpu().numpy().view("uint32").reshape(ring, n_tokens, 40)[:, :, :8]
    u = sum(len(set(ids[i].reshape(-1).tolist())) for i in range(ring)) / ring
    L = layers[0]
    H, F = 2048, 512
    flops = 2.0 * n_tokens * 8 * (2 * F * H + H * F) + 2.0 * n_tokens * (256 * H + 3 * F * H)
    return dict(ms_event=ev, distinct_experts=u, bytes_step=L.active_bytes(u) + n_tokens * 2 * H * 4, flops=flops)


def attn_workload(qk, n_slots, ctx, steps, warmup, tmax=4096, seed=5):
    """The full-attention decode step (prep + attention) of n_slots slots at position ctx - 1: the
    reference's head shape (16 query heads of 256 on 2 KV heads, 64 rotated dims), fp32 caches of
    tmax positions.  A ring of distinct cache sets (> 1 GB in all) stands for the attention layers
    of a model, so no step finds its keys in a cache.  Bytes: the K and V rows of the ctx positions."""
    import numpy as np
    import torch
    dev = "cuda:0"
    hQ, hKV, dh, n_rot = 16, 2, 256, 64
    per_set = 2 * n_slots * hKV * tmax * dh * 4
    ring = max(2, min(64, (1 << 30) // per_set + 1))
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    kc = [torch.randn((n_slots, hKV, tmax, dh), device=dev, generator=g) for _ in range(ring)]
    vc = [torch.randn((n_slots, hKV, tmax, dh), device=dev, generator=g) for _ in range(ring)]
    qfull = torch.randn((ring, n_slots, hQ, 2 * dh), device=dev, generator=g)
    kin = torch.randn((ring, n_slots, hKV, dh), device=dev, generator=g)
    vin = torch.randn((ring, n_slots, hKV, dh), device=dev, generator=g)
    w = torch.ones(dh, device=dev)
    rope = torch.from_numpy(qk.rope_table(tmax, n_rot)).to(dev)
    pos = torch.full((n_slots,), ctx - 1, dtype=torch.int32, device=dev)
    qhat = torch.empty((ring, n_slots, hQ, dh), device=dev)
    att = torch.empty((ring, n_slots, hQ, dh), device=dev)
    ws = torch.empty(qk.attn_workspace_bytes(n_slots, hQ), dtype=torch.uint8, device=dev)

    def step(i):
        def f():
            qk.attn_prep(qfull[i], kin[i], vin[i], w, w, rope, pos, kc[i], vc[i], n_rot, qhat=qhat[i])
            qk.attn_decode(qhat[i], kc[i], vc[i], qfull[i], pos, ws, att=att[i])
        return f
    wall, ev, n = run_ring([step(i) for i in range(ring)], steps // ring * ring, warmup)
    return dict(ms_event=ev, steps=n, ring=ring, bytes_step=2 * n_slots * hKV * ctx * dh * 4)


def attn_prefill_workload(qk, n_pos, steps, warmup, tmax=4096, seed=8):
    """The full-attention mixer over n_pos consecutive positions of one slot from an empty cache (prep +
    causal attention, the prefill form): 16 query heads of 256 on 2 KV heads.  Flops: QK^T and PV over the
    causal triangle, 2 * 2 * hQ * dh * n_pos * (n_pos + 1) / 2."""
    import torch
    dev = "cuda:0"
    hQ, hKV, dh, n_rot, ring = 16, 2, 256, 64, 4
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    kc = [torch.zeros((1, hKV, tmax, dh), device=dev) for _ in range(ring)]
    vc = [torch.zeros((1, hKV, tmax, dh), device=dev) for _ in range(ring)]
    qfull = torch.randn((ring, n_pos, hQ, 2 * dh), device=dev, generator=g)
    kin = torch.randn((ring, n_pos, hKV, dh), device=dev, generator=g)
    vin = torch.randn((ring, n_pos, hKV, dh), device=dev, generator=g)
    w = torch.ones(dh, device=dev)
    rope = torch.from_numpy(qk.rope_table(tmax, n_rot)).to(dev)
    pos = torch.arange(n_pos, dtype=torch.int32, device=dev)
    qhat = torch.empty((ring, n_pos, hQ, dh), device=dev)
    att = torch.empty((ring, n_pos, hQ, dh), device=dev)
    ws = torch.empty(qk.attn_workspace_bytes(n_pos, hQ), dtype=torch.uint8, device=dev)

    def step(i):
        def f():
            qk.attn_prep(qfull[i], kin[i], vin[i], w, w, rope, pos, kc[i], vc[i], n_rot, qhat=qhat[i], seq=True)
            qk.attn_decode(qhat[i], kc[i], vc[i], qfull[i], pos, ws, att=att[i], seq=True)
        return f
    wall, ev, n = run_ring([step(i) for i in range(ring)], steps // ring * ring, warmup)
    return dict(ms_event=ev, steps=n, ring=ring, flops=2.0 * 2 * hQ * dh * n_pos * (n_pos + 1) / 2)


def deltanet_workload(qk, n_slots, steps, warmup, seed=6):
    """The gated-DeltaNet decode step (decay/beta dots, conv, state update + gated norm) of n_slots
    slots at the reference's shape (32 value heads on 16 key heads, state 128 x 128 per head).  A
    ring of distinct state sets (> 1 GB in all) stands for the DeltaNet layers of a model.  Bytes:
    the states, read and written (2 * 32 * 128 * 128 * 4 B each way per slot)."""
    import torch
    dev = "cuda:0"
    hK, hV, dS, ne = 16, 32, 128, 2048
    ch, qkc = (2 * hK + hV) * dS, 2 * hK * dS
    per_set = n_slots * hV * dS * dS * 4
    ring = max(2, min(128, (1 << 30) // per_set + 1))
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    S = [torch.randn((n_slots, hV, dS, dS), device=dev, generator=g) * 0.1 for _ in range(ring)]
    st = [torch.randn((n_slots, ch, 3), device=dev, generator=g) for _ in range(ring)]
    x = torch.randn((ring, n_slots, ne), device=dev, generator=g)
    qkv = torch.randn((ring, n_slots, ch), device=dev, generator=g)
    z = torch.randn((ring, n_slots, hV * dS), device=dev, generator=g)
    aw, bw = (torch.randn((hV, ne), device=dev, generator=g) * 0.03 for _ in range(2))
    dt = torch.randn(hV, device=dev, generator=g)
    av = -torch.rand(hV, device=dev, generator=g) - 0.05
    ker = torch.randn((ch, 4), device=dev, generator=g) * 0.5
    nw = torch.ones(dS, device=dev)
    gb = torch.empty((ring, n_slots, 2 * hV), device=dev)
    conv = torch.empty((ring, n_slots, ch), device=dev)
    att = torch.empty((ring, n_slots, hV * dS), device=dev)

    def step(i):
        def f():
            qk.dn_ab(x[i], aw, bw, dt, av, gb=gb[i])
            qk.dn_conv(st[i], qkv[i], ker, qkc, out=conv[i])
            qk.dn_step(conv[i], gb[i], S[i], nw, z[i], hK, hV, att=att[i])
        return f
    wall, ev, n = run_ring([step(i) for i in range(ring)], max(ring, steps // ring * ring), warmup)
    return dict(ms_event=ev, steps=n, ring=ring, bytes_step=2 * n_slots * hV * dS * dS * 4)


def engine_workload(qk, n_layer, slots_list, chunks, warm_chunks, seed=31, kinds=None, prefill_only=0):
    """Tokens per second through the engine ABI (qk_open / qk_slot_start / qk_step_chunk) on a
    synthetic model file at the full layer shape and vocabulary: host wall clock over whole chunks,
    host synchronisation after every step included.  kinds = None: MoE-only layers; else one letter
    per layer, "R" gated DeltaNet or "A" full attention in front of each MoE block (a whole model).
    prefill_only = P: no decode steps, P positions through qk_stage_run four times instead.
    Two distinct layers' MoE weights alternate through the file; each layer has its own copy in
    device memory."""
    import shutil
    import tempfile
    if kinds is None:
        model = qk.engine.StackModel(seed, n_layer=2, vocab=151936, n_expert=256, n_ff=512, n_used=8,
                                     down_types=[qk.IQ4_XS, qk.Q6_K], eos=151935)
        model.layers = [model.layers[l % 2] for l in range(n_layer)]
        model.post_norm = [model.post_norm[l % 2] for l in range(n_layer)]
    else:
        model = qk.engine.FullModel(seed, kinds=kinds, vocab=151936, n_expert=256, n_ff=512, n_used=8, eos=151935,
                                    distinct_moe=2)
    tmp = tempfile.mkdtemp(prefix="qk_bench_")
    res = {}
    try:
        path = model.write(os.path.join(tmp, "model.gguf"))
        del model
        for n_slots in slots_list:
            t0 = time.perf_counter()
            with qk.engine.Engine(path, n_slots=n_slots, n_ctx=4096, chunk=32) as eng:
                t_open = time.perf_counter() - t0

                def run(n_chunks):
                    toks = 0
                    for _ in range(n_chunks):
                        for s in range(n_slots):   # a finished slot (EOS or max_gen) takes the next request
                            eng.slot_start(s, [100 + s], 4000)
                        rc, out, _ = eng.step_chunk()
                        if rc < 0:
                            sys.exit(f"bench.py: qk_step_chunk returned {rc}")
                        toks += sum(len(v) for v in out.values())
                    return toks
                if not prefill_only:
                    run(warm_chunks)
                t0 = time.perf_counter()
                toks = 0 if prefill_only else run(chunks)
                dt = time.perf_counter() - t0
                pre = {}
                if kinds is not None and n_slots == slots_list[0]:
                    # prompt positions per second: qk_stage_run over 512 positions of one slot, twice
                    # (the first pass warms the prefill path's launch set-up)
                    ptoks = [(7 * i + 3) % 151000 for i in range(prefill_only or 512)]
                    for _ in range(4 if prefill_only else 2):
                        tp = time.perf_counter()
                        rcp, _ids = eng.stage_run(0, ptoks, 0)
                        tp = time.perf_counter() - tp
                        if rcp != 0:
                            sys.exit(f"bench.py: qk_stage_run returned {rcp}")
                    pre = dict(prefill_tok_per_s=len(ptoks) / tp, prefill_positions=len(ptoks))
                    # the serving path: qk_slot_start prefills all but the last prompt token (no LM head there)
                    for s in range(n_slots):
                        eng.slot_cancel(s)
                    for _ in range(2):
                        tp = time.perf_counter()
                        rcs = eng.slot_start(0, ptoks + [5], 8)
                        tp = time.perf_counter() - tp
                        eng.slot_cancel(0)
                        if rcs != 0:
                            sys.exit(f"bench.py: qk_slot_start returned {rcs}")
                    pre["slot_start_prefill_tok_per_s"] = len(ptoks) / tp
            res[f"slots_{n_slots}"] = dict(tok_per_s=toks / dt, us_per_step=dt / (max(chunks, 1) * 32) * 1e6, tokens=toks,
                                           open_s=t_open, **pre)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    res["config"] = dict(n_layer=n_layer, vocab=151936, chunk=32, mixers=kinds or "none",
                         layer="256 experts, IQ3_XXS gate/up, IQ4_XS / Q6_K down alternating, Q8_0 shared")
    return res


def guarded(ex, key, fn, quiet=False):
    """Runs one extra measurement; a Python-level failure becomes an entry of the line instead of ending the run
    (the headline figure is already measured by then)."""
    try:
        ex[key] = fn()
    except Exception as e:   # noqa: BLE001 -- whatever it is, the line still goes out
        ex[key] = dict(error=f"{type(e).__name__}: {e}")
    if not quiet or "error" in ex[key]:
        log(f"[bench] {key}: {ex[key]}")


def host_threads():
    """Threads of the all-cores CPU runs: the cores this process may use, at most 16 (a one-GPU box's share)."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    return max(1, min(16, n))


def _timed(fn, reps):
    fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


def cpu_baseline(qk, orc):
    """The reference's scalar CPU path restated (oracle: dequantise a row, dot in double,
    src/main.cpp:673-679; moeCpuRef, src/main.cpp:1316-1387) timed on this host: one thread, as the
    reference runs it, and all host threads (rows or tokens split), per BASELINE config, on bounded
    samples of each workload.  `value` is the headline config (one fused MoE decode step, bs=1)."""
    import numpy as np
    nt = host_threads()
    per = {}
    rng = np.random.default_rng(5)

    def entry_(us1, usN, nbytes, sample):
        return dict(us_1_thread=us1, us_all_threads=usN, threads=nt, gbps_1_thread=nbytes / us1 / 1e3,
                    gbps_all_threads=nbytes / usN / 1e3, bytes=nbytes, sample=sample)

    # C1: one GEMV 8192 x 2048 per format (a quarter of the rows timed, scaled: rows are independent)
    M, K, part = 8192, 2048, 2048
    x = rng.standard_normal(K).astype(np.float32)
    for name, t in (("q8_0", orc.Q8_0), ("q6_k", orc.Q6_K), ("iq4_xs", orc.IQ4_XS), ("iq3_xxs", orc.IQ3_XXS)):
        W = qk.synth.tensor_host(t, part, K, seed=42)
        t1 = _timed(lambda: orc.gemv(t, W, x, part, K), 3) * (M / part)
        tn = _timed(lambda: orc.gemv(t, W, x, part, K, threads=nt), 5) * (M / part)
        per[f"C1_gemv_{name}_8192x2048"] = entry_(t1 * 1e6, tn * 1e6, M * orc.row_bytes(t, K) + (K + M) * 4,
                                                  f"{part} of {M} rows timed, scaled")
    # C2: the fused MoE decode step, one row
    hl = qk.synth.HostLayer(seed=4321)
    xs = rng.standard_normal((16, 2048)).astype(np.float32)
    it = [0]

    def step1():
        it[0] += 1
        orc.moe_ref(hl, xs[it[0] % 16])

    def stepn():
        it[0] += 1
        orc.moe_ref_threads(hl, xs[it[0] % 16][None, :], nt)
    t1, tn = _timed(step1, 5), _timed(stepn, 9)
    layer_bytes = 256 * 2048 * 4 + 2048 * 4 + 8 * (2 * 512 * 784 + 2048 * 272) + 2 * 512 * 2176 + 2048 * 544
    per["C2_moe_decode_bs1"] = entry_(t1 * 1e6, tn * 1e6, layer_bytes, "whole steps, a fresh activation row per step")
    c2 = per["C2_moe_decode_bs1"]
    # C3: the same step for 16 slots, Q6_K down (tokens split over the threads; one thread: 2 slots timed, scaled)
    hl6 = qk.synth.HostLayer(seed=4322, down_type=qk.Q6_K)
    t1 = _timed(lambda: orc.moe_ref_threads(hl6, xs[:2], 1), 1) * 8
    tn = _timed(lambda: orc.moe_ref_threads(hl6, xs, nt), 3)
    per["C3_moe_decode_bs16_q6k_down"] = entry_(t1 * 1e6, tn * 1e6, 0, "16 slots; one thread: 2 slots timed, scaled; "
                                                "the CPU path re-reads the weights per slot, so no byte rate is given")
    for k_ in ("gbps_1_thread", "gbps_all_threads"):
        per["C3_moe_decode_bs16_q6k_down"][k_] = None
    # C4: the LM head (Q6_K, 151,936 x 2048) + argmax: 1/16 of the vocabulary timed, scaled
    V, Vs = 151936, 9496
    Wh = qk.synth.tensor_host(qk.Q6_K, Vs, K, seed=77)
    t1 = _timed(lambda: orc.argmax(orc.gemv(orc.Q6_K, Wh, x, Vs, K)), 2) * (V / Vs)
    tn = _timed(lambda: orc.argmax(orc.gemv(orc.Q6_K, Wh, x, Vs, K, threads=nt)), 3) * (V / Vs)
    per["C4_lm_head_q6k_151936_bs1"] = entry_(t1 * 1e6, tn * 1e6, V * orc.row_bytes(orc.Q6_K, K) + K * 4,
                                              f"{Vs} of {V} rows timed, scaled")
    # C5a: the Q8_0 GEMM 8192 x 2048 x 128 tokens (1/8 of the weight rows timed, scaled)
    Wg = qk.synth.tensor_host(qk.Q8_0, 1024, K, seed=55)
    Xg = rng.standard_normal((128, K)).astype(np.float32)
    t1 = _timed(lambda: orc.gemm_q8_0(Wg, Xg, 1024, K), 1) * 8
    tn = _timed(lambda: orc.gemm_q8_0(Wg, Xg, 1024, K, threads=nt), 3) * 8
    per["C5a_gemm_q8_0_8192x2048x128"] = dict(entry_(t1 * 1e6, tn * 1e6, 8192 * 2176 + 128 * (K + 8192) * 4,
                                                     "1024 of 8192 weight rows timed, scaled"),
                                              gflops_1_thread=2.0 * 8192 * K * 128 / t1 / 1e9,
                                              gflops_all_threads=2.0 * 8192 * K * 128 / tn / 1e9)
    # C5b: the MoE block for 128 tokens (tokens split; one thread: 2 tokens timed, scaled)
    X128 = rng.standard_normal((128, 2048)).astype(np.float32)
    t1 = _timed(lambda: orc.moe_ref_threads(hl, X128[:2], 1), 1) * 64
    tn = _timed(lambda: orc.moe_ref_threads(hl, X128[:4 * nt], nt), 1) * (128 / (4 * nt))
    per["C5b_moe_prefill_128_tokens"] = dict(us_1_thread=t1 * 1e6, us_all_threads=tn * 1e6, threads=nt,
                                             tok_per_s_1_thread=128 / t1, tok_per_s_all_threads=128 / tn,
                                             sample=f"one thread: 2 tokens timed, scaled; all threads: {4 * nt} tokens timed, scaled")
    return dict(value=c2["gbps_all_threads"], unit="GB/s", cores=nt, kind="port",
                sample=f"fused MoE decode step (bs=1, one synthetic layer, a fresh activation row per step), oracle moeCpuRef "
                       f"restatement with its row loops split over {nt} host threads: {c2['us_all_threads']:.0f} us/step "
                       f"({c2['us_1_thread']:.0f} us/step on one thread, as the reference runs it)",
                us_per_step=c2["us_all_threads"],
                one_thread=dict(value=c2["gbps_1_thread"], unit="GB/s", cores=1, us_per_step=c2["us_1_thread"]),
                host_cpus=os.cpu_count(), per_config=per)


def qk_env():
    """The library's environment switches that were set for this run (they change which kernels run)."""
    return {k: v for k, v in os.environ.items() if k.startswith("QK_")}


def kernel_forms(qk):
    """The library's switches as they stand (which form of each kernel the figures belong to)."""
    return {n: qk.get_option(n) for n in ("one_row", "dense_reg", "fused_norm", "attn_block", "dn_fused", "gemm_tiled", "moe_rows", "head_rows", "select_ranked")}


def rate(bytes_step, ms, **more):
    gb = bytes_step / (ms * 1e-3) / 1e9
    return dict(us=ms * 1e3, gbps=gb, frac=gb / HBM_PEAK_GBPS, **more)


def gemv_entry(qk, t, M, K, batch, steps, warmup):
    """One GEMV figure; M = None: a sustained size (one tensor of at least 256 MiB per launch, two tensors
    alternating, so neither launch latency nor the caches carry the figure)."""
    if M is None:
        M = -(-(256 << 20) // qk.row_bytes(t, K) // 64) * 64
        g = gemv_workload(qk, t, M, K, batch, steps, warmup, ring=2)
    else:
        g = gemv_workload(qk, t, M, K, batch, steps, warmup)
    return rate(g["bytes_step"], g["ms_event"], rows=M, steps_timed=g["steps"])


def gemm_entry(qk):
    g = gemm_workload(qk, 8192, 2048, 128, 200, 20)
    tf = g["flops"] / (g["ms_event"] * 1e-3) / 1e12
    return dict(us=g["ms_event"] * 1e3, tflops=tf, frac_mfma_peak=tf / MFMA_F16_PEAK_TFLOPS,
                gbps=g["bytes_step"] / (g["ms_event"] * 1e-3) / 1e9,
                frac_hbm_peak=g["bytes_step"] / (g["ms_event"] * 1e-3) / 1e9 / HBM_PEAK_GBPS)


def extras(qk, a, steps):
    """The other BASELINE configs (C1 GEMVs, C3 16-slot step, C4 head, C5 prefill) and the rows beside the
    path (glue, mixers, engine), each as an entry of its own; a failing one becomes an error entry."""
    import torch
    ex = {}
    es, ew = 400, 40
    fmts = (("q8_0", qk.Q8_0), ("q6_k", qk.Q6_K), ("iq4_xs", qk.IQ4_XS), ("iq3_xxs", qk.IQ3_XXS), ("f16", qk.F16))

    t_start = time.perf_counter()

    def run(key, fn):
        # the BASELINE configs come first; whatever is left when the budget is spent is named, not run
        if time.perf_counter() - t_start > a.extras_seconds:
            ex[key] = dict(skipped=f"the extras' time budget of {a.extras_seconds} s was spent (--extras-seconds)")
            return
        guarded(ex, key, fn)
        torch.cuda.empty_cache()

    for name, t in fmts:   # C1 and its four sisters, one slot and sixteen (weights read once)
        run(f"gemv_{name}_8192x2048", lambda t=t: gemv_entry(qk, t, 8192, 2048, 1, es, ew))
        if t != qk.F16:
            run(f"gemv_{name}_8192x2048_bs16", lambda t=t: gemv_entry(qk, t, 8192, 2048, 16, es, ew))
    for name, t in fmts:
        run(f"gemv_{name}_sustained_256MiB", lambda t=t: gemv_entry(qk, t, None, 2048, 1, 40, 4))
    def head(b):
        h = head_workload(qk, 151936, 2048, b, 40, 8)
        return rate(h["bytes_step"], h["ms_event"], steps_timed=h["steps"])
    for b in (1, 16):   # C4
        run(f"head_q6k_151936_bs{b}", lambda b=b: head(b))

    def stages(m, **more):
        return dict(us=m["ms_event"] * 1e3, steps_timed=m["steps"], stage_us={k: v * 1e3 for k, v in m["stage_ms"].items()}, **more)

    def moe16():   # C3
        m16 = moe_workload(qk, 16, qk.Q6_K, 4, 200, 20)
        r = rate(m16["bytes_step"], m16["ms_event"], distinct_experts=m16["distinct_experts"])
        r["stage_us"] = {k: v * 1e3 for k, v in m16["stage_ms"].items()}
        return r
    run("moe_decode_bs16_q6k_down", moe16)
    run("prefill_gemm_q8_0_8192x2048x128", lambda: gemm_entry(qk))   # C5a

    def prefill_moe():   # C5b
        pm = prefill_moe_workload(qk, 128, 20, 4)
        tf = pm["flops"] / (pm["ms_event"] * 1e-3) / 1e12
        return rate(pm["bytes_step"], pm["ms_event"], tok_per_s=128 / (pm["ms_event"] * 1e-3),
                    distinct_experts=pm["distinct_experts"], tflops=tf, frac_mfma_peak=tf / MFMA_F16_PEAK_TFLOPS)
    run("prefill_moe_128_tokens", prefill_moe)
    # the same step on ONE layer replayed: its 16 MB stay in the caches, so this is the step without
    # HBM in the way (launch, selection and dependency chain) beside the ring's figure
    run("moe_decode_bs1_cache_hot", lambda: stages(moe_workload(qk, 1, qk.IQ4_XS, 1, 400, 40)))
    # the ring's tensors carved from one allocation: what the many separate mappings cost, if anything
    run("moe_decode_bs1_ring_in_one_allocation",
        lambda: stages(moe_workload(qk, 1, qk.IQ4_XS, a.ring, min(steps, 800), a.warmup, slab=True)))
    # the other dense projections of a decode step at the reference's shapes (src/main.cpp:4310-4335)
    for M, K in ((4096, 2048), (2048, 4096), (512, 2048)):
        for b in (1, 16):
            run(f"gemv_q8_0_{M}x{K}" + ("_bs16" if b > 1 else ""), lambda M=M, K=K, b=b: gemv_entry(qk, qk.Q8_0, M, K, b, es, ew))
    # a few concurrent slots: every row through the one-row launches (grid.y = row)
    for nr in (2, 4, 8):
        run(f"moe_decode_{nr}_rows_q6k_down", lambda nr=nr: dict(us=moe_workload(qk, nr, qk.Q6_K, 8, 400, 40)["ms_event"] * 1e3))
    # layer glue (add + RMS norm alone, and behind the step in one call)
    run("add_rmsnorm_2048", lambda: dict(us_1_row=norm_workload(qk, 1, 640, 64), us_16_rows=norm_workload(qk, 16, 640, 64)))
    run("moe_decode_tail_bs1", lambda: dict(us=moe_tail_workload(qk, 1, qk.IQ4_XS, 8, 400, 40)))
    run("moe_layer_row_bs1", lambda: dict(us=moe_tail_workload(qk, 1, qk.IQ4_XS, 8, 400, 40, layer_row=True)))
    run("moe_decode_tail_bs16_q6k_down", lambda: dict(us=moe_tail_workload(qk, 16, qk.Q6_K, 4, 200, 20)))
    for b in (1, 16):   # the full-attention mixer's decode step at 4096 cached positions
        def attn(b=b):
            at = attn_workload(qk, b, 4096, 200, 20)
            return rate(at["bytes_step"], at["ms_event"], ring=at["ring"])
        run(f"attn_decode_ctx4096_bs{b}", attn)

    def attn_prefill():   # the attention mixer over a 1,024-position prompt
        p = attn_prefill_workload(qk, 1024, 40, 8)
        return dict(us=p["ms_event"] * 1e3, tflops=p["flops"] / (p["ms_event"] * 1e-3) / 1e12, steps_timed=p["steps"])
    run("attn_prefill_1024_positions", attn_prefill)
    for b in (1, 16):   # the gated-DeltaNet mixer's decode step
        def dn(b=b):
            d = deltanet_workload(qk, b, 256, 32)
            return rate(d["bytes_step"], d["ms_event"], ring=d["ring"])
        run(f"deltanet_decode_bs{b}", dn)
    if a.ab_forms:
        # both forms of the one-row kernels side by side: block fields loaded per lane (the default) against rows
        # streamed through LDS; the C1 shapes, the sustained size, the head and the bs = 1 step with its stages
        for form, on in (("lane", 0), ("stream", 1)):
            with qk.option("one_row", on), qk.option("dense_reg", on):
                for name, t in fmts:
                    run(f"{form}:gemv_{name}_8192x2048", lambda t=t: gemv_entry(qk, t, 8192, 2048, 1, es, ew))
                    run(f"{form}:gemv_{name}_sustained_256MiB", lambda t=t: gemv_entry(qk, t, None, 2048, 1, 40, 4))
                run(f"{form}:head_q6k_151936_bs1", lambda: head(1))
                run(f"{form}:moe_decode_bs1", lambda: stages(moe_workload(qk, 1, qk.IQ4_XS, a.ring, min(steps, 800), a.warmup)))
                run(f"{form}:moe_decode_bs1_cache_hot", lambda: stages(moe_workload(qk, 1, qk.IQ4_XS, 1, 400, 40)))
                run(f"{form}:moe_decode_4_rows_q6k_down", lambda: dict(us=moe_workload(qk, 4, qk.Q6_K, 8, 400, 40)["ms_event"] * 1e3))
    if a.ab_forms:   # the prefill product with every weight tile decoded once per 128 rows, beside the default above
        with qk.option("gemm_tiled", 1):
            run("gemm_tiled:prefill_gemm_q8_0_8192x2048x128", lambda: gemm_entry(qk))
        with qk.option("moe_rows", 1):   # the routed experts with the waves splitting the weight rows, beside C3 and C5b above
            run("moe_rows:moe_decode_bs16_q6k_down", moe16)
            run("moe_rows:prefill_moe_128_tokens", prefill_moe)
        with qk.option("head_rows", 1):  # the 16-row head with the waves splitting the vocabulary rows, beside C4 above
            run("head_rows:head_q6k_151936_bs16", lambda: head(16))
    run("engine_decode_8_layers", lambda: engine_workload(qk, 8, (1, 4, 16), 8, 2))
    # a whole model: three gated-DeltaNet layers and one full-attention layer, twice (positions 1..320)
    run("engine_decode_whole_model_8_layers", lambda: engine_workload(qk, 8, (1, 16), 8, 2, kinds="RRRARRRA"))
    return ex


def run_child(argv, timeout_s):
    """Runs this file with `argv` as a child process and returns the object of its JSON line (its stderr
    is this process's)."""
    import subprocess
    r = subprocess.run([sys.executable, os.path.abspath(__file__)] + argv, stdout=subprocess.PIPE, text=True, timeout=timeout_s)
    if r.returncode != 0:
        raise RuntimeError(f"`bench.py {' '.join(argv)}` ended with status {r.returncode}")
    return json.loads(r.stdout.strip().splitlines()[-1])


def headline_and_extras(a):
    """The default run as three parts: the headline workload in a child process, the side measurements in
    a second one, the CPU baseline here.  This process never touches the GPU, so starting the children is
    an ordinary process start, and whatever happens to a side measurement -- a Python error is an entry
    of `extras`, a child that dies or stalls an error for the whole object -- the headline line goes out."""
    common = ["--ring", str(a.ring), "--steps", str(a.steps), "--warmup", str(a.warmup)]
    try:
        out = run_child(["--workload", a.workload, "--no-extras", "--no-cpu"] + common, 900)
    except Exception as e:   # noqa: BLE001 -- no headline, no line
        sys.exit(f"bench.py: the headline workload did not complete: {type(e).__name__}: {e}")
    ex_args = ["--workload", "extras", "--no-cpu", "--extras-seconds", str(a.extras_seconds)] + common + (["--ab-forms"] if a.ab_forms else [])
    guarded(out, "extras", lambda: run_child(ex_args, a.extras_seconds + 600)["extras"], quiet=True)
    if a.cpu:
        guarded(out, "cpu_baseline", lambda: cpu_baseline(entry.load_package(), entry.load_oracle()))
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="moe_decode_bs1")
    ap.add_argument("--ring", type=int, default=40)
    ap.add_argument("--prefill-rows", dest="maxb", type=int, default=0,
                    help="engine workloads: positions per prefill pass (sets QK_PREFILL_ROWS, 16..1024; default the engine's 1024)")
    ap.add_argument("--layers", type=int, default=8,
                    help="layers of the synthetic model of the engine workloads (40 = the reference model's depth, a 16 GB file)")
    ap.add_argument("--extras", dest="extras", action="store_true", default=True)
    ap.add_argument("--no-extras", dest="extras", action="store_false")
    ap.add_argument("--extras-seconds", type=float, default=240.0,
                    help="time budget of the side measurements; entries not reached are listed as skipped")
    ap.add_argument("--ab-forms", action="store_true",
                    help="extras: also time the one-row kernels in both forms (per-lane loads / rows streamed through LDS)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 256 MiB device copy (calibrates FETCH_SIZE/WRITE_SIZE counter runs)")
    ap.add_argument("--cpu", dest="cpu", action="store_true", default=True)
    ap.add_argument("--no-cpu", dest="cpu", action="store_false")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build drives ONE GPU (one process, one device); "
                 "--gpus N with N > 1 is not supported")
    if a.workload == "moe_decode_bs1" and a.extras:
        return headline_and_extras(a)
    import torch
    qk = entry.load_package()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device; libqk.so has no CPU path")
    qk.lib()
    info = qk.device_info()
    log(f"[bench] device {info}")

    if a.copy_probe:
        src = torch.full((64 << 20,), 1.0, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # 256 MiB read + 256 MiB written: the counters' yardstick
        torch.cuda.synchronize()
        del src, dst
    steps = max(a.ring, a.steps // a.ring * a.ring)
    if a.workload == "engine_whole_model":   # the engine ABI on a whole model (mixers + MoE blocks)
        r = engine_workload(qk, a.layers, (1, 16), 8, 2, kinds=("RRRA" * ((a.layers + 3) // 4))[:a.layers])
        print(json.dumps(dict(metric="engine_decode_tok_per_s", value=r["slots_16"]["tok_per_s"], unit="tok/s", n_gpus=1,
                              higher_is_better=True, data="synthetic", dtype="f32",
                              config=dict(workload="engine_whole_model", **r["config"]), detail=r)), flush=True)
        return
    if a.maxb:
        os.environ["QK_PREFILL_ROWS"] = str(a.maxb)
    if a.workload == "engine_prefill":   # prompt positions through qk_stage_run on a whole model
        r = engine_workload(qk, a.layers, (1,), 0, 0, kinds=("RRRA" * ((a.layers + 3) // 4))[:a.layers], prefill_only=1024)
        print(json.dumps(dict(metric="engine_prefill_tok_per_s", value=r["slots_1"]["prefill_tok_per_s"], unit="tok/s",
                              n_gpus=1, higher_is_better=True, data="synthetic", dtype="f32",
                              config=dict(workload="engine_prefill", positions=1024, positions_per_pass=a.maxb or 1024,
                                          **r["config"]), detail=r)), flush=True)
        return
    if a.workload == "engine_decode":   # the engine ABI alone (for kernel traces of its graph replays)
        r = engine_workload(qk, 8, (1, 4, 16), 8, 2)
        print(json.dumps(dict(metric="engine_decode_tok_per_s", value=r["slots_16"]["tok_per_s"], unit="tok/s", n_gpus=1,
                              higher_is_better=True, data="synthetic", dtype="f32",
                              config=dict(workload="engine_decode", **r["config"]), detail=r)), flush=True)
        return
    if a.workload in ("deltanet_bs1", "deltanet_bs16"):   # the gated-DeltaNet decode step alone
        b = 1 if a.workload == "deltanet_bs1" else 16
        dn = deltanet_workload(qk, b, min(a.steps, 512), min(a.warmup, 64))
        gb = dn["bytes_step"] / (dn["ms_event"] * 1e-3) / 1e9
        print(json.dumps(dict(metric="deltanet_decode_hbm_gbps", value=gb, unit="GB/s", n_gpus=1, steps=dn["steps"],
                              ms_per_step=dn["ms_event"], higher_is_better=True, data="synthetic", dtype="f32",
                              config=dict(workload=a.workload, slots=b, heads="32 value heads on 16 key heads, state 128 x 128",
                                          ring=dn["ring"]),
                              bytes_per_step=dn["bytes_step"], frac_of_hbm_peak=gb / HBM_PEAK_GBPS)), flush=True)
        return
    if a.workload in ("attn_bs1", "attn_bs16"):   # the attention decode step alone
        b = 1 if a.workload == "attn_bs1" else 16
        at = attn_workload(qk, b, 4096, min(a.steps, 400), min(a.warmup, 40))
        gb = at["bytes_step"] / (at["ms_event"] * 1e-3) / 1e9
        print(json.dumps(dict(metric="attn_decode_hbm_gbps", value=gb, unit="GB/s", n_gpus=1, steps=at["steps"],
                              ms_per_step=at["ms_event"], higher_is_better=True, data="synthetic", dtype="f32",
                              config=dict(workload=a.workload, slots=b, positions=4096, heads="16 x 256 on 2 KV heads",
                                          ring=at["ring"]),
                              bytes_per_step=at["bytes_step"], frac_of_hbm_peak=gb / HBM_PEAK_GBPS)), flush=True)
        return
    if a.workload == "gemv_sustained":   # every block format at a sustained size and at the 8192 x 2048 shape
        res = {}
        for name, t in (("q8_0", qk.Q8_0), ("q6_k", qk.Q6_K), ("iq4_xs", qk.IQ4_XS), ("iq3_xxs", qk.IQ3_XXS), ("f16", qk.F16)):
            guarded(res, f"gemv_{name}_sustained_256MiB", lambda t=t: gemv_entry(qk, t, None, 2048, 1, 40, 4))
            torch.cuda.empty_cache()
            guarded(res, f"gemv_{name}_8192x2048", lambda t=t: gemv_entry(qk, t, 8192, 2048, 1, 400, 40))
            torch.cuda.empty_cache()
        first = res["gemv_q8_0_sustained_256MiB"]
        print(json.dumps(dict(metric="gemv_hbm_gbps", value=first.get("gbps"), unit="GB/s", n_gpus=1,
                              higher_is_better=True, data="synthetic", dtype="f32",
                              config=dict(workload="gemv_sustained", K=2048, env=qk_env()),
                              detail=res)), flush=True)
        return
    if a.workload in ("head_bs1", "head_bs16"):   # the LM head alone (for counter runs on its kernel)
        b = 1 if a.workload == "head_bs1" else 16
        h = head_workload(qk, 151936, 2048, b, min(a.steps, 40), min(a.warmup, 8))
        gb = h["bytes_step"] / (h["ms_event"] * 1e-3) / 1e9
        print(json.dumps(dict(metric="lm_head_argmax_hbm_gbps", value=gb, unit="GB/s", n_gpus=1, steps=h["steps"],
                              ms_per_step=h["ms_event"], higher_is_better=True, data="synthetic", dtype="f32",
                              config=dict(workload=a.workload, vocab=151936, n_embd=2048, weights="Q6_K", rows=b),
                              bytes_per_step=h["bytes_step"], frac_of_hbm_peak=gb / HBM_PEAK_GBPS)), flush=True)
        return
    if a.workload == "prefill_gemm":   # the Q8_0 prefill GEMM alone (for counter runs on its kernel)
        res = {}
        guarded(res, "prefill_gemm_q8_0_8192x2048x128", lambda: gemm_entry(qk))
        print(json.dumps(dict(metric="prefill_gemm_tflops", value=res["prefill_gemm_q8_0_8192x2048x128"].get("tflops"),
                              unit="TFLOP/s", n_gpus=1, higher_is_better=True, data="synthetic", dtype="f16",
                              config=dict(workload=a.workload, M=8192, K=2048, N=128, weights="Q8_0"), detail=res)), flush=True)
        return
    if a.workload == "extras":   # the other BASELINE configs and the rows beside the path, as one JSON object
        print(json.dumps(dict(extras=extras(qk, a, steps))), flush=True)
        return
    if a.workload == "moe_decode_bs1":
        m = moe_workload(qk, 1, qk.IQ4_XS, a.ring, steps, a.warmup)
    elif a.workload == "moe_decode_bs16":
        m = moe_workload(qk, 16, qk.Q6_K, min(a.ring, 8), steps, a.warmup)
    elif a.workload == "moe_prefill_128":
        m = moe_workload(qk, 128, qk.IQ4_XS, min(a.ring, 4), min(steps, 400), min(a.warmup, 40))
    else:
        sys.exit(f"unknown workload {a.workload}")
    log(f"[bench] {a.workload}: {m['ms_wall'] * 1e3:.2f} us/step wall, {m['ms_event'] * 1e3:.2f} us/step events, "
        f"stages {m['stage_ms']}")
    gbps = m["bytes_step"] / (m["ms_wall"] * 1e-3) / 1e9
    # dominant kernel = the routed gate/up launch (most bytes of the step); its average launch
    # duration is measured live with HIP events on the launch stream over a replay of that
    # stage alone on the same ring (profiles/ holds the rocprofv3 figure for the same kernel)
    gu_ms = m["stage_ms"]["gateup"]
    ach = m["gateup_bytes"] / (gu_ms * 1e-3) / 1e9
    kname, kwhat = {"moe_decode_bs1": ("moe_gateup_kernel", "select + routed IQ3_XXS gate/up + SiLU"),
                    "moe_decode_bs16": ("moe_gateup_fused_kernel", "routed IQ3_XXS + shared Q8_0 gate/up + SiLU"),
                    "moe_prefill_128": ("moe_gateup_mfma_kernel", "routed IQ3_XXS gate/up + SiLU; the stage time also "
                                        "covers the shared expert's launch on the side stream")}[a.workload]
    roof = dict(bound="hbm", kernel=f"{kname} ({kwhat})", achieved=ach,
                peak=HBM_PEAK_GBPS, unit="GB/s", frac=ach / HBM_PEAK_GBPS,
                # the counter run is of the per-lane form of the one-row kernel; the streamed form has none yet
                traffic=TRAFFIC.get(kname) if not (a.workload == "moe_decode_bs1" and qk.get_option("one_row")) else None,
                bytes_per_launch=m["gateup_bytes"], us_per_launch=gu_ms * 1e3)
    out = dict(metric="fused_moe_decode_step_hbm_gbps", value=gbps, unit="GB/s", n_gpus=1, steps=a.steps,
               warmup=a.warmup, ms_per_step=m["ms_wall"], higher_is_better=True, scaling="weak", vs_baseline=None,
               dtype="f32", data="synthetic",
               config=dict(workload=a.workload, n_embd=2048, n_ff=512, n_expert=256, n_used=8,
                           gate_up="IQ3_XXS", down="Q6_K" if a.workload.endswith("bs16") else "IQ4_XS",
                           shared="Q8_0", slots={"moe_decode_bs1": 1, "moe_decode_bs16": 16}.get(a.workload, 128),
                           ring_layers=m["ring"], ring_bytes=m["ring_bytes"],
                           steps_timed=m["steps"], graph_replays_timed=m["steps"] // m["ring"],
                           timing=f"hipGraph replays of the ring (one launch set per layer of the ring), at least "
                                  f"{MIN_REPLAYS} replays whatever --steps asks; value from the host clock over all of them, "
                                  f"us_per_step_events the median replay by HIP events", env=qk_env(), kernel_forms=kernel_forms(qk)),
               us_per_step=m["ms_wall"] * 1e3, us_per_step_events=m["ms_event"] * 1e3,
               bytes_per_step=m["bytes_step"], frac_of_hbm_peak=gbps / HBM_PEAK_GBPS,
               distinct_experts_per_step=m["distinct_experts"],
               three_launch_stage_us={k: v * 1e3 for k, v in m["stage_ms"].items()}, roofline=roof, device=info)
    del m
    torch.cuda.empty_cache()

    if a.cpu:
        guarded(out, "cpu_baseline", lambda: cpu_baseline(qk, entry.load_oracle()))
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
