"""The host side of bench.py: argument handling and the CPU-baseline leg (no GPU needed)."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and not r.stdout.strip()


def test_default_run_without_a_device_says_so():
    """The real process tree of the default run on a host without a GPU: the headline child reports the missing
    device, the parent ends with a message and prints no line (there is no CPU path to fall back on)."""
    import torch
    if torch.cuda.is_available():
        import pytest
        pytest.skip("a device is present")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "20", "--warmup", "5"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode != 0 and not r.stdout.strip()
    assert "no HIP device" in r.stderr and "headline workload did not complete" in r.stderr


def test_cpu_baseline_line(qk, orc):
    """Every BASELINE config has a one-thread and an all-threads figure, the thread count is stated and
    the headline entry is the fused MoE step; the object goes into the JSON line as it is."""
    sys.path.insert(0, ROOT)
    import bench
    b = bench.cpu_baseline(qk, orc)
    json.dumps(b)
    assert b["kind"] == "port" and b["unit"] == "GB/s" and 1 <= b["cores"] == bench.host_threads() <= 16
    assert b["one_thread"]["cores"] == 1 and 0 < b["one_thread"]["value"] <= b["value"] * 1.5
    per = b["per_config"]
    want = ["C1_gemv_q8_0_8192x2048", "C1_gemv_q6_k_8192x2048", "C1_gemv_iq4_xs_8192x2048", "C1_gemv_iq3_xxs_8192x2048",
            "C2_moe_decode_bs1", "C3_moe_decode_bs16_q6k_down", "C4_lm_head_q6k_151936_bs1", "C5a_gemm_q8_0_8192x2048x128",
            "C5b_moe_prefill_128_tokens"]
    assert sorted(per) == sorted(want)
    for name, e in per.items():
        assert e["us_1_thread"] > 0 and e["us_all_threads"] > 0 and e["threads"] == b["cores"] and e["sample"], name
    assert per["C2_moe_decode_bs1"]["bytes"] == 16326656      # the weights one step touches: router, shared gate, 8 experts, shared expert
    assert per["C1_gemv_q8_0_8192x2048"]["bytes"] == 17866752
    assert per["C4_lm_head_q6k_151936_bs1"]["bytes"] == 255252480 + 8192


def test_no_function_of_bench_reads_a_name_nothing_binds():
    """Every name a function of bench.py takes from the module's namespace exists there (or is a
    builtin): a block that lost the statement that bound its variables cannot come back unnoticed."""
    import builtins
    import symtable
    sys.path.insert(0, ROOT)
    import bench
    src = open(os.path.join(ROOT, "bench.py")).read()
    missing = []

    def walk(tab):
        for s in tab.get_symbols():
            if s.is_global() and s.is_referenced() and not hasattr(bench, s.get_name()) and not hasattr(builtins, s.get_name()):
                missing.append((tab.get_name(), s.get_name()))
        for c in tab.get_children():
            walk(c)
    walk(symtable.symtable(src, "bench.py", "exec"))
    assert not missing, missing


class _FakeCuda:
    @staticmethod
    def is_available():
        return True

    @staticmethod
    def empty_cache():
        pass


def _bench_with_stub_workloads(monkeypatch, qk):
    """bench with every GPU workload replaced by a stub of the same signature and result keys, so main()
    runs from the arguments to the JSON line on the CPU."""
    sys.path.insert(0, ROOT)
    import bench
    import torch
    monkeypatch.setattr(torch, "cuda", _FakeCuda)
    monkeypatch.setattr(qk, "lib", lambda: None)
    monkeypatch.setattr(qk, "device_info", lambda: dict(name="stub"))
    stage = dict(route=0.004, gateup=0.009, down=0.007)
    monkeypatch.setattr(bench, "moe_workload", lambda qk_, n, down, ring, steps, warmup, seed=1234, slab=False: dict(
        ms_wall=0.021, ms_event=0.0205, steps=max(20 * ring, steps), bytes_step=16343200, distinct_experts=8.0, stage_ms=dict(stage),
        gateup_bytes=6449152, ring=ring, ring_bytes=ring * 351000000))
    monkeypatch.setattr(bench, "moe_tail_workload", lambda *a, **k: 22.0)
    monkeypatch.setattr(bench, "norm_workload", lambda *a, **k: 2.1)
    monkeypatch.setattr(bench, "gemv_workload", lambda qk_, t, M, K, batch, steps, warmup, seed=99, ring=None: dict(
        ms_wall=0.007, ms_event=0.0068, steps=steps, bytes_step=M * qk.row_bytes(t, K) + batch * (K + M) * 4, ring=ring or 16))
    monkeypatch.setattr(bench, "head_workload", lambda qk_, V, K, batch, steps, warmup, seed=77: dict(
        ms_wall=0.06, ms_event=0.059, steps=steps, bytes_step=V * 1680 + batch * (K * 4 + 4), ring=2))
    monkeypatch.setattr(bench, "gemm_workload", lambda qk_, M, K, N, steps, warmup, seed=55: dict(
        ms_event=0.032, flops=2.0 * M * K * N, bytes_step=M * K // 32 * 34 + N * (K + M) * 4))
    monkeypatch.setattr(bench, "prefill_moe_workload", lambda qk_, n, steps, warmup, seed=4242: dict(
        ms_event=0.21, distinct_experts=251.0, bytes_step=342e6, flops=6.4e9))
    monkeypatch.setattr(bench, "attn_workload", lambda qk_, b, ctx, steps, warmup, **k: dict(ms_event=0.05, bytes_step=b * 16777216, ring=4))
    monkeypatch.setattr(bench, "attn_prefill_workload", lambda qk_, n, steps, warmup, **k: dict(ms_event=0.9, flops=1e12, steps=steps))
    monkeypatch.setattr(bench, "deltanet_workload", lambda qk_, b, steps, warmup, **k: dict(ms_event=0.02, bytes_step=b * 4194304, ring=8))
    monkeypatch.setattr(bench, "engine_workload", lambda *a, **k: dict(config=dict(layers=8), slots_1=dict(tok_per_s=1.0, prefill_tok_per_s=1.0),
                                                                      slots_16=dict(tok_per_s=2.0)))
    monkeypatch.setattr(bench, "cpu_baseline", lambda qk_, orc_: dict(value=0.5, unit="GB/s", cores=8, kind="port", sample="stub", per_config={}))
    # the default run starts a child process per part; here the parts run in this process, on the stubs
    def child(argv, timeout_s):
        import contextlib
        import io
        saved, buf = sys.argv, io.StringIO()
        sys.argv = ["bench.py"] + argv
        try:
            with contextlib.redirect_stdout(buf):
                bench.main()
        finally:
            sys.argv = saved
        return json.loads(buf.getvalue().strip().splitlines()[-1])
    monkeypatch.setattr(bench, "run_child", child)
    return bench


def _one_json_line(capsys):
    lines = [ln for ln in capsys.readouterr().out.splitlines() if ln.strip()]
    assert len(lines) == 1, lines
    return json.loads(lines[0])


def test_default_run_prints_the_headline_line(monkeypatch, capsys, qk):
    """The driver's command line, from the arguments to the one JSON line, on stub workloads: the keys the
    contract names, the roofline and CPU objects, and an entry per BASELINE config among the extras."""
    bench = _bench_with_stub_workloads(monkeypatch, qk)
    monkeypatch.setattr(sys, "argv", ["bench.py", "--gpus", "1", "--steps", "20", "--warmup", "5"])
    bench.main()
    out = _one_json_line(capsys)
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
              "dtype", "data", "config", "roofline", "cpu_baseline", "extras"):
        assert k in out, k
    assert out["steps"] == 20 and out["warmup"] == 5 and out["n_gpus"] == 1 and out["vs_baseline"] is None
    assert out["config"]["workload"] == "moe_decode_bs1" and out["config"]["steps_timed"] >= 20 * out["config"]["ring_layers"]
    r = out["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-12
    assert abs(r["achieved"] - r["bytes_per_launch"] / r["us_per_launch"] / 1e3) < 1e-6 * r["achieved"] and "traffic" in r
    assert out["cpu_baseline"]["kind"] == "port"
    ex = out["extras"]
    for k in ("gemv_q8_0_8192x2048", "gemv_q6_k_8192x2048", "gemv_iq4_xs_8192x2048", "gemv_iq3_xxs_8192x2048", "gemv_f16_8192x2048",
              "gemv_q8_0_sustained_256MiB", "gemv_iq3_xxs_sustained_256MiB", "head_q6k_151936_bs1", "head_q6k_151936_bs16",
              "moe_decode_bs16_q6k_down", "prefill_gemm_q8_0_8192x2048x128", "prefill_moe_128_tokens", "moe_decode_bs1_cache_hot",
              "moe_decode_bs1_ring_in_one_allocation"):
        assert k in ex and "error" not in ex[k], (k, ex.get(k))
    assert ex["gemv_q8_0_8192x2048"]["gbps"] > 0 and ex["prefill_gemm_q8_0_8192x2048x128"]["frac_mfma_peak"] > 0


def test_other_workloads_print_one_line_each(monkeypatch, capsys, qk):
    bench = _bench_with_stub_workloads(monkeypatch, qk)
    for wl, metric in (("gemv_sustained", "gemv_hbm_gbps"), ("head_bs1", "lm_head_argmax_hbm_gbps"), ("head_bs16", "lm_head_argmax_hbm_gbps"),
                       ("moe_decode_bs16", "fused_moe_decode_step_hbm_gbps"), ("moe_prefill_128", "fused_moe_decode_step_hbm_gbps"),
                       ("prefill_gemm", "prefill_gemm_tflops"), ("engine_decode", "engine_decode_tok_per_s")):
        monkeypatch.setattr(sys, "argv", ["bench.py", "--workload", wl, "--no-cpu", "--no-extras"])
        bench.main()
        out = _one_json_line(capsys)
        assert out["metric"] == metric and out["config"]["workload"] == wl and out["value"] > 0, wl
    monkeypatch.setattr(sys, "argv", ["bench.py", "--workload", "extras", "--no-cpu"])
    bench.main()
    ex = _one_json_line(capsys)["extras"]
    assert "gemv_q8_0_8192x2048" in ex and not any(k.startswith("stream:") for k in ex)
    # both forms of the one-row kernels side by side, on request only
    monkeypatch.setattr(sys, "argv", ["bench.py", "--workload", "extras", "--no-cpu", "--ab-forms"])
    bench.main()
    ex = _one_json_line(capsys)["extras"]
    for form in ("lane", "stream"):
        for k in ("gemv_iq4_xs_8192x2048", "gemv_q6_k_sustained_256MiB", "head_q6k_151936_bs1", "moe_decode_bs1"):
            assert "error" not in ex[f"{form}:{k}"], (form, k, ex[f"{form}:{k}"])
    for k in ("gemm_tiled:prefill_gemm_q8_0_8192x2048x128", "moe_rows:moe_decode_bs16_q6k_down", "moe_rows:prefill_moe_128_tokens", "head_rows:head_q6k_151936_bs16"):
        assert "error" not in ex[k], (k, ex[k])
    assert qk.get_option("one_row") == 0 and qk.get_option("moe_rows") == 0   # the switches are back at their defaults


def test_a_failing_side_measurement_is_an_entry_of_the_line(monkeypatch, capsys, qk):
    bench = _bench_with_stub_workloads(monkeypatch, qk)

    def broken(*a, **k):
        raise RuntimeError("no such kernel")
    monkeypatch.setattr(bench, "head_workload", broken)
    monkeypatch.setattr(sys, "argv", ["bench.py", "--steps", "20", "--warmup", "5", "--no-cpu"])
    bench.main()
    out = _one_json_line(capsys)
    assert out["value"] > 0 and "no such kernel" in out["extras"]["head_q6k_151936_bs1"]["error"]
    assert "error" not in out["extras"]["gemv_q8_0_8192x2048"]
