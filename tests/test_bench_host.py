"""The host side of bench.py: argument handling and the CPU-baseline leg (no GPU needed)."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and not r.stdout.strip()


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
