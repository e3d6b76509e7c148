"""`qk`, the operator test program (qwen-kernel_amd/csrc/qk_cli.cpp; the modes of the reference's binary,
src/main.cpp:6952-6978).  Without a GPU its logic runs over the host-side build of the kernels (tests/emu/qk_emu:
the same source against the stand-in runtime); on a device the real binary runs a small case per mode."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
QK = os.path.join(ROOT, "qwen-kernel_amd", "qk")
QK_EMU = os.path.join(ROOT, "tests", "emu", "qk_emu")


def run(binary, *args, timeout=300, env=None):
    return subprocess.run([binary, *map(str, args)], capture_output=True, text=True, timeout=timeout,
                          env=None if env is None else {**os.environ, **env})


@pytest.fixture(scope="module")
def qk_emu():
    if not os.path.exists(QK_EMU):
        subprocess.run(["make", "-C", os.path.dirname(QK_EMU), "-j", "8"], check=True, stdout=subprocess.DEVNULL)
    return QK_EMU


def test_usage_and_no_device():
    """No mode, or an unknown one: the usage text and status 1.  A mode without a HIP device: a message that
    says so and status 2 -- the program has no CPU arithmetic to fall back on."""
    if not os.path.exists(QK):
        pytest.skip("qk is not built")
    for args in ((), ("frobnicate",)):
        r = run(QK, *args)
        assert r.returncode == 1 and "usage: qk suite" in r.stderr and not r.stdout
    import torch
    if not torch.cuda.is_available():
        r = run(QK, "q8_0", 64, 256, 1)
        assert r.returncode == 2 and "no HIP device" in r.stderr


@pytest.mark.parametrize("args", [("q8_0", 96, 512, 2), ("q6_k", 33, 2048, 1), ("iq4_xs", 40, 1024, 1), ("iq3_xxs", 40, 2048, 1),
                                  ("f16", 21, 768, 1), ("bgemm", 48, 512, 20, 1), ("moe", 1, 1, 1, 8), ("moe", 2, 1, 3, 8)],
                         ids=lambda a: "-".join(map(str, a)))
def test_modes_in_the_host_build(qk_emu, args):
    """Every mode on a small shape: the line with the rates, the verdict of the second computation (the
    dequantise + dense product for the GEMVs, one GEMV per token for the GEMM, the expert-major path for the
    MoE rows), status 0."""
    r = run(qk_emu, *args)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "us/iter" in r.stdout and "GB/s" in r.stdout and "-> OK" in r.stdout and "FAIL" not in r.stdout
    assert r.stdout.strip().endswith("ALL OK")


def test_bad_shapes_are_refused(qk_emu):
    r = run(qk_emu, "q6_k", 8, 100, 1)     # K is not a multiple of the 256-weight block
    assert r.returncode == 1 and "not a multiple" in r.stderr
    r = run(qk_emu, "moe", 0, 1, 5000)
    assert r.returncode == 1 and "outside" in r.stderr


@pytest.fixture(scope="module")
def model_file(qk, tmp_path_factory):
    """A GGUF file with one MoE layer under the reference's tensor names (blk.3.ffn_*) and an F16 tensor."""
    import numpy as np
    hl = qk.synth.HostLayer(seed=5, n_embd=2048, n_ff=256, n_expert=8, n_used=2, down_type=qk.Q6_K)
    path = str(tmp_path_factory.mktemp("gguf") / "model.gguf")
    half = np.random.default_rng(1).standard_normal((24, 512)).astype(np.float16)
    qk.gguf.write(path, {"general.architecture": "qwen3next", "qwen3next.expert_used_count": 2},
                  qk.gguf.layer_tensors(hl, 3) + [("token_embd.weight", qk.F16, (512, 24), half)])
    return path


def test_modes_on_a_model_file_in_the_host_build(qk_emu, model_file):
    """The reference's real-weight modes (src/main.cpp:846-915, 920-1254) on a file named by QK_GGUF: the tensor
    list, y = W x on named tensors (a 3-D expert tensor: its first slice) with the dequantise + dense verdict,
    and the fused step on a layer's tensors, one row and three, with the expert-major path as second opinion."""
    env = {"QK_GGUF": model_file}
    r = run(qk_emu, "list", "blk.3.ffn_down", env=env)
    assert r.returncode == 0 and "9 tensors" in r.stdout, r.stdout + r.stderr
    lines = [ln for ln in r.stdout.splitlines() if ln.startswith("blk.")]
    assert len(lines) == 2 and "q6_k" in lines[0] and "[256, 2048, 8, 1]" in lines[0] and "q8_0" in lines[1]
    for tensor, typ in (("blk.3.ffn_gate_exps.weight", "iq3_xxs"), ("blk.3.ffn_down_shexp.weight", "q8_0"),
                        ("token_embd.weight", "f16")):
        r = run(qk_emu, "gguf", tensor, 1, env=env)
        assert r.returncode == 0 and typ in r.stdout and "-> OK" in r.stdout and r.stdout.strip().endswith("ALL OK"), r.stdout + r.stderr
    r = run(qk_emu, "gguf", "blk.3.ffn_gate_inp.weight", 1, env=env)
    assert r.returncode == 0 and "check: none" in r.stdout
    for slots in (1, 3):
        r = run(qk_emu, "layer", 3, 1, slots, env=env)
        assert r.returncode == 0, r.stdout + r.stderr
        assert "8 experts, 2 used, down q6_k" in r.stdout and "picks equal on both paths -> OK" in r.stdout
        assert r.stdout.strip().endswith("ALL OK")


def test_model_file_errors(qk_emu, model_file):
    r = run(qk_emu, "gguf", "x", env={"QK_GGUF": ""})
    assert r.returncode == 1 and "Set QK_GGUF" in r.stderr
    r = run(qk_emu, "list", env={"QK_GGUF": model_file + ".missing"})
    assert r.returncode == 1 and "model.gguf.missing" in r.stderr
    r = run(qk_emu, "gguf", "blk.9.nothing", env={"QK_GGUF": model_file})
    assert r.returncode == 1 and "not found" in r.stderr
    r = run(qk_emu, "layer", 4, 1, env={"QK_GGUF": model_file})
    assert r.returncode == 1 and "layer 4" in r.stderr
    r = run(qk_emu, "gguf")
    assert r.returncode == 1 and "usage" in r.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("args", [("q8_0", 8192, 2048, 50), ("iq3_xxs", 8192, 2048, 50), ("f16", 4096, 4096, 20),
                                  ("bgemm", 8192, 2048, 128, 10), ("moe", 0, 40, 1), ("moe", 0, 20, 4), ("head", 1, 6)],
                         ids=lambda a: "-".join(map(str, a)))
def test_modes_on_the_device(dev, args):
    if dev == "cpu":
        pytest.skip("the host-side build has its own cases above")
    print(f"[case] qk {' '.join(map(str, args))}", flush=True)
    r = run(QK, *args, timeout=600)
    print(r.stdout, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "GB/s" in r.stdout and r.stdout.strip().endswith("ALL OK")


@pytest.fixture(scope="module")
def whole_model(qk, tmp_path_factory):
    """A small whole model of the reference's family (a gated-DeltaNet layer and a full-attention layer) and a prompt."""
    d = tmp_path_factory.mktemp("whole")
    path = qk.engine.FullModel(23, kinds="RA", vocab=192, eos=197).write(str(d / "model.gguf"))
    ids = d / "prompt.txt"
    ids.write_text("5, 17 3\n44,9\n120 7")
    return path, str(ids)


def gen_of(out):
    return [ln for ln in out.splitlines() if ln.startswith("GEN:")][0].split()[1:]


def test_whole_model_modes_in_the_host_build(qk_emu, whole_model):
    """`qk token` and `qk warm` (reference src/main.cpp:2500-3062) over the engine ABI: the prompt's ids from a
    file, greedy tokens on one slot and on three slots fed the same prompt (identical streams, and the stream of
    the single slot), and the stream behind a restored snapshot equal to the one behind the prefill."""
    path, ids = whole_model
    env = {"QK_GGUF": path}
    one = run(qk_emu, "token", ids, 5, 64, env=env)
    assert one.returncode == 0 and "token mode: 7 prompt ids, gen 5, vocab 192" in one.stdout, one.stdout + one.stderr
    assert len(gen_of(one.stdout)) == 5 and one.stdout.strip().endswith("ALL OK")
    three = run(qk_emu, "token", ids, 5, 64, 3, env=env)
    assert three.returncode == 0 and "streams identical: YES" in three.stdout, three.stdout + three.stderr
    assert gen_of(three.stdout) == gen_of(one.stdout)
    warm = run(qk_emu, "warm", ids, 5, 64, env={**env, "QK_PCACHE": "5"})   # the reference's knob for the snapshot entries
    assert warm.returncode == 0 and "warm stream identical to cold: YES" in warm.stdout, warm.stdout + warm.stderr
    assert "5 snapshot entries" in warm.stdout
    assert gen_of(warm.stdout) == gen_of(one.stdout)
    # twelve slots: the expert-major MoE path and the several-row head inside the captured step; with the row-split
    # forms switched on the shared expert's launches fork onto the library's side stream inside the capture
    many = run(qk_emu, "token", ids, 3, 64, 12, env={**env, "QK_MOE_ROWS": "1", "QK_HEAD_ROWS": "1"}, timeout=600)
    assert many.returncode == 0 and "streams identical: YES" in many.stdout, many.stdout + many.stderr
    assert gen_of(many.stdout) == gen_of(one.stdout)[:3]
    # QK_WEIGHT_SLAB=1: the file's tensors carved from one device allocation; the same stream
    slab = run(qk_emu, "token", ids, 5, 64, env={**env, "QK_WEIGHT_SLAB": "1"})
    assert slab.returncode == 0 and gen_of(slab.stdout) == gen_of(one.stdout), slab.stdout + slab.stderr
    # QK_STEP_PROF (reference src/main.cpp:4591-4632): the first decode step's stages on stderr, once, the stream unchanged
    prof = run(qk_emu, "token", ids, 5, 64, env={**env, "QK_STEP_PROF": "1", "QK_STEP_PROF_DETAIL": "1"})
    assert prof.returncode == 0 and gen_of(prof.stdout) == gen_of(one.stdout), prof.stdout + prof.stderr
    assert prof.stderr.count("[prof] decode step:") == 1 and "across 15 stages" in prof.stderr, prof.stderr
    for stage in ("emb", "rms0", "dn.proj", "dn.ab+conv", "dn.step", "dn.out", "at.proj", "at.prep", "at.attn", "at.out", "moe", "rms", "head"):
        assert f"[prof]   {stage:<10s} n=" in prof.stderr, (stage, prof.stderr)
    assert prof.stderr.count("[prof-detail]") == 15 and "[prof]   moe        n=2" in prof.stderr
    # QK_COUNTERS (reference src/main.cpp:5250-5281): the stages of the first prefill pass (a prompt of 20 ids: 19
    # positions are prefilled together, the last one is a serial step)
    long_ids = os.path.join(os.path.dirname(ids), "long.txt")
    with open(long_ids, "w") as f:
        f.write(" ".join(str(3 + 7 * i) for i in range(20)))
    plain = run(qk_emu, "token", long_ids, 3, 64, env=env)
    cnt = run(qk_emu, "token", long_ids, 3, 64, env={**env, "QK_COUNTERS": "1", "QK_COUNTER_RAW": "1"})
    assert cnt.returncode == 0 and gen_of(cnt.stdout) == gen_of(plain.stdout), cnt.stdout + cnt.stderr
    assert cnt.stderr.count("[qk counters] HIP batched prefill N=19 base=0") == 1, cnt.stderr
    for stage in ("emb", "rms0", "dn.proj", "dn.ab+conv", "dn.step", "dn.out", "at.proj", "at.prep", "at.attn", "at.out", "addN",
                  "moe+tail"):   # more than ten rows: the add + norm launch and the MoE step with its tail
        assert f"[qk counters] {stage:<22s}" in cnt.stderr, (stage, cnt.stderr)
    assert "[qk counter raw] 001 emb" in cnt.stderr
    # refusals: a prompt that does not fit, a batch the engine has no slots for, a missing file, no model
    r = run(qk_emu, "token", ids, 60, 64, env=env)
    assert r.returncode == 1 and "bad prompt" in r.stderr
    r = run(qk_emu, "token", ids, 5, 64, 17, env=env)
    assert r.returncode == 1 and "batch must be" in r.stderr
    r = run(qk_emu, "token", ids + ".missing", 5, env=env)
    assert r.returncode == 1
    r = run(qk_emu, "token", ids, 5, env={"QK_GGUF": ""})
    assert r.returncode == 1 and "Set QK_GGUF" in r.stderr
    r = run(qk_emu, "warm", ids)
    assert r.returncode == 1 and "usage" in r.stderr


SWITCH_SETS = [{}, {"QK_ONE_ROW": "stream", "QK_DENSE_REG": "1", "QK_FUSED_NORM": "1", "QK_DN_FUSED": "1", "QK_ATTN_BLOCK": "1"},
               {"QK_ONE_ROW": "stream", "QK_SELECT_RANKED": "0"},
               {"QK_GEMM_TILED": "1", "QK_MOE_ROWS": "1", "QK_HEAD_ROWS": "1", "QK_PREFILL_ROWS": "16"}]


@pytest.mark.skipif(os.environ.get("QK_TEST_SANITIZE") != "1", reason="set QK_TEST_SANITIZE=1: builds every kernel under "
                    "AddressSanitizer + UndefinedBehaviorSanitizer (minutes) and runs the program's modes through it")
def test_modes_under_the_sanitizers(model_file, whole_model):
    """The host-side build of every kernel, the engine and the test program as ONE executable under ASan and UBSan
    (tests/emu/Makefile, target qk_emu_san): each mode under each set of switches must end with its verdict and
    without a report -- static LDS arrays, arrays on a thread's stack and the kernels' address arithmetic are
    what the guard pages of the other tests cannot see."""
    subprocess.run(["make", "-C", os.path.dirname(QK_EMU), "-j", "8", "qk_emu_san"], check=True, stdout=subprocess.DEVNULL)
    san = os.path.join(os.path.dirname(QK_EMU), "qk_emu_san")
    path, ids = whole_model
    base = {"ASAN_OPTIONS": "detect_stack_use_after_return=0:detect_leaks=0", "UBSAN_OPTIONS": "print_stacktrace=1"}
    cases = [((f, 67, 2048, 1), {}) for f in ("q8_0", "q6_k", "iq4_xs", "iq3_xxs")] + [(("iq4_xs", 9, 768, 1), {}), (("f16", 40, 2048, 1), {}),
             (("bgemm", 48, 512, 20, 1), {}), (("bgemm", 64, 2048, 130, 1), {}), (("moe", 1, 1, 1, 8), {}), (("moe", 2, 1, 3, 8), {}),
             (("moe", 3, 1, 16, 8), {}), (("moe", 3, 1, 40, 16), {}), (("layer", 3, 1, 1), {"QK_GGUF": model_file}),
             (("layer", 3, 1, 12), {"QK_GGUF": model_file}), (("token", ids, 4, 64, 1), {"QK_GGUF": path}),
             (("token", ids, 4, 64, 3), {"QK_GGUF": path}), (("warm", ids, 4, 64), {"QK_GGUF": path})]
    for sw in SWITCH_SETS:
        for args, env in cases:
            r = run(san, *args, timeout=1500, env={**base, **sw, **env})
            assert r.returncode == 0 and "runtime error" not in r.stderr and "Sanitizer" not in r.stderr, (sw, args, r.stdout[-500:], r.stderr[-3000:])


@pytest.mark.gpu
def test_whole_model_modes_on_the_device(dev, whole_model):
    if dev == "cpu":
        pytest.skip("the host-side build has its own cases above")
    path, ids = whole_model
    outs = []
    for args in (("token", ids, 8, 64), ("token", ids, 8, 64, 4), ("warm", ids, 8, 64)):
        print(f"[case] QK_GGUF=... qk {' '.join(map(str, args))}", flush=True)
        r = run(QK, *args, timeout=300, env={"QK_GGUF": path})
        print(r.stdout, flush=True)
        assert r.returncode == 0 and r.stdout.strip().endswith("ALL OK"), r.stdout + r.stderr
        outs.append(gen_of(r.stdout))
    # one slot twice: the same kernels, the same stream (four slots run other kernel families, whose sums differ
    # in the last bits: their streams are compared with each other inside the program, not with the single slot's)
    assert outs[0] == outs[2]


@pytest.mark.gpu
def test_modes_on_a_model_file_on_the_device(dev, model_file):
    if dev == "cpu":
        pytest.skip("the host-side build has its own cases above")
    env = {"QK_GGUF": model_file}
    for args in (("gguf", "blk.3.ffn_gate_exps.weight", 20), ("gguf", "blk.3.ffn_down_exps.weight", 20), ("layer", 3, 20, 1),
                 ("layer", 3, 10, 4)):
        print(f"[case] QK_GGUF=... qk {' '.join(map(str, args))}", flush=True)
        r = run(QK, *args, timeout=300, env=env)
        print(r.stdout, flush=True)
        assert r.returncode == 0, r.stdout + r.stderr
        assert r.stdout.strip().endswith("ALL OK")
