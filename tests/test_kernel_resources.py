"""What the device compiler made of the kernels, without a GPU: every .hip file is compiled for gfx950 with
-Rpass-analysis=kernel-resource-usage and the figures per kernel are checked -- no kernel keeps registers in
scratch memory (a spill in a streaming loop costs more than any tuning gains), static LDS stays inside the
64 KB a kernel may declare, and the one-row streaming kernels keep at least two waves per SIMD."""
import concurrent.futures
import glob
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "qwen-kernel_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def compile_file(path, include_dir=None):
    """One device compilation of a .hip file: ({kernel: resource figures}, {kernel: its assembly})."""
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        r = subprocess.run([HIPCC, "--offload-arch=gfx950", "--cuda-device-only", "-O3", "-std=c++17", "-Xclang", "-target-feature",
                            "-Xclang", "-packed-fp32-ops", "-I" + (include_dir or os.path.join(ROOT, "include")), "-S", path,
                            "-Rpass-analysis=kernel-resource-usage", "-o", out], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        text = open(out).read()
    use = {}
    for block in re.split(r"remark: Function Name: ", r.stderr)[1:]:
        num = lambda key: int(re.search(key + r": (\d+)", block).group(1))
        use[block.split(" ")[0]] = dict(scratch=num(r"ScratchSize \[bytes/lane\]"), occupancy=num(r"Occupancy \[waves/SIMD\]"),
                                        lds=num(r"LDS Size \[bytes/block\]"), vgprs=num(r"  VGPRs"))
    funcs = {}
    for chunk in re.split(r"\n(?=_ZN2qk\w+:)", text):
        name = chunk.split(":", 1)[0]
        if name.startswith("_ZN2qk") and ".amdhsa_kernel" in chunk:
            funcs[name] = chunk.split(".end_amdhsa_kernel")[0]
    return use, funcs


@pytest.fixture(scope="module")
def compiled():
    """Every .hip file of the library compiled once for gfx950: (resource figures, assembly) per kernel."""
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    files = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=7) as pool:
        per_file = list(pool.map(compile_file, files))
    use, funcs = {}, {}
    for u, f in per_file:
        use.update(u)
        funcs.update(f)
    return use, funcs


@pytest.fixture(scope="module")
def usage(compiled):
    return compiled[0]


@pytest.fixture(scope="module")
def isa(compiled):
    return compiled[1]


def test_no_kernel_spills_and_static_lds_fits(usage):
    assert len(usage) > 200   # every instantiation of every file
    spills = {k: v for k, v in usage.items() if v["scratch"]}
    assert not spills, spills
    assert all(v["lds"] <= 65536 and v["occupancy"] >= 1 for v in usage.values())


def test_streaming_kernels_keep_two_waves_per_simd(usage):
    """The kernels of the one-row decode step at the reference's shapes (mangled names): GEMV at K = 2048 in
    every format, the head, the three MoE launches with 512-wide experts and eight picks."""
    hot = [k for k in usage if ("gemv_stream_kernelILi" in k and "ELi64ELi1E" in k) or "head_q6k_kernelILi1E" in k
           or "moe_route_kernelILi8E" in k or "moe_gateup_kernelILi1ELi4E" in k
           or re.search(r"moe_down_kernelILi(23|14)ELi16ELi2ELi2E", k)]
    assert len(hot) >= 20, len(hot)
    low = {k: usage[k] for k in hot if usage[k]["occupancy"] < 2}
    assert not low, low


def test_row_split_kernels_keep_four_waves_per_simd(usage):
    """The kernels whose waves split the weight rows (512 threads, 64 KB of LDS) are meant to run two workgroups to
    a CU: four waves per SIMD, so at most 128 registers per lane -- and none of them in scratch memory."""
    rows = {k: v for k, v in usage.items() if "moe_rows_kernel" in k or "head_q6k_rows_kernel" in k}
    assert len(rows) == 4, sorted(rows)
    assert all(v["occupancy"] >= 4 and v["vgprs"] <= 128 and v["scratch"] == 0 for v in rows.values()), rows


def test_one_row_kernels_fetch_the_weights_as_16_byte_pieces(isa):
    """The instruction stream of the one-row kernels at the reference's shapes: the weight bytes arrive through
    global_load_dwordx4 (the staged 16-byte pieces, the activations, the tables' sources); in the GEMV and
    head kernels narrower global loads remain only for the rows behind the last full chunk -- at most a third
    as many as the wide ones (the MoE launches also fetch logits, picks and h)."""
    funcs = isa
    hot = [k for k in funcs if ("gemv_stream_kernelILi" in k and "ELi64ELi1E" in k) or "head_q6k_kernelILi1E" in k
           or "moe_route_kernelILi8ELb0E" in k or "moe_gateup_kernelILi1ELi4ELb0E" in k
           or re.search(r"moe_down_kernelILi(23|14)ELi16ELi2ELi2ELb[01]ELb0E", k)]
    assert len(hot) >= 16, len(hot)
    for k in hot:
        loads = re.findall(r"\bglobal_load_(\w+)", funcs[k])
        wide = sum(1 for l in loads if l.startswith("dwordx4"))
        narrow = len(loads) - wide
        assert wide >= 8, (k, wide, narrow)
        if "gemv_stream" in k or "head_q6k" in k:   # the MoE launches also fetch logits, picks and h: scalars and short rows
            assert narrow * 3 <= wide, (k, wide, narrow, sorted(set(loads)))


def test_matrix_kernels_keep_their_loads_in_the_global_address_space(isa):
    """The tiled GEMM and the row-split expert / head kernels: every weight fetch is a global_load_dwordx4.  A
    pointer that loses its address space on the way (a tensor chosen through an array of pointers did) becomes a
    flat load, which also counts against the LDS counter -- every wait for an LDS read then waits for the
    fetches in flight, and the overlap of fetch and arithmetic is gone.  Flat loads are allowed only where a
    kernel reads other workgroups' candidates with system scope (the head's last fold)."""
    funcs = isa
    hot = [k for k in funcs if "moe_rows_kernel" in k or "gemm_tiled_kernel" in k or "head_q6k_rows_kernel" in k]
    assert len(hot) == 8, sorted(hot)
    for k in hot:
        flat = re.findall(r"\bflat_load_\w+[^\n]*", funcs[k])
        assert all("sc0 sc1" in f for f in flat) and len(flat) <= 2, (k, flat)
        assert len(re.findall(r"\bglobal_load_dwordx4", funcs[k])) >= 4, k
        assert "scratch_" not in funcs[k], k


def kernel_key(mangled):
    """(in namespace qk::lane, kernel name, template arguments) of a mangled kernel name."""
    lane = mangled.startswith("_ZN2qk4lane")
    rest = mangled[len("_ZN2qk4lane") if lane else len("_ZN2qk"):]
    digits = re.match(r"\d+", rest).group(0)
    base, tail = rest[len(digits):len(digits) + int(digits)], rest[len(digits) + int(digits):]
    templ = re.match(r"I.*?EEv", tail)
    return lane, base, templ.group(0) if templ else ""


def fingerprints_of(funcs):
    """{"name|template arguments": SHA-1 of the kernel's instruction stream} -- comments, directives, labels and
    symbol names removed, so that a kernel moved to another namespace or file keeps its fingerprint."""
    import hashlib
    out = {}
    for name, chunk in funcs.items():
        ins = []
        for ln in re.split(r"\n\.Lfunc_end\d+:", chunk)[0].split("\n")[1:]:   # up to the end of the function, early exits included
            ln = ln.split(";")[0].strip()
            if not ln or ln.startswith(".") or ln.endswith(":"):
                continue
            ins.append(re.sub(r"_ZN[\w$.]+", "SYM", re.sub(r"\.LBB\d+_\d+", "L", ln)))
        lane, base, templ = kernel_key(name)
        out[("lane::" if lane else "") + base + "|" + templ] = hashlib.sha1("\n".join(ins).encode()).hexdigest()
    return out


# kernels of the same name that are NOT the code of that run: the streamed forms behind the "one_row" switch
STREAMED = {"moe_down_kernel", "moe_route_kernel", "moe_gateup_kernel", "head_q6k_kernel"}
# changed since, on purpose: the routing launches of several rows check the workspace header in one wave
CHANGED = {"moe_logits_tiled_kernel", "moe_route_multi_kernel"}


def test_default_kernels_are_the_device_code_of_the_last_run_on_a_device(isa):
    """tests/golden/device_code_62fdaf6.json holds a fingerprint of every kernel of the last tree that ran, and
    passed its GPU tests, on an MI355X.  Every kernel the library runs BY DEFAULT must still compile to that code,
    instruction for instruction: the per-lane one-row kernels (now in namespace qk::lane, the head's renamed),
    the cooperative matrix-core kernels, the mixers, the glue, the dequantisation.  What was written since sits
    behind switches and has other names; the two routing kernels that changed are named above."""
    import json
    golden = json.load(open(os.path.join(ROOT, "tests", "golden", "device_code_62fdaf6.json")))["kernels"]
    now = fingerprints_of(isa)
    same, differ, checked = 0, [], set()
    for key, sha in now.items():
        name, templ = key.split("|")
        lane = name.startswith("lane::")
        base = name[6:] if lane else name
        if not lane and base in STREAMED:
            continue
        old = ("head_q6k_kernel" if base == "head_q6k_lane_kernel" else base) + "|" + templ
        if old not in golden and templ.endswith("Lb0EEEv"):   # a template switch added since, here at "off"
            old = old[:-len("Lb0EEEv")] + "EEv"
        if old not in golden:
            continue
        checked.add(old)
        if golden[old] == sha:
            same += 1
        elif base not in CHANGED:
            differ.append(key)
    assert not differ, differ
    assert same >= 320, same
    # and nothing that ran then has gone missing from the library
    gone = [k for k in golden if k not in checked]
    assert not gone, gone
