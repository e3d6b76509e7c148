"""The library's switches (include/qk_kernels.h: qkk_set_option / qkk_get_option, QK_<NAME> in the environment):
names, defaults, ranges, and how the environment is read.  Host code of libqk.so only -- no GPU call is made."""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# name: (default, lowest, highest); the default of every switch is the form that has run on a device
SWITCHES = {"one_row": (0, 0, 1), "dense_reg": (0, 0, 1), "fused_norm": (0, 0, 1), "attn_block": (0, 0, 1), "dn_fused": (0, 0, 1),
            "gemm_tiled": (0, 0, 1), "moe_rows": (0, 0, 1), "head_rows": (0, 0, 1), "select_ranked": (1, 0, 1),
            "gemv_depth": (0, 0, 16), "head_depth": (0, 0, 8), "rowwise_max": (0, 0, 64)}


def in_a_fresh_process(env, code):
    """The switches are read from the environment on first use, so each case gets a process of its own."""
    full = {k: v for k, v in os.environ.items() if not k.startswith("QK_")}
    full.update(env)
    r = subprocess.run([sys.executable, "-c", "import sys; sys.path.insert(0, %r)\nimport __graft_entry__ as g\nqk = g.load_package()\n" % ROOT + code],
                       capture_output=True, text=True, env=full, cwd=ROOT, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stdout.strip()


def test_every_documented_switch_exists_with_its_default():
    out = in_a_fresh_process({}, "print({n: qk.get_option(n) for n in %r})" % list(SWITCHES))
    assert eval(out) == {n: d for n, (d, _, _) in SWITCHES.items()}
    # the header's list and this one name the same switches
    header = open(os.path.join(ROOT, "include", "qk_kernels.h")).read()
    block = header[header.index("Names and values:"):header.index("int qkk_set_option")]
    assert set(re.findall(r'"([a-z_]+)"', block)) - {"lane", "stream"} == set(SWITCHES)   # "lane" / "stream": values of QK_ONE_ROW


def test_ranges_and_unknown_names(qk):
    for name, (default, lo, hi) in SWITCHES.items():
        old = qk.get_option(name)
        try:
            for v in (lo, hi):
                qk.set_option(name, v)
                assert qk.get_option(name) == v
            for bad in (lo - 1, hi + 1):
                with pytest.raises(qk.QkError) as e:
                    qk.set_option(name, bad)
                assert e.value.code == -1 and qk.get_option(name) == hi   # refused, the switch keeps its value
        finally:
            qk.set_option(name, old)
    for call in (lambda: qk.set_option("no_such_switch", 1), lambda: qk.get_option("no_such_switch")):
        with pytest.raises(qk.QkError) as e:
            call()
        assert e.value.code == -1
    with qk.option("moe_rows", 1):
        assert qk.get_option("moe_rows") == 1
    assert qk.get_option("moe_rows") == 0


def test_the_environment_is_read_on_first_use():
    env = {"QK_ONE_ROW": "stream", "QK_MOE_ROWS": "1", "QK_HEAD_ROWS": "1", "QK_GEMM_TILED": "1", "QK_SELECT_RANKED": "0",
           "QK_GEMV_DEPTH": "4", "QK_ROWWISE_MAX": "12"}
    out = eval(in_a_fresh_process(env, "print({n: qk.get_option(n) for n in %r})" % list(SWITCHES)))
    assert out == {**{n: d for n, (d, _, _) in SWITCHES.items()}, "one_row": 1, "moe_rows": 1, "head_rows": 1, "gemm_tiled": 1,
                   "select_ranked": 0, "gemv_depth": 4, "rowwise_max": 12}
    # "lane" is the other spelling of QK_ONE_ROW; values outside a switch's range, or not numbers, are ignored
    env = {"QK_ONE_ROW": "lane", "QK_MOE_ROWS": "2", "QK_GEMV_DEPTH": "17", "QK_HEAD_DEPTH": "-1", "QK_DN_FUSED": "yes", "QK_ATTN_BLOCK": ""}
    out = eval(in_a_fresh_process(env, "print({n: qk.get_option(n) for n in %r})" % list(SWITCHES)))
    assert out == {n: d for n, (d, _, _) in SWITCHES.items()}
    # a switch set by a call is not overwritten by a later look at the same environment
    out = in_a_fresh_process({"QK_MOE_ROWS": "1"}, "qk.set_option('moe_rows', 0); print(qk.get_option('moe_rows'), qk.get_option('head_rows'))")
    assert out == "0 0"
