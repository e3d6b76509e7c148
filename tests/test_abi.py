"""libqk.so loads on a machine without a GPU, exports every symbol its headers declare, and
fails loudly (no CPU path) when asked to compute without a device."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header):
    src = open(os.path.join(ROOT, "include", header)).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(qkk?_[a-z0-9_]+)\s*\(", src)))


def test_headers_declare_the_expected_surface():
    eng = declared("qk.h")
    assert len(eng) == 20, eng   # the reference header declares 20 functions
    for must in ["qk_open", "qk_close", "qk_slot_start", "qk_slot_cancel", "qk_step_chunk", "qk_stage_run",
                 "qk_stage_topk", "qk_state_n", "qk_state_save", "qk_state_load", "qk_n_embd"]:
        assert must in eng
    assert "qkk_moe_decode" in declared("qk_kernels.h")


@pytest.mark.parametrize("header", ["qk.h", "qk_kernels.h"])
def test_library_exports_every_declared_symbol(qk, header):
    L = qk.lib()
    for name in declared(header):
        assert hasattr(L, name), name


def test_sel_record_is_160_bytes(qk):
    assert C.sizeof(qk.QkSel) == 160


def test_row_bytes(qk):
    assert qk.row_bytes(qk.Q8_0, 2048) == 2176
    assert qk.row_bytes(qk.Q6_K, 2048) == 1680
    assert qk.row_bytes(qk.IQ4_XS, 512) == 272
    assert qk.row_bytes(qk.IQ3_XXS, 2048) == 784
    assert qk.row_bytes(qk.F16, 10) == 20 and qk.row_bytes(qk.F32, 10) == 40
    assert qk.row_bytes(qk.Q6_K, 100) == 0 and qk.row_bytes(99, 256) == 0


def test_engine_abi_argument_checks(qk):
    L = qk.lib()
    L.qk_open.restype = C.c_void_p
    L.qk_open.argtypes = [C.c_char_p, C.c_void_p, C.c_char_p, C.c_size_t]
    err = C.create_string_buffer(256)

    class Cfg(C.Structure):
        _fields_ = [("n_slots", C.c_uint32), ("n_ctx", C.c_uint32), ("chunk", C.c_uint32)]

    assert L.qk_open(None, None, err, 256) is None and err.value == b"qk_open: null arg"
    for bad in [Cfg(0, 4096, 4), Cfg(17, 4096, 4), Cfg(4, 63, 4), Cfg(4, 65537, 4), Cfg(4, 4096, 0), Cfg(4, 4096, 33)]:
        assert L.qk_open(b"/nonexistent.gguf", C.byref(bad), err, 256) is None
        assert err.value == b"qk_open: bad config"
    assert L.qk_open(b"/nonexistent.gguf", C.byref(Cfg(4, 4096, 4)), err, 256) is None
    assert err.value == b"qk_open: cannot open GGUF"
    small = C.create_string_buffer(8)
    assert L.qk_open(None, None, small, 8) is None and small.raw[7:8] == b"\0"
    # null engine: the entry points that check return the reference's codes
    L.qk_slot_start.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32]
    L.qk_step_chunk.argtypes = [C.c_void_p] * 4
    L.qk_stage_run.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
    L.qk_stage_topk.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p]
    L.qk_state_save.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32]
    assert L.qk_slot_start(None, 0, None, 0, 0, 0) == -1
    assert L.qk_step_chunk(None, None, None, None) == -1
    assert L.qk_stage_run(None, 0, None, None, 1, 0, None, None) == -1
    assert L.qk_stage_topk(None, 1, None, None) == -1
    assert L.qk_state_save(None, 0, 0, 0) == -1
    L.qk_close.argtypes = [C.c_void_p]
    L.qk_close(None)


def test_no_cpu_fallback(qk):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    assert qk.device_info()["devices"] == 0
    rc = qk.lib().qkk_gemv(qk.Q8_0, 16, 16, 16, 4, 32, 1, None)   # non-null dummy pointers
    assert rc == -4
    assert b"no HIP device" in qk.lib().qkk_last_error()
    assert qk.lib().qkk_gemv(qk.Q8_0, None, None, None, 4, 32, 1, None) == -1
