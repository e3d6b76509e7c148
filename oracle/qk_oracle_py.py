"""ctypes binding of the CPU oracle (oracle/liboracle.so) and of the reference build
(oracle/_ref/libqkref.so).  TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke
check and by the benchmark's cpu_baseline leg; the product never imports it."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
F32, F16, Q8_0, Q6_K, IQ3_XXS, IQ4_XS = 0, 1, 8, 14, 18, 23


class Sel(C.Structure):
    _fields_ = [("ids", C.c_uint32 * 16), ("w", C.c_float * 16), ("w_shared", C.c_float), ("pad", C.c_float * 7)]


class SelF64(C.Structure):
    _fields_ = [("ids", C.c_uint32 * 16), ("w", C.c_double * 16), ("w_shared", C.c_double), ("gap", C.c_double)]


class Layer(C.Structure):
    _fields_ = [("n_embd", C.c_uint32), ("n_ff", C.c_uint32), ("n_expert", C.c_uint32), ("n_used", C.c_uint32),
                ("gu_type", C.c_int32), ("down_type", C.c_int32),
                ("gate_inp", C.c_void_p), ("gate_inp_shexp", C.c_void_p), ("gate_exps", C.c_void_p),
                ("up_exps", C.c_void_p), ("down_exps", C.c_void_p), ("gate_shexp", C.c_void_p),
                ("up_shexp", C.c_void_p), ("down_shexp", C.c_void_p)]


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        p = os.path.join(HERE, "liboracle.so")
        if not os.path.exists(p):
            raise RuntimeError(f"{p} missing: run `make -C oracle`")
        L = C.CDLL(p)
        vp, u32 = C.c_void_p, C.c_uint32
        L.qko_f16_to_f32.restype = C.c_float
        L.qko_f16_to_f32.argtypes = [C.c_uint16]
        L.qko_f32_to_f16.restype = C.c_uint16
        L.qko_f32_to_f16.argtypes = [C.c_float]
        L.qko_ksign.restype = C.c_uint8
        L.qko_ksign.argtypes = [u32]
        L.qko_row_bytes.restype = C.c_size_t
        L.qko_row_bytes.argtypes = [C.c_int, C.c_uint64]
        L.qko_dequant_row.argtypes = [C.c_int, vp, vp, C.c_int64]
        L.qko_gemv.argtypes = [C.c_int, vp, vp, vp, u32, u32, u32]
        L.qko_argmax.restype = u32
        L.qko_argmax.argtypes = [vp, u32]
        L.qko_select_f64.argtypes = [vp, u32, u32, vp]
        L.qko_select_f32.argtypes = [vp, u32, u32, vp]
        L.qko_moe_ref.argtypes = [vp, vp, vp, vp, vp, vp]
        L.qko_group_pairs.argtypes = [vp, u32, u32, u32, vp, vp]
        L.qko_gemm_q8_0.argtypes = [vp, vp, vp, u32, u32, u32]
        L.qko_gemv_mt.argtypes = [C.c_int, vp, vp, vp, u32, u32, u32, u32]
        L.qko_gemm_q8_0_mt.argtypes = [vp, vp, vp, u32, u32, u32, u32]
        L.qko_moe_ref_mt.argtypes = [vp, vp, vp, u32]
        L.qko_moe_ref_tokens_mt.argtypes = [vp, vp, vp, u32, u32]
        L.qko_max_rel_err.restype = C.c_double
        L.qko_max_rel_err.argtypes = [vp, vp, C.c_size_t]
        L.qko_max_err_over_rms.restype = C.c_double
        L.qko_max_err_over_rms.argtypes = [vp, vp, C.c_size_t]
        L.qko_add_rms.restype = None
        L.qko_add_rms.argtypes = [vp, vp, vp, vp, vp, vp, u32, C.c_float]
        L.qko_embed.argtypes = [C.c_int, vp, u32, u32, vp, u32, u32, vp, u32]
        _lib = L
    return _lib


def ref():
    """The reference's own dequantisation header compiled in this container; None when the
    library has not been built (the reference tree is not present on the GPU box)."""
    global _ref
    if _ref is None:
        p = os.path.join(HERE, "_ref", "libqkref.so")
        if not os.path.exists(p):
            return None
        R = C.CDLL(p)
        R.qkref_f16_to_f32.restype = C.c_float
        R.qkref_f16_to_f32.argtypes = [C.c_uint16]
        R.qkref_f32_to_f16.restype = C.c_uint16
        R.qkref_f32_to_f16.argtypes = [C.c_float]
        R.qkref_block_bytes.restype = C.c_size_t
        R.qkref_dequant_row.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64]
        R.qkref_iq3xxs_grid.restype = C.c_uint32
        R.qkref_ksigns.restype = C.c_uint8
        R.qkref_kmask.restype = C.c_uint8
        R.qkref_iq4nl.restype = C.c_int8
        R.qkref_gemv.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_uint32,
                                 C.c_uint32, C.c_void_p]
        _ref = R
    return _ref


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def row_bytes(type_, k):
    return lib().qko_row_bytes(type_, k)


def dequant(type_, raw, n_elems, use_ref=False):
    """raw: uint8 array of blocks; returns float32[n_elems]."""
    raw = np.ascontiguousarray(raw).reshape(-1)
    out = np.empty(n_elems, dtype=np.float32)
    if use_ref:
        rc = ref().qkref_dequant_row(type_, _p(raw), _p(out), n_elems)
    else:
        rc = lib().qko_dequant_row(type_, _p(raw), _p(out), n_elems)
    if rc:
        raise ValueError(f"dequant rc={rc}")
    return out


def gemv(type_, W, x, M, K, threads=1):
    """threads > 1: the rows split over host threads (bit for bit the same result)."""
    W = np.ascontiguousarray(W).reshape(-1)
    x = np.ascontiguousarray(x, dtype=np.float32)
    batch = 1 if x.ndim == 1 else x.shape[0]
    y = np.empty((batch, M), dtype=np.float32)
    if threads > 1:
        rc = lib().qko_gemv_mt(type_, _p(W), _p(x), _p(y), M, K, batch, threads)
    else:
        rc = lib().qko_gemv(type_, _p(W), _p(x), _p(y), M, K, batch)
    if rc:
        raise ValueError(f"gemv rc={rc}")
    return y if x.ndim == 2 else y[0]


def add_rms(a, w, eps, b=None, c=None, want_sum=False):
    """Rows of a (+b (+c)) summed in float32, RMS-normed in double with weight w.  Returns xn, or
    (sum, xn)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    rows = a.reshape(-1, a.shape[-1])
    n = rows.shape[1]
    bb = None if b is None else np.ascontiguousarray(b, dtype=np.float32).reshape(-1, n)
    cc = None if c is None else np.ascontiguousarray(c, dtype=np.float32).reshape(-1, n)
    w = np.ascontiguousarray(w, dtype=np.float32)
    s = np.empty_like(rows)
    xn = np.empty_like(rows)
    for r in range(rows.shape[0]):
        lib().qko_add_rms(_p(rows[r]), None if bb is None else _p(bb[r]), None if cc is None else _p(cc[r]), _p(w),
                          _p(s[r]), _p(xn[r]), n, eps)
    s, xn = s.reshape(a.shape), xn.reshape(a.shape)
    return (s, xn) if want_sum else xn


def embed(type_, W, n_vocab, kdim, ids, idx, per_req, rows):
    W = np.ascontiguousarray(W).reshape(-1)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    x = np.empty((rows, kdim), dtype=np.float32)
    rc = lib().qko_embed(type_, _p(W), n_vocab, kdim, _p(ids), idx, per_req, _p(x), rows)
    if rc:
        raise ValueError(f"embed rc={rc}")
    return x


def argmax(v):
    v = np.ascontiguousarray(v, dtype=np.float32)
    return int(lib().qko_argmax(_p(v), v.size))


def select_f64(logits, n_used):
    logits = np.ascontiguousarray(logits, dtype=np.float64)
    s = SelF64()
    lib().qko_select_f64(_p(logits), logits.size, n_used, C.byref(s))
    return s


def select_f32(logits, n_used):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    s = Sel()
    lib().qko_select_f32(_p(logits), logits.size, n_used, C.byref(s))
    return s


def make_layer(h):
    """h: an object with numpy attributes named like the Layer fields (synth.HostLayer)."""
    keep = [np.ascontiguousarray(getattr(h, n)) for n in ("gate_inp", "gate_inp_shexp", "gate_exps", "up_exps",
                                                         "down_exps", "gate_shexp", "up_shexp", "down_shexp")]
    L = Layer(h.n_embd, h.n_ff, h.n_expert, h.n_used, h.gu_type, h.down_type, *[a.ctypes.data for a in keep])
    L._keep = keep
    return L


def moe_ref(h, x, want_h=False, want_logits=False):
    """Returns dict(y, sel(SelF64), h, logits) for one activation row."""
    L = make_layer(h)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(h.n_embd, dtype=np.float32)
    sel = SelF64()
    hbuf = np.empty((h.n_used + 1, h.n_ff), dtype=np.float32) if want_h else None
    lbuf = np.empty(h.n_expert, dtype=np.float64) if want_logits else None
    rc = lib().qko_moe_ref(C.byref(L), _p(x), _p(y), C.byref(sel), _p(hbuf) if want_h else None,
                           _p(lbuf) if want_logits else None)
    if rc:
        raise ValueError(f"moe_ref rc={rc}")
    return dict(y=y, sel=sel, h=hbuf, logits=lbuf)


def moe_ref_threads(h, X, threads):
    """y of the fused step for the rows of X on `threads` host threads: one row -> the row loops of
    the step are split; several rows -> the rows are (each a single-threaded step).  Bit for bit
    moe_ref()["y"]."""
    L = make_layer(h)
    X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, h.n_embd)
    Y = np.empty_like(X)
    if X.shape[0] == 1:
        rc = lib().qko_moe_ref_mt(C.byref(L), _p(X), _p(Y), threads)
    else:
        rc = lib().qko_moe_ref_tokens_mt(C.byref(L), _p(X), _p(Y), X.shape[0], threads)
    if rc:
        raise ValueError(f"moe_ref_mt rc={rc}")
    return Y


def group_pairs(sel_bytes, n_tokens, n_expert, n_used):
    """sel_bytes: uint8 [n_tokens, 160] of Sel records."""
    sel_bytes = np.ascontiguousarray(sel_bytes)
    offsets = np.empty(n_expert + 1, dtype=np.uint32)
    pairs = np.empty(n_tokens * n_used, dtype=np.uint32)
    rc = lib().qko_group_pairs(_p(sel_bytes), n_tokens, n_expert, n_used, _p(offsets), _p(pairs))
    if rc:
        raise ValueError(f"group_pairs rc={rc}")
    return offsets, pairs


def gemm_q8_0(W, X, M, K, threads=1):
    W = np.ascontiguousarray(W).reshape(-1)
    X = np.ascontiguousarray(X, dtype=np.float32)
    Y = np.empty((X.shape[0], M), dtype=np.float32)
    if threads > 1:
        rc = lib().qko_gemm_q8_0_mt(_p(W), _p(X), _p(Y), M, K, X.shape[0], threads)
    else:
        rc = lib().qko_gemm_q8_0(_p(W), _p(X), _p(Y), M, K, X.shape[0])
    if rc:
        raise ValueError(f"gemm rc={rc}")
    return Y


def max_rel_err(got, ref_):
    got = np.ascontiguousarray(got, dtype=np.float32).reshape(-1)
    ref_ = np.ascontiguousarray(ref_, dtype=np.float32).reshape(-1)
    return lib().qko_max_rel_err(_p(got), _p(ref_), got.size)


def max_err_over_rms(got, ref_):
    got = np.ascontiguousarray(got, dtype=np.float32).reshape(-1)
    ref_ = np.ascontiguousarray(ref_, dtype=np.float32).reshape(-1)
    return lib().qko_max_err_over_rms(_p(got), _p(ref_), got.size)


def rel_maxabs_err(got, ref_):
    """max|got-ref| / max|ref|: the 1e-3 bar for GEMV / MoE outputs."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref_ = np.asarray(ref_, dtype=np.float64).reshape(-1)
    den = np.max(np.abs(ref_))
    err = np.max(np.abs(got - ref_))
    if not np.isfinite(err):
        return float("inf")
    return float(err / den) if den > 0 else float(err)
