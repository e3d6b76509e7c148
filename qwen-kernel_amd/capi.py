"""ctypes binding of include/qk_kernels.h.  Arguments are torch CUDA tensors (device
memory) or plain ints; every wrapper passes raw device pointers and the current torch
stream to the C entry point and raises QkError on a negative status."""
import ctypes as C
import os

F32, F16, Q8_0, Q6_K, IQ3_XXS, IQ4_XS = 0, 1, 8, 14, 18, 23
BLOCK = {F32: (1, 4), F16: (1, 2), Q8_0: (32, 34), Q6_K: (256, 210), IQ4_XS: (256, 136), IQ3_XXS: (256, 98)}
TYPE_NAMES = {F32: "f32", F16: "f16", Q8_0: "q8_0", Q6_K: "q6_k", IQ4_XS: "iq4_xs", IQ3_XXS: "iq3_xxs"}


class QkError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"libqk status {code}: {msg}")
        self.code = code


class QkSel(C.Structure):
    _fields_ = [("ids", C.c_uint32 * 16), ("w", C.c_float * 16), ("w_shared", C.c_float), ("pad", C.c_float * 7)]


class _Layer(C.Structure):
    _fields_ = [("n_embd", C.c_uint32), ("n_ff", C.c_uint32), ("n_expert", C.c_uint32), ("n_used", C.c_uint32),
                ("gu_type", C.c_int32), ("down_type", C.c_int32),
                ("gate_inp", C.c_void_p), ("gate_inp_shexp", C.c_void_p), ("gate_exps", C.c_void_p),
                ("up_exps", C.c_void_p), ("down_exps", C.c_void_p), ("gate_shexp", C.c_void_p),
                ("up_shexp", C.c_void_p), ("down_shexp", C.c_void_p)]


def lib_path():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "libqk.so")


_lib = None


def _signatures():
    """name -> (restype or None for int, argtypes) of every entry point the wrappers call."""
    vp, u32, u64, sz, f32, i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_size_t, C.c_float, C.c_int
    dn_conv = [vp] * 4 + [u32] * 3 + [f32, u32, vp]
    dn_step = [vp] * 6 + [u32] * 4 + [f32, u32, vp]
    attn_prep = [vp] * 10 + [u32] * 6 + [f32, vp]
    attn_decode = [vp] * 7 + [sz] + [u32] * 5 + [vp]
    return {
        "qkk_last_error": (C.c_char_p, []),
        "qkk_row_bytes": (sz, [i32, u64]),
        "qkk_moe_workspace_bytes": (sz, [vp, u32]),
        "qkk_moe_prefill_workspace_bytes": (sz, [vp, u32]),
        "qkk_head_workspace_bytes": (sz, [u32, u32]),
        "qkk_attn_workspace_bytes": (sz, [u32, u32, u32]),
        "qkk_device_info": (None, [C.c_char_p, sz, C.POINTER(u32)]),
        "qkk_set_option": (None, [C.c_char_p, i32]),
        "qkk_get_option": (None, [C.c_char_p, C.POINTER(i32)]),
        "qkk_dequant": (None, [i32, vp, vp, u64, vp]),
        "qkk_gemv": (None, [i32, vp, vp, vp, u32, u32, u32, vp]),
        "qkk_gemv_norm": (None, [i32, vp, vp, vp, f32, vp, u32, u32, u32, vp]),
        "qkk_moe_decode": (None, [vp, vp, vp, vp, vp, sz, u32, vp]),
        "qkk_moe_decode_static": (None, [vp, vp, vp, vp, u32, vp]),
        "qkk_moe_workspace_status": (None, [vp]),
        "qkk_moe_decode_stages": (None, [vp, vp, vp, vp, vp, sz, u32, u32, vp]),
        "qkk_moe_decode_tail": (None, [vp, vp, vp, vp, f32, vp, vp, vp, vp, sz, u32, vp]),
        "qkk_moe_layer_rows": (None, [vp, vp, vp, f32, vp, vp, sz, u32, vp]),
        "qkk_moe_layer_rows_add": (None, [vp, vp, vp, vp, vp, f32, vp, vp, sz, u32, vp]),
        "qkk_moe_group_pairs": (None, [vp, u32, u32, u32, vp, vp, vp]),
        "qkk_head_argmax": (None, [vp, vp, vp, vp, u32, u32, u32, vp, sz, vp]),
        "qkk_head_argmax_norm": (None, [vp, vp, vp, f32, vp, vp, u32, u32, vp, sz, vp]),
        "qkk_argmax": (None, [vp, vp, u32, u32, vp]),
        "qkk_gemm_q8_0": (None, [vp, vp, vp, u32, u32, u32, vp]),
        "qkk_moe_prefill": (None, [vp, vp, vp, vp, vp, sz, u32, vp]),
        "qkk_rmsnorm": (None, [vp, vp, vp, u32, u32, f32, vp]),
        "qkk_add_rmsnorm": (None, [vp, vp, vp, vp, vp, u32, u32, f32, vp]),
        "qkk_add_rms3": (None, [vp, vp, vp, vp, vp, vp, u32, u32, f32, vp]),
        "qkk_vec_add": (None, [vp, vp, vp, u64, vp]),
        "qkk_embed": (None, [i32, vp, u32, u32, vp, u32, u32, u32, vp, u32, vp]),
        "qkk_dn_ab": (None, [vp] * 6 + [u32] * 3 + [vp]),
        "qkk_dn_conv": (None, dn_conv),
        "qkk_dn_conv_seq": (None, dn_conv),
        "qkk_dn_step": (None, dn_step),
        "qkk_dn_step_seq": (None, dn_step),
        "qkk_dn_ab_conv": (None, [vp] * 6 + [u32, u32] + [vp] * 4 + [u32] * 3 + [f32, u32, vp]),
        "qkk_dn_step_fused": (None, [vp, vp, f32] + [vp] * 4 + [u32] + [vp] * 7 + [u32] * 4 + [f32, u32, vp]),
        "qkk_dn_ab_conv_norm": (None, [vp, vp, f32] + [vp] * 5 + [u32, u32] + [vp] * 4 + [u32] * 3 + [f32, u32, vp]),
        "qkk_rope_table": (None, [vp, u32, u32, f32]),
        "qkk_attn_prep": (None, attn_prep),
        "qkk_attn_prep_seq": (None, attn_prep),
        "qkk_attn_decode": (None, attn_decode),
        "qkk_attn_seq": (None, attn_decode),
    }


def bind(L, partial=False):
    """Declares the C signatures on a loaded library.  partial: skip entry points the library does not
    export (the tests' host-side build of some kernels)."""
    for name, (restype, argtypes) in _signatures().items():
        if partial and not hasattr(L, name):
            continue
        f = getattr(L, name)
        f.argtypes = argtypes
        if restype is not None:
            f.restype = restype
    return L


def lib():
    """Loads libqk.so from the package directory; raises if it has not been built."""
    global _lib
    if _lib is None:
        p = lib_path()
        if not os.path.exists(p):
            raise QkError(-4, f"{p} is missing: build it with `make -C qwen-kernel_amd` "
                              "(or __graft_entry__.build()); there is no fallback path")
        _lib = bind(C.CDLL(p))
    return _lib


def _check(rc):
    if rc < 0:
        raise QkError(rc, lib().qkk_last_error().decode())
    return rc


def set_option(name, value):
    """Sets one switch of the library (include/qk_kernels.h lists them), e.g. set_option("one_row", 1)."""
    _check(lib().qkk_set_option(name.encode(), int(value)))


def get_option(name):
    v = C.c_int32(0)
    _check(lib().qkk_get_option(name.encode(), C.byref(v)))
    return v.value


class option:
    """with option("one_row", 1): ...  -- a switch set for the block, its previous value afterwards."""

    def __init__(self, name, value):
        self.name, self.value = name, value

    def __enter__(self):
        self.old = get_option(self.name)
        set_option(self.name, self.value)
        return self

    def __exit__(self, *exc):
        set_option(self.name, self.old)
        return False


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def device_info():
    buf = C.create_string_buffer(64)
    ncu = C.c_uint32(0)
    n = lib().qkk_device_info(buf, 64, C.byref(ncu))
    return {"devices": n, "arch": buf.value.decode(), "cus": ncu.value}


def row_bytes(type_, k):
    return lib().qkk_row_bytes(type_, k)


def dequant(type_, W, n_elems, out=None):
    import torch
    if out is None:
        out = torch.empty(n_elems, dtype=torch.float32, device=W.device)
    _check(lib().qkk_dequant(type_, _ptr(W), _ptr(out), n_elems, _stream()))
    return out


def gemv(type_, W, X, M, K, out=None):
    """Y[b][m] = W[m] . X[b]; X is [batch, K] (or [K]) fp32 on the device."""
    import torch
    batch = 1 if X.dim() == 1 else X.shape[0]
    if out is None:
        out = torch.empty((batch, M), dtype=torch.float32, device=X.device)
    _check(lib().qkk_gemv(type_, _ptr(W), _ptr(X), _ptr(out), M, K, batch, _stream()))
    return out if X.dim() == 2 else out[0]


def gemv_norm(type_, W, X, w_norm, M, K, eps=1e-6, out=None):
    """Y[b][m] = W[m] . rmsnorm(X[b]) * w_norm, the norm applied inside the launch."""
    import torch
    batch = 1 if X.dim() == 1 else X.shape[0]
    if out is None:
        out = torch.empty((batch, M), dtype=torch.float32, device=X.device)
    _check(lib().qkk_gemv_norm(type_, _ptr(W), _ptr(X), _ptr(w_norm), eps, _ptr(out), M, K, batch, _stream()))
    return out if X.dim() == 2 else out[0]


class MoeLayer:
    """Device tensors of one MoE layer plus the C struct that names them."""

    def __init__(self, n_embd, n_ff, n_expert, n_used, down_type, gate_inp, gate_inp_shexp, gate_exps, up_exps,
                 down_exps, gate_shexp, up_shexp, down_shexp, gu_type=IQ3_XXS):
        self.tensors = dict(gate_inp=gate_inp, gate_inp_shexp=gate_inp_shexp, gate_exps=gate_exps,
                            up_exps=up_exps, down_exps=down_exps, gate_shexp=gate_shexp, up_shexp=up_shexp,
                            down_shexp=down_shexp)
        self.n_embd, self.n_ff, self.n_expert, self.n_used = n_embd, n_ff, n_expert, n_used
        self.gu_type, self.down_type = gu_type, down_type
        self.c = _Layer(n_embd, n_ff, n_expert, n_used, gu_type, down_type,
                        *[t.data_ptr() for t in (gate_inp, gate_inp_shexp, gate_exps, up_exps, down_exps,
                                                 gate_shexp, up_shexp, down_shexp)])

    def active_bytes(self, n_distinct_experts=None):
        """Weight bytes one decode step must read (reference src/main.cpp:1239-1241)."""
        u = self.n_used if n_distinct_experts is None else n_distinct_experts
        H, F = self.n_embd, self.n_ff
        per_expert = 2 * F * row_bytes(self.gu_type, H) + H * row_bytes(self.down_type, F)
        shared = 2 * F * row_bytes(Q8_0, H) + H * row_bytes(Q8_0, F)
        return self.n_expert * H * 4 + H * 4 + u * per_expert + shared


def moe_workspace_bytes(layer, n_slots):
    return lib().qkk_moe_workspace_bytes(C.byref(layer.c), n_slots)


def moe_decode(layer, X, workspace, Y=None, sel=None, stages=None):
    """Fused MoE step. X [n_slots, n_embd] fp32. Returns (Y, sel) where sel is a uint8 tensor
    [n_slots, 160] holding QkSel records.  stages: optional mask of the launches to run
    (1 route, 2 gate/up, 4 down) for per-stage timing."""
    import torch
    n = X.shape[0]
    if Y is None:
        Y = torch.empty_like(X)
    if sel is None:
        sel = torch.zeros((n, 160), dtype=torch.uint8, device=X.device)
    wsb = workspace.numel() * workspace.element_size()
    if stages is None:
        _check(lib().qkk_moe_decode(C.byref(layer.c), _ptr(X), _ptr(Y), _ptr(sel), _ptr(workspace), wsb, n,
                                    _stream()))
    else:
        _check(lib().qkk_moe_decode_stages(C.byref(layer.c), _ptr(X), _ptr(Y), _ptr(sel), _ptr(workspace), wsb,
                                           n, stages, _stream()))
    return Y, sel


MOE_STATIC_MAX_SLOTS = 16        # QKK_MOE_STATIC_MAX_SLOTS
MOE_STATIC_BYTES = 2 << 20       # QKK_MOE_STATIC_BYTES


def moe_workspace_status():
    """Waits for the current stream; raises QkError (QKK_EINVAL) if a routing launch since the last such
    call found a workspace header that was not zero."""
    _check(lib().qkk_moe_workspace_status(_stream()))


def moe_decode_static(layer, X, Y, sel):
    """qkk_moe_decode on the library's own static workspace: allocates nothing, so the caller
    passes every output (Y [n_slots, n_embd] fp32, sel uint8 [n_slots, 160])."""
    _check(lib().qkk_moe_decode_static(C.byref(layer.c), _ptr(X), _ptr(Y), _ptr(sel), X.shape[0], _stream()))
    return Y, sel


def moe_decode_tail(layer, X, resid, w_next, workspace, eps=1e-6, S=None, Xn=None, sel=None):
    """The MoE step with the layer tail: S = resid + step(X), Xn = rmsnorm(S) * w_next.
    Returns (S, Xn, sel).  S may be resid."""
    import torch
    n = X.shape[0]
    S = torch.empty_like(X) if S is None else S
    Xn = torch.empty_like(X) if Xn is None else Xn
    if sel is None:
        sel = torch.zeros((n, 160), dtype=torch.uint8, device=X.device)
    _check(lib().qkk_moe_decode_tail(C.byref(layer.c), _ptr(X), _ptr(resid), _ptr(w_next), eps, _ptr(S), _ptr(Xn),
                                     _ptr(sel), _ptr(workspace), workspace.numel() * workspace.element_size(), n,
                                     _stream()))
    return S, Xn, sel


ROWWISE_MAX = 10   # QKK_ROWWISE_MAX


def moe_layer_rows(layer, S, w_norm, workspace, eps=1e-6, sel=None, mix=None, T=None):
    """The MoE block of a layer for up to ROWWISE_MAX rows, in place: S <- S + step(rmsnorm(S) * w_norm).
    With mix (a mixer's output rows): T <- S + mix, S <- T + step(rmsnorm(T) * w_norm).
    Returns (S, sel)."""
    import torch
    n = S.shape[0]
    if sel is None:
        sel = torch.zeros((n, 160), dtype=torch.uint8, device=S.device)
    nbytes = workspace.numel() * workspace.element_size()
    if mix is None:
        _check(lib().qkk_moe_layer_rows(C.byref(layer.c), _ptr(S), _ptr(w_norm), eps, _ptr(sel), _ptr(workspace), nbytes, n,
                                        _stream()))
    else:
        if T is None:
            T = torch.empty_like(S)
        if mix.shape != S.shape or T.shape != S.shape:
            raise ValueError("moe_layer_rows: mix and T must have the shape of S")
        _check(lib().qkk_moe_layer_rows_add(C.byref(layer.c), _ptr(S), _ptr(mix), _ptr(T), _ptr(w_norm), eps, _ptr(sel),
                                            _ptr(workspace), nbytes, n, _stream()))
    return S, sel


def moe_prefill_workspace_bytes(layer, n_tokens):
    return lib().qkk_moe_prefill_workspace_bytes(C.byref(layer.c), n_tokens)


def moe_prefill(layer, X, workspace, Y=None, sel=None):
    import torch
    n = X.shape[0]
    if Y is None:
        Y = torch.empty_like(X)
    if sel is None:
        sel = torch.zeros((n, 160), dtype=torch.uint8, device=X.device)
    _check(lib().qkk_moe_prefill(C.byref(layer.c), _ptr(X), _ptr(Y), _ptr(sel), _ptr(workspace),
                                 workspace.numel() * workspace.element_size(), n, _stream()))
    return Y, sel


def moe_group_pairs(sel, n_tokens, n_expert, n_used):
    import torch
    offsets = torch.empty(n_expert + 1, dtype=torch.int32, device=sel.device)
    pairs = torch.empty(n_tokens * n_used, dtype=torch.int32, device=sel.device)
    _check(lib().qkk_moe_group_pairs(_ptr(sel), n_tokens, n_expert, n_used, _ptr(offsets), _ptr(pairs), _stream()))
    return offsets, pairs


def head_workspace_bytes(V, batch):
    return lib().qkk_head_workspace_bytes(V, batch)


def head_argmax(W, X, V, K, workspace, want_logits=False):
    import torch
    batch = X.shape[0]
    tok = torch.empty(batch, dtype=torch.int32, device=X.device)
    logits = torch.empty((batch, V), dtype=torch.float32, device=X.device) if want_logits else None
    _check(lib().qkk_head_argmax(_ptr(W), _ptr(X), _ptr(tok), _ptr(logits), V, K, batch, _ptr(workspace),
                                 workspace.numel() * workspace.element_size(), _stream()))
    return tok, logits


def head_argmax_norm(W, X, w_norm, V, K, workspace, eps=1e-6, want_logits=False):
    """The head for ONE row X [1, K] with the output norm (weights w_norm) applied inside the launch."""
    import torch
    tok = torch.empty(1, dtype=torch.int32, device=X.device)
    logits = torch.empty((1, V), dtype=torch.float32, device=X.device) if want_logits else None
    _check(lib().qkk_head_argmax_norm(_ptr(W), _ptr(X), _ptr(w_norm), eps, _ptr(tok), _ptr(logits), V, K, _ptr(workspace),
                                      workspace.numel() * workspace.element_size(), _stream()))
    return tok, logits


def argmax(logits):
    import torch
    batch, n = logits.shape
    tok = torch.empty(batch, dtype=torch.int32, device=logits.device)
    _check(lib().qkk_argmax(_ptr(logits), _ptr(tok), n, batch, _stream()))
    return tok


def gemm_q8_0(W, X, M, K, out=None):
    import torch
    N = X.shape[0]
    if out is None:
        out = torch.empty((N, M), dtype=torch.float32, device=X.device)
    _check(lib().qkk_gemm_q8_0(_ptr(W), _ptr(X), _ptr(out), M, K, N, _stream()))
    return out


def _rows(t):
    return (1, t.shape[0]) if t.dim() == 1 else (t.shape[0], t.shape[1])


def rmsnorm(x, w, eps=1e-6, out=None):
    """out = x * w / sqrt(mean(x^2) + eps) per row of x ([rows, n] or [n])."""
    import torch
    rows, n = _rows(x)
    if out is None:
        out = torch.empty_like(x)
    _check(lib().qkk_rmsnorm(_ptr(x), _ptr(w), _ptr(out), n, rows, eps, _stream()))
    return out


def add_rmsnorm(a, b, w, eps=1e-6, y=None, xn=None):
    """y = a + b; xn = rmsnorm(y) * w.  Returns (y, xn)."""
    import torch
    rows, n = _rows(a)
    y = torch.empty_like(a) if y is None else y
    xn = torch.empty_like(a) if xn is None else xn
    _check(lib().qkk_add_rmsnorm(_ptr(a), _ptr(b), _ptr(w), _ptr(y), _ptr(xn), n, rows, eps, _stream()))
    return y, xn


def add_rms3(a, b, c, w, eps=1e-6, s=None, xn=None):
    """s = (a + b) + c; xn = rmsnorm(s) * w.  Returns (s, xn)."""
    import torch
    rows, n = _rows(a)
    s = torch.empty_like(a) if s is None else s
    xn = torch.empty_like(a) if xn is None else xn
    _check(lib().qkk_add_rms3(_ptr(a), _ptr(b), _ptr(c), _ptr(w), _ptr(s), _ptr(xn), n, rows, eps, _stream()))
    return s, xn


def vec_add(a, b, out=None):
    import torch
    if out is None:
        out = torch.empty_like(a)
    _check(lib().qkk_vec_add(_ptr(a), _ptr(b), _ptr(out), a.numel(), _stream()))
    return out


def embed(type_, W, n_vocab, kdim, ids, rows, idx=0, per_req=1, out=None):
    """x[r] = dequantised row ids[idx + per_req*r] of the embedding tensor W; ids is a uint32/int32
    device tensor."""
    import torch
    if out is None:
        out = torch.empty((rows, kdim), dtype=torch.float32, device=W.device)
    _check(lib().qkk_embed(type_, _ptr(W), n_vocab, kdim, _ptr(ids), ids.numel(), idx, per_req, _ptr(out), rows,
                           _stream()))
    return out


def rope_table(tmax, n_rot, freq_base=1e7):
    """[tmax][n_rot/2][2] (cos, sin) as a float32 numpy array, computed by the library on the host."""
    import numpy as np
    out = np.empty((tmax, n_rot // 2, 2), dtype=np.float32)
    _check(lib().qkk_rope_table(out.ctypes.data_as(C.c_void_p), tmax, n_rot, freq_base))
    return out


def attn_prep(qfull, kin, vin, q_norm_w, k_norm_w, rope, slot_pos, k_cache, v_cache, n_rot, eps=1e-6, qhat=None, seq=False):
    """Head norm + RoPE + cache write for the slots' new tokens.  qfull [slots][hQ][2*dh],
    kin / vin [slots][hKV][dh], caches [slots][hKV][tmax][dh].  Returns qhat [slots][hQ][dh].
    seq: the rows are positions slot_pos[t] of ONE slot, caches [1][hKV][tmax][dh]."""
    import torch
    n, hQ, dh2 = qfull.shape
    hKV, tmax, dh = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    if qhat is None:
        qhat = torch.empty((n, hQ, dh), dtype=torch.float32, device=qfull.device)
    if k_cache.shape[0] != (1 if seq else n) or v_cache.shape != k_cache.shape:
        raise ValueError("attn_prep: caches do not match the rows")
    fn = lib().qkk_attn_prep_seq if seq else lib().qkk_attn_prep
    _check(fn(_ptr(qfull), _ptr(kin), _ptr(vin), _ptr(q_norm_w), _ptr(k_norm_w), _ptr(rope), _ptr(slot_pos), _ptr(qhat),
              _ptr(k_cache), _ptr(v_cache), n, hQ, hKV, dh, n_rot, tmax, eps, _stream()))
    return qhat


def attn_workspace_bytes(n_slots, hQ, dh=256):
    return lib().qkk_attn_workspace_bytes(n_slots, hQ, dh)


def attn_decode(qhat, k_cache, v_cache, qfull, slot_pos, workspace, att=None, seq=False):
    """Attention of the slots' new tokens over positions 0..slot_pos with the output gate.
    Returns att [slots][hQ][dh].  seq: the rows are positions of ONE slot (caches [1][hKV][tmax][dh]),
    row t attends to cache rows 0..slot_pos[t]."""
    import torch
    n, hQ, dh = qhat.shape
    hKV, tmax = k_cache.shape[1], k_cache.shape[2]
    if att is None:
        att = torch.empty_like(qhat)
    if k_cache.shape[0] != (1 if seq else n) or v_cache.shape != k_cache.shape:
        raise ValueError("attn_decode: caches do not match the rows")
    fn = lib().qkk_attn_seq if seq else lib().qkk_attn_decode
    _check(fn(_ptr(qhat), _ptr(k_cache), _ptr(v_cache), _ptr(qfull), _ptr(slot_pos), _ptr(att), _ptr(workspace),
              workspace.numel() * workspace.element_size(), n, hQ, hKV, dh, tmax, _stream()))
    return att


def dn_ab(x, alpha_w, beta_w, dt_bias, a_vec, gb=None):
    """DeltaNet log decay and write strength: gb [slots][2*hV] (g first, then beta)."""
    import torch
    n, hV = x.shape[0], alpha_w.shape[0]
    if gb is None:
        gb = torch.empty((n, 2 * hV), dtype=torch.float32, device=x.device)
    _check(lib().qkk_dn_ab(_ptr(x), _ptr(alpha_w), _ptr(beta_w), _ptr(dt_bias), _ptr(a_vec), _ptr(gb), x.shape[1], hV, n,
                           _stream()))
    return gb


def dn_ab_conv(x, alpha_w, beta_w, dt_bias, a_vec, conv_state, qkv, ker, qk_channels, d_state=128, eps=1e-6,
               w_norm=None, norm_eps=1e-6):
    """dn_ab and dn_conv in one launch.  Returns (gb [slots][2*hV], out [slots][channels]); conv_state is
    updated in place.  w_norm: x is the residual row, its RMS norm is applied inside the launch."""
    import torch
    n, hV, channels = x.shape[0], alpha_w.shape[0], qkv.shape[1]
    if qkv.shape[0] != n or conv_state.numel() != n * channels * 3:
        raise ValueError("dn_ab_conv: shapes do not match the rows")
    gb = torch.empty((n, 2 * hV), dtype=torch.float32, device=x.device)
    out = torch.empty_like(qkv)
    if w_norm is not None:
        _check(lib().qkk_dn_ab_conv_norm(_ptr(x), _ptr(w_norm), norm_eps, _ptr(alpha_w), _ptr(beta_w), _ptr(dt_bias),
                                         _ptr(a_vec), _ptr(gb), x.shape[1], hV, _ptr(conv_state), _ptr(qkv), _ptr(ker),
                                         _ptr(out), channels, d_state, qk_channels, eps, n, _stream()))
        return gb, out
    _check(lib().qkk_dn_ab_conv(_ptr(x), _ptr(alpha_w), _ptr(beta_w), _ptr(dt_bias), _ptr(a_vec), _ptr(gb), x.shape[1], hV,
                                _ptr(conv_state), _ptr(qkv), _ptr(ker), _ptr(out), channels, d_state, qk_channels, eps, n,
                                _stream()))
    return gb, out


def dn_step_fused(x, alpha_w, beta_w, dt_bias, a_vec, conv_state, qkv, ker, state, norm_w, z, hK, hV, kdiv=0, d_state=128,
                  eps=1e-6, w_norm=None, norm_eps=1e-6):
    """ab + conv + step of the slots' new tokens in one launch (two value heads per key head).  conv_state
    and state are updated in place; returns att [slots][hV * dS]."""
    import torch
    n = x.shape[0]
    att = torch.empty((n, hV * d_state), dtype=torch.float32, device=x.device)
    _check(lib().qkk_dn_step_fused(_ptr(x), _ptr(w_norm), norm_eps, _ptr(alpha_w), _ptr(beta_w), _ptr(dt_bias), _ptr(a_vec),
                                   x.shape[1], _ptr(conv_state), _ptr(qkv), _ptr(ker), _ptr(state), _ptr(norm_w), _ptr(z),
                                   _ptr(att), d_state, hK, hV, kdiv, eps, n, _stream()))
    return att


def dn_conv(conv_state, qkv, ker, qk_channels, d_state=128, eps=1e-6, out=None, seq=False):
    """Depthwise conv(4) + SiLU + window shift, q/k heads scaled to unit length.  conv_state
    [slots][channels][3] is updated in place; returns out [slots][channels].  seq: the rows are
    consecutive positions of ONE slot, conv_state [1][channels][3]."""
    import torch
    n, channels = qkv.shape
    if out is None:
        out = torch.empty_like(qkv)
    if conv_state.numel() != (1 if seq else n) * channels * 3:
        raise ValueError("dn_conv: conv_state does not match the rows")
    fn = lib().qkk_dn_conv_seq if seq else lib().qkk_dn_conv
    _check(fn(_ptr(conv_state), _ptr(qkv), _ptr(ker), _ptr(out), channels, d_state, qk_channels, eps, n, _stream()))
    return out


def dn_step(conv, gb, state, norm_w, z, hK, hV, kdiv=0, d_state=128, eps=1e-6, att=None, seq=False):
    """Gated delta-rule update of state [slots][hV][dS][dS] (column-major per head, in place) and the
    gated, normalised output att [slots][hV*dS].  seq: the rows are consecutive positions of ONE
    slot, state [1][hV][dS][dS]."""
    import torch
    n = conv.shape[0]
    if att is None:
        att = torch.empty((n, hV * d_state), dtype=torch.float32, device=conv.device)
    if state.numel() != (1 if seq else n) * hV * d_state * d_state:
        raise ValueError("dn_step: state does not match the rows")
    fn = lib().qkk_dn_step_seq if seq else lib().qkk_dn_step
    _check(fn(_ptr(conv), _ptr(gb), _ptr(state), _ptr(norm_w), _ptr(z), _ptr(att), d_state, hK, hV, kdiv, eps, n, _stream()))
    return att
