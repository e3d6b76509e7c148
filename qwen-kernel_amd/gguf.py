"""ctypes binding of include/qk_gguf.h (read-only GGUF access in libqk.so) and a small GGUF writer
for synthetic files.  Reading goes through the library; the writer is plain Python and exists so
that tests and benchmarks can build files of the reference's shape without a model download."""
import ctypes as C
import struct

import numpy as np

from . import capi

EFORMAT, ENOTFOUND, EIO = -6, -7, -8


class _Tensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("type", C.c_uint32), ("n_dims", C.c_uint32), ("ne", C.c_uint64 * 4),
                ("data", C.c_void_p), ("nbytes", C.c_uint64), ("shard", C.c_uint32), ("pad", C.c_uint32)]


class _MoeTensors(C.Structure):
    _fields_ = [("n_embd", C.c_uint32), ("n_ff", C.c_uint32), ("n_expert", C.c_uint32), ("n_used", C.c_uint32),
                ("gu_type", C.c_int32), ("down_type", C.c_int32)] + \
               [(n, _Tensor) for n in ("gate_inp", "gate_inp_shexp", "gate_exps", "up_exps", "down_exps", "gate_shexp",
                                       "up_shexp", "down_shexp")]


_bound = False


def _lib():
    global _bound
    L = capi.lib()
    if not _bound:
        vp = C.c_void_p
        L.qkg_open.restype = vp
        L.qkg_open.argtypes = [C.c_char_p]
        L.qkg_close.restype = None
        L.qkg_close.argtypes = [vp]
        L.qkg_version.restype = C.c_uint32
        L.qkg_version.argtypes = [vp]
        L.qkg_n_shards.restype = C.c_uint32
        L.qkg_n_shards.argtypes = [vp]
        L.qkg_n_tensors.restype = C.c_uint64
        L.qkg_n_tensors.argtypes = [vp]
        L.qkg_tensor_at.argtypes = [vp, C.c_uint64, C.POINTER(_Tensor)]
        L.qkg_find.argtypes = [vp, C.c_char_p, C.POINTER(_Tensor)]
        L.qkg_kv_int.argtypes = [vp, C.c_char_p, C.POINTER(C.c_uint64)]
        L.qkg_kv_str.argtypes = [vp, C.c_char_p, C.POINTER(C.c_char_p)]
        L.qkg_moe_layer.argtypes = [vp, C.c_uint32, C.POINTER(_MoeTensors)]
        _bound = True
    return L


class Tensor:
    """One entry of the tensor directory; `bytes()` is a zero-copy uint8 view of the mapping (copy it
    if it must outlive the File)."""

    def __init__(self, t, owner):
        self.name = t.name.decode()
        self.type, self.n_dims, self.ne = t.type, t.n_dims, tuple(t.ne)
        self.nbytes, self.shard = t.nbytes, t.shard
        self._addr, self._owner = t.data, owner

    def bytes(self):
        if self.nbytes == 0:
            raise capi.QkError(-3, f"tensor {self.name}: row size of type {self.type} is unknown")
        buf = (C.c_uint8 * self.nbytes).from_address(self._addr)
        a = np.frombuffer(buf, dtype=np.uint8)
        a.flags.writeable = False
        return a   # valid while the File is open


class File:
    """An open GGUF file (or split set).  Keep it alive while tensor views are in use."""

    def __init__(self, path):
        L = _lib()
        self._h = L.qkg_open(str(path).encode())
        if not self._h:
            msg = L.qkk_last_error().decode()
            code = EIO if ("mmap" in msg or "stat" in msg or ": No such" in msg or "Permission" in msg) else EFORMAT
            raise capi.QkError(code, msg)

    def close(self):
        if self._h:
            _lib().qkg_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def version(self):
        return _lib().qkg_version(self._h)

    @property
    def n_shards(self):
        return _lib().qkg_n_shards(self._h)

    def __len__(self):
        return _lib().qkg_n_tensors(self._h)

    def tensor_at(self, i):
        t = _Tensor()
        capi._check(_lib().qkg_tensor_at(self._h, i, C.byref(t)))
        return Tensor(t, self)

    def names(self):
        return [self.tensor_at(i).name for i in range(len(self))]

    def find(self, name):
        t = _Tensor()
        capi._check(_lib().qkg_find(self._h, name.encode(), C.byref(t)))
        return Tensor(t, self)

    def kv_int(self, key, default=None):
        v = C.c_uint64(0)
        rc = _lib().qkg_kv_int(self._h, key.encode(), C.byref(v))
        if rc == ENOTFOUND and default is not None:
            return default
        capi._check(rc)
        return v.value

    def kv_str(self, key, default=None):
        v = C.c_char_p()
        rc = _lib().qkg_kv_str(self._h, key.encode(), C.byref(v))
        if rc == ENOTFOUND and default is not None:
            return default
        capi._check(rc)
        return v.value.decode()

    def moe_tensors(self, layer):
        """The eight tensors of MoE layer `layer` after the library's checks: (dims dict, {name: Tensor})."""
        m = _MoeTensors()
        capi._check(_lib().qkg_moe_layer(self._h, layer, C.byref(m)))
        dims = dict(n_embd=m.n_embd, n_ff=m.n_ff, n_expert=m.n_expert, n_used=m.n_used, gu_type=m.gu_type,
                    down_type=m.down_type)
        names = ("gate_inp", "gate_inp_shexp", "gate_exps", "up_exps", "down_exps", "gate_shexp", "up_shexp",
                 "down_shexp")
        return dims, {n: Tensor(getattr(m, n), self) for n in names}

    def moe_layer(self, layer, device="cuda"):
        """Copies MoE layer `layer` to the device and returns the capi.MoeLayer the kernels take."""
        import torch
        dims, ts = self.moe_tensors(layer)
        dev = {}
        for n, t in ts.items():
            raw = torch.from_numpy(np.array(t.bytes())).to(device)   # one host copy out of the mapping, then H2D
            dev[n] = raw.view(torch.float32) if t.type == capi.F32 else raw
        return capi.MoeLayer(dims["n_embd"], dims["n_ff"], dims["n_expert"], dims["n_used"], dims["down_type"],
                             gu_type=dims["gu_type"], **dev)


# ---- writer (synthetic files) -----------------------------------------------------------------

_KV_U32, _KV_I32, _KV_F32, _KV_BOOL, _KV_STR, _KV_ARR, _KV_U64 = 4, 5, 6, 7, 8, 9, 10


def _s(b):
    b = b.encode() if isinstance(b, str) else b
    return struct.pack("<Q", len(b)) + b


def _kv(key, val):
    out = _s(key)
    if isinstance(val, bool):
        return out + struct.pack("<IB", _KV_BOOL, int(val))
    if isinstance(val, int):
        return out + (struct.pack("<II", _KV_U32, val) if 0 <= val < 2 ** 32 else struct.pack("<IQ", _KV_U64, val))
    if isinstance(val, float):
        return out + struct.pack("<If", _KV_F32, val)
    if isinstance(val, str):
        return out + struct.pack("<I", _KV_STR) + _s(val)
    if isinstance(val, (list, tuple)):   # array of strings or of u32
        if all(isinstance(v, str) for v in val):
            return out + struct.pack("<IIQ", _KV_ARR, _KV_STR, len(val)) + b"".join(_s(v) for v in val)
        return out + struct.pack("<IIQ", _KV_ARR, _KV_U32, len(val)) + b"".join(struct.pack("<I", v) for v in val)
    raise TypeError(f"{key}: unsupported value {val!r}")


def write(path, kvs, tensors, alignment=32, version=3):
    """Writes a GGUF file.  kvs: {key: int | float | bool | str | list}; tensors: list of
    (name, ggml_type, ne tuple (ne0 first), uint8 array of the tensor's bytes)."""
    kvs = dict(kvs)
    if alignment != 32:
        kvs["general.alignment"] = alignment
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(kvs)) + b"".join(_kv(k, v) for k, v in kvs.items())
    infos, off, blobs = b"", 0, []
    for name, type_, ne, data in tensors:
        data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        infos += _s(name) + struct.pack("<I", len(ne)) + b"".join(struct.pack("<Q", d) for d in ne)
        infos += struct.pack("<IQ", type_, off)
        blobs.append((off, data))
        off = (off + data.size + alignment - 1) // alignment * alignment
    start = (len(head) + len(infos) + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head + infos)
        f.write(b"\0" * (start - len(head) - len(infos)))
        for o, data in blobs:
            f.seek(start + o)
            f.write(data.tobytes())
        f.truncate(start + off if blobs else start)


def layer_tensors(hl, layer):
    """The writer's tensor list for one synth.HostLayer under the reference's names and shapes
    (reference src/main.cpp:1270-1277, 1292-1294)."""
    H, F, E = hl.n_embd, hl.n_ff, hl.n_expert
    p = f"blk.{layer}."
    return [(p + "ffn_gate_inp.weight", capi.F32, (H, E), hl.gate_inp),
            (p + "ffn_gate_inp_shexp.weight", capi.F32, (H,), hl.gate_inp_shexp),
            (p + "ffn_gate_exps.weight", hl.gu_type, (H, F, E), hl.gate_exps),
            (p + "ffn_up_exps.weight", hl.gu_type, (H, F, E), hl.up_exps),
            (p + "ffn_down_exps.weight", hl.down_type, (F, H, E), hl.down_exps),
            (p + "ffn_gate_shexp.weight", capi.Q8_0, (H, F), hl.gate_shexp),
            (p + "ffn_up_shexp.weight", capi.Q8_0, (H, F), hl.up_shexp),
            (p + "ffn_down_shexp.weight", capi.Q8_0, (F, H), hl.down_shexp)]
