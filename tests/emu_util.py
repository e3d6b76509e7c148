"""Test-side access to tests/emu/libqk_emu.so: the HIP kernel sources compiled as host C++ (one OS
thread per GPU thread), so that indexing and logic of the kernels can be checked on the CPU --
every tensor handed to them ends at an inaccessible page, as a device allocation can, so a read or
write behind a tensor faults in the test instead of on the GPU.  Test infrastructure only: the
product (qwen-kernel_amd/, bench.py) never loads this library."""
import contextlib
import ctypes as C
import os
import subprocess

import numpy as np

EMU_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu")
EMU_LIB = os.path.join(EMU_DIR, "libqk_emu.so")

_emu = None
plain_from_numpy = None   # set where torch.from_numpy is replaced by a copying one (the GPU tests' emu mode)


def build_emu():
    subprocess.run(["make", "-C", EMU_DIR, "-j", "8"], check=True, stdout=subprocess.DEVNULL)


def emu_lib(qk):
    """The host-side library, bound like libqk.so (built on first use if the tree holds none)."""
    global _emu
    if _emu is None:
        if not os.path.exists(EMU_LIB):
            build_emu()
        L = qk.capi.bind(C.CDLL(EMU_LIB), partial=True)
        L.emu_guard_alloc.restype = C.c_void_p
        L.emu_guard_alloc.argtypes = [C.c_size_t, C.c_size_t, C.POINTER(C.c_void_p)]
        L.emu_guard_free.argtypes = [C.c_void_p]
        L.emu_set_schedule.argtypes = [C.c_int, C.c_uint64]
        L.emu_set_schedule.restype = None
        _emu = L
    return _emu


class GuardPool:
    """Tensors in host memory whose last byte lies directly in front of a PROT_NONE page."""

    def __init__(self, qk):
        self.L = emu_lib(qk)
        self.handles = []

    def tensor(self, arr, align=16):
        """A torch CPU tensor with the contents of `arr` (numpy) in guarded memory, its start aligned to
        `align` bytes (the end is exact when the size is a multiple of that)."""
        import torch
        arr = np.ascontiguousarray(arr)
        n = arr.nbytes
        h = C.c_void_p()
        p = self.L.emu_guard_alloc(n, align, C.byref(h))
        self.handles.append(h)
        raw = np.ctypeslib.as_array((C.c_uint8 * max(n, 1)).from_address(p))[:n]
        view = raw.view(arr.dtype).reshape(arr.shape)
        view[...] = arr
        return (plain_from_numpy or torch.from_numpy)(view)

    def zeros(self, shape, dtype, align=16):
        return self.tensor(np.zeros(shape, dtype=dtype), align)

    def workspace(self, nbytes):
        """A zero-filled, 256-byte aligned workspace."""
        return self.zeros(nbytes, np.uint8, align=256)

    def close(self):
        for h in self.handles:
            self.L.emu_guard_free(h)
        self.handles = []


@contextlib.contextmanager
def emulated(qk):
    """Inside the block the ctypes wrappers of qwen-kernel_amd/capi.py call the host-side build; tensors
    are torch CPU tensors (take them from the GuardPool this yields)."""
    capi = qk.capi
    saved = (capi._lib, capi._stream)
    pool = GuardPool(qk)
    capi._lib = emu_lib(qk)
    capi._stream = lambda: C.c_void_p(0)
    try:
        yield pool
    finally:
        capi._lib, capi._stream = saved
        pool.close()


def layer_in_pool(qk, pool, hl):
    """HostLayer -> MoeLayer whose tensors live in guarded host memory."""
    t = {n: pool.tensor(getattr(hl, n)) for n in hl.NAMES}
    return qk.MoeLayer(hl.n_embd, hl.n_ff, hl.n_expert, hl.n_used, hl.down_type, gu_type=hl.gu_type, **t)
