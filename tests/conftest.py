import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


@pytest.fixture(scope="session")
def qk():
    return entry.load_package()


@pytest.fixture(scope="session")
def orc():
    return entry.load_oracle()


@pytest.fixture(scope="session")
def dev(qk):
    import torch
    if os.environ.get("QK_EMU") == "1":
        # The GPU tests against the host-side build of the kernels (tests/emu): tensors live in host
        # memory, the wrappers call libqk_emu.so.  For checking kernel logic where no GPU is at hand;
        # entry points that build leaves out fail with a status, not silently.
        import emu_util
        qk.capi._lib = emu_util.emu_lib(qk)
        qk.capi._stream = lambda: None
        torch.cuda.synchronize = lambda *a, **k: None
        def aligned(plain):   # workspaces must be 256-byte aligned; host allocations are 64-byte aligned
            def make(*a, **k):
                t = plain(*a, **k)
                if t.dtype == torch.uint8 and t.dim() == 1 and t.data_ptr() % 256:
                    big = plain(t.numel() + 256, dtype=torch.uint8)
                    off = (-big.data_ptr()) % 256
                    return big[off:off + t.numel()]
                return t
            return make
        torch.zeros, torch.empty = aligned(torch.zeros), aligned(torch.empty)
        # the tests upload with torch.from_numpy(a).to(dev), which copies to a device but aliases the numpy array
        # here: a kernel that updates its input in place would change the oracle's input too
        emu_util.plain_from_numpy = torch.from_numpy
        torch.from_numpy = lambda a: emu_util.plain_from_numpy(a).clone()
        print("[emu] kernels run in the host-side build", flush=True)
        return "cpu"
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    print(f"[gpu] {torch.cuda.get_device_name(0)}", flush=True)
    return "cuda:0"


SWITCHES = ("one_row", "dense_reg", "fused_norm", "attn_block", "dn_fused", "gemm_tiled", "moe_rows", "head_rows", "gemv_depth", "head_depth", "rowwise_max")
SWITCH_ENV_DEFAULTS = {"QK_ONE_ROW": "lane", "QK_DENSE_REG": "0", "QK_FUSED_NORM": "0", "QK_ATTN_BLOCK": "0", "QK_DN_FUSED": "0", "QK_GEMM_TILED": "0", "QK_MOE_ROWS": "0", "QK_HEAD_ROWS": "0"}
UNRUN = ("a form of the kernels that has not had its first supervised run on a device is reached through a switch "
         "and tested on hardware only with QK_TEST_UNRUN_FORMS=1 (the host-side build always runs it)")


def unrun_forms_allowed(dev):
    """Kernel forms written after the last run on a device: always tested in the host-side build; on a
    device only when asked for, so that an unattended run of the suite exercises the forms that have run
    there before."""
    return dev == "cpu" or os.environ.get("QK_TEST_UNRUN_FORMS") == "1"


@pytest.fixture(params=["lane", "stream"])
def one_row_form(request, qk, dev):
    """Both forms of the one-row kernels (GEMV, MoE step, LM head): block fields loaded per lane -- the
    default -- and rows streamed as 16-byte pieces through LDS (with the dense rows' x in registers)."""
    on = int(request.param == "stream")
    if on and not unrun_forms_allowed(dev):
        pytest.skip(UNRUN)
    with qk.option("one_row", on), qk.option("dense_reg", on):
        yield request.param


@pytest.fixture
def switches_back_to_defaults(qk, dev):
    """qk_open applies the QK_* switches of the environment to the library; this puts the defaults back."""
    yield
    for name in SWITCHES:
        qk.set_option(name, 0)


@pytest.fixture
def unrun_form(dev):
    """For a test of an entry point or switch whose kernels have not had their first run on a device."""
    if not unrun_forms_allowed(dev):
        pytest.skip(UNRUN)
