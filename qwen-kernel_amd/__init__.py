"""Host-side Python mirror of libqk.so's operator-level C ABI (include/qk_kernels.h).

The product is the shared library built from csrc/ (HIP kernels for gfx950 behind a C ABI);
this package only binds it with ctypes for the benchmark and the tests, and generates the
seeded synthetic GGUF block streams both use.  PyTorch appears only as the owner of device
memory and streams.  There is no CPU fallback: every compute call goes to the library and
raises QkError when it fails (for instance when no HIP device is present).
"""
from .capi import (  # noqa: F401
    F32, F16, Q8_0, Q6_K, IQ3_XXS, IQ4_XS, QkError, QkSel, MoeLayer, lib, lib_path, row_bytes,
    dequant, gemv, moe_decode, moe_workspace_bytes, head_argmax, head_workspace_bytes, argmax,
    moe_group_pairs, gemm_q8_0, moe_prefill, moe_prefill_workspace_bytes, device_info,
    rmsnorm, add_rmsnorm, add_rms3, vec_add, embed, moe_decode_tail, moe_layer_rows, ROWWISE_MAX,
    rope_table, attn_prep, attn_workspace_bytes, attn_decode, dn_ab, dn_conv, dn_step, dn_ab_conv,
    moe_decode_static, moe_workspace_status, gemv_norm, head_argmax_norm, dn_step_fused, MOE_STATIC_MAX_SLOTS, MOE_STATIC_BYTES,
    set_option, get_option, option,
)
from . import capi  # noqa: F401
from . import synth  # noqa: F401
from . import gguf  # noqa: F401
from . import engine  # noqa: F401
