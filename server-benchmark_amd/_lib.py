"""ctypes loader for libawq_mi355x.so.  There is no fallback: if the shared object is
missing or a symbol is absent, importing callers get a loud error."""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libawq_mi355x.so")

c_int, c_void_p, c_size_t = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/awq_mi355x.h and include/awq_mi355x_dev.h one to one
SIGNATURES = {
    "awqmi_init": (c_int, []),
    "awqmi_version": (c_int, []),
    "awqmi_status_string": (ctypes.c_char_p, [c_int]),
    "awqmi_last_hip_error": (c_int, []),
    "awqmi_dequantize_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "awqmi_gemm_auto_split_k": (c_int, [c_int, c_int, c_int, c_int]),
    "awqmi_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "awqmi_gemm_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                               c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "awqmi_gemm_ld_f16": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                  c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "awqmi_dequantize_ld_f16": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                        c_void_p]),
    "awqmi_gemm_f16_noalloc": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                       c_int, c_int, c_void_p]),
    "awqmi_moe_topk_softmax_f32": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "awqmi_moe_topk_f32": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, ctypes.c_float, c_void_p,
                                   c_void_p, c_void_p]),
    "awqmi_moe_align_capacity": (c_size_t, [c_int, c_int, c_int]),
    "awqmi_moe_align": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "awqmi_moe_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "awqmi_moe_gemm_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                   c_void_p, c_size_t, c_void_p]),
    "awqmi_silu_and_mul_f16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "awqmi_moe_sum_f16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "awqmi_fused_moe_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "awqmi_fused_moe_block_rows": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "awqmi_fused_moe_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t,
                                    c_void_p]),
    "awqmi_fused_moe_routed_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                           c_int, c_int, ctypes.c_float, c_void_p, c_size_t, c_void_p]),
    "awqmi_workspace_reset": (c_int, [c_void_p, c_size_t, c_void_p]),
}
# development entry points: the call they wrap plus a trailing `variant`
for _name in ("awqmi_gemm_f16", "awqmi_moe_gemm_f16", "awqmi_fused_moe_routed_f16", "awqmi_fused_moe_block_rows"):
    _res, _args = SIGNATURES[_name]
    SIGNATURES[_name.replace("awqmi_", "awqmi_dev_", 1)] = (_res, [*_args, c_int])

SIGNATURES["awqmi_dev_last_gemm_form"] = (c_int, [])
SIGNATURES["awqmi_dev_gemm_dense_workspace_bytes"] = (c_size_t, [c_int, c_int, c_int])
SIGNATURES["awqmi_dev_stream_probe"] = (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_size_t, c_void_p])
SIGNATURES["awqmi_dev_gemm_timeline_f16"] = (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                                      c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t])
SIGNATURES["awqmi_dev_mfma_probe"] = (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p])
FORM_SKINNY, FORM_FUSED, FORM_DENSE, FORM_GENERIC = 1, 2, 3, 4   # awqmi_dev_last_gemm_form()

_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it first with `python server-benchmark_amd/build.py` "
            "(hipcc --offload-arch=gfx950); there is no CPU or eager fallback for these ops")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


STATUS_OK = 0


class AWQKernelError(RuntimeError):
    pass


def check(status: int, what: str):
    if status == STATUS_OK:
        return
    lib = load()
    msg = lib.awqmi_status_string(status).decode()
    if status == 5:
        raise AWQKernelError(f"{what}: {msg} (hipError {lib.awqmi_last_hip_error()})")
    if status in (1, 2, 4, 6, 7, 8):
        raise ValueError(f"{what}: {msg}")
    raise AWQKernelError(f"{what}: {msg}")
