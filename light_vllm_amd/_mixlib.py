"""ctypes binding of liblvmix.so (include/lv_mixers.h): the kernels of the recurrent and windowed
sequence mixers (delta rule, windowed and latent attention), the residual streams, the gated units
and the mixture-of-experts router.

The library is separate from liblvattn.so so that a model that needs only these kernels builds
only these: `load()` compiles the sources once when no built library is there (a fresh checkout),
otherwise it loads what is built. On a GPU process a missing library is an error, never a fallback.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc", "mixers")
LIB_PATH = os.path.join(_HERE, "lib", "liblvmix.so")
SOURCES = ["mix_stream.hip", "mix_window_attn.hip", "mix_window_mfma.hip", "mix_latent.hip", "mix_moe_gemm.hip",
           "mix_sandwich.hip", "mix_parallel.hip"]
ABI_VERSION = 7

_P = c_void_p
SIGNATURES = {
    "lv_mix_abi_version": (c_int, []),
    "lv_mix_last_error": (c_char_p, []),
    "lv_hc_update_norm": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_float, c_int, _P]),
    "lv_residual_add_norm": (c_int, [_P, _P, _P, _P, c_float, _P, c_int64, c_int, c_float, c_int, _P]),
    "lv_clamped_glu": (c_int, [_P, c_int64, _P, c_int64, c_int, c_float, c_float, c_int, _P]),
    "lv_delta_prep": (c_int, [_P, c_int64, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int64,
                              c_int, c_int, c_int, c_int, c_int, c_int, _P, c_int64, c_int, c_float, c_int, _P]),
    "lv_conv_state_update": (c_int, [_P, c_int64, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P]),
    "lv_gated_delta_rule": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    "lv_head_norm_gate": (c_int, [_P, _P, c_int64, _P, _P, c_int64, c_int, c_int, c_float, c_int, c_int, _P]),
    "lv_qk_fullnorm_store": (c_int, [_P, _P, _P, c_int64, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int64,
                                     c_int, c_int, c_int, c_int, c_int, c_float, c_int, _P]),
    "lv_pool_update": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                               c_int, c_int, _P]),
    "lv_window_pool_attn": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, _P, _P, _P, _P, _P, c_int, c_int64, c_int,
                                    c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int64, c_int64, c_int, c_int, _P]),
    "lv_window_pool_attn_mfma": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                                         c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P, c_int64,
                                         c_int64, c_int64, c_int, _P]),
    "lv_latent_prep": (c_int, [_P, c_int64, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int64, c_int, c_int,
                               c_int, c_int, c_int, c_float, c_int, _P]),
    "lv_latent_q_finish": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    "lv_latent_out_gate": (c_int, [_P, _P, c_int64, c_int, _P, c_int64, c_int, c_int, c_int, _P]),
    "lv_moe_route": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, _P]),
    "lv_router_logits": (c_int, [_P, c_int64, _P, _P, c_int64, c_int, c_int, c_int, _P]),
    "lv_relu2_scale": (c_int, [_P, _P, _P, c_int64, c_int, c_int, c_int, _P]),
    "lv_moe_grouped_ff": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, _P]),
    "lv_moe_grouped_workspace_bytes": (c_int64, [c_int64, c_int, c_int, c_int, c_int]),
    "lv_moe_sort": (c_int, [_P, c_int64, c_int, c_int, _P, _P, _P, _P]),
    "lv_moe_combine": (c_int, [_P, _P, _P, _P, c_int64, c_int, c_int, _P]),
    "lv_sandwich_add_norm": (c_int, [_P, _P, _P, _P, _P, _P, c_float, _P, c_int64, c_int, c_float, c_int, _P]),
    "lv_rotary_store": (c_int, [_P, c_int64, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int64,
                                c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    "lv_polynorm": (c_int, [_P, c_int64, _P, _P, c_int64, c_int, c_float, c_int, _P]),
    "lv_expert_glu": (c_int, [_P, c_int64, _P, _P, c_int64, _P, c_int64, c_int64, c_int, c_int, c_float, c_float, c_int, _P]),
    "lv_moe_grouped_glu_ff": (c_int, [_P, _P, _P, _P, _P, c_int64, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_float,
                                      c_float, _P]),
    "lv_residual_dyt": (c_int, [_P, _P, _P, _P, _P, c_float, c_float, _P, _P, _P, _P, c_int64, c_int, c_int, _P]),
    "lv_qk_prep_store": (c_int, [_P, c_int64, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int64,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P]),
    "lv_masked_attn": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, _P, _P, _P, _P, _P, c_int, c_int64, c_int, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_int, c_int, c_float, c_int, _P, c_int64, c_int64, c_int, c_int, _P]),
    "lv_masked_attn_mfma": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, _P, c_int, _P, c_int64, c_int64,
                                    c_int64, c_int, _P]),
    "lv_lightning_attn": (c_int, [_P, c_int64, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P]),
    "lv_glu_act": (c_int, [_P, c_int64, _P, c_int64, c_int, c_int, c_int, _P]),
    "lv_moe_route_scored": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    "lv_expert_act_scale": (c_int, [_P, _P, c_int64, _P, c_int64, c_int, c_int, c_int, c_int, _P]),
    "lv_moe_grouped_act_ff": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    "lv_moe_combine_through": (c_int, [_P, _P, _P, _P, c_int64, c_int, c_int, _P, c_int, _P, _P]),
    "lv_scaled_row_add": (c_int, [_P, _P, _P, c_int64, c_int, c_int64, c_int, c_int, _P]),
}

_lib = None


def build() -> str:
    """Compile the library for gfx950 in-tree. Packed 32-bit float instructions are switched off:
    the compiler may otherwise form them from ordinary float code."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(os.path.dirname(LIB_PATH), exist_ok=True)
    root = os.path.dirname(_HERE)
    tmp = LIB_PATH + f".{os.getpid()}.tmp"
    srcs = [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           f"-I{os.path.join(root, 'include')}", f"-I{CSRC}", "-Wall", "-Wno-unused-function",
           "-shared", *srcs, "-o", tmp]
    subprocess.run(cmd, check=True, cwd=CSRC, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        try:
            build()
        except (OSError, subprocess.CalledProcessError) as exc:
            detail = getattr(exc, "stderr", b"") or b""
            raise RuntimeError(f"{LIB_PATH} is not built and building it failed: {exc}\n"
                               f"{detail.decode('utf-8', 'replace')[-2000:]}") from exc
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    got = lib.lv_mix_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"liblvmix.so ABI version {got} != expected {ABI_VERSION}; rebuild")
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().lv_mix_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed ({code}): {msg}")
