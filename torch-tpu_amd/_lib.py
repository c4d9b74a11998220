"""ctypes binding of libmoe_hip.so (the C ABI declared in include/moe_hip.h).

There is no fallback: if the library is missing or a symbol is absent, importing this
module raises, and every op built on it is unavailable.
"""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmoe_hip.so")

MIN_VERSION = 200        # MOE_HIP_VERSION of include/moe_hip.h: weights are handed over tile-blocked

# name -> (restype, argtypes); the single source for both binding and the symbol test
SIGNATURES = {
    "moe_hip_version": (c_int, []),
    "moe_hip_arch": (c_char_p, []),
    "moe_hip_strerror": (c_char_p, [c_int]),
    "moe_tile_rows": (c_int, [c_int, c_int, c_int]),
    "moe_noaux_tc_topk": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "moe_route_topk": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                               c_int, c_float, c_void_p, c_void_p, c_void_p]),
    "moe_permute_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "moe_permute": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t]),
    "moe_pack_weights": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "moe_unpack_weights": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "moe_scale_pitch": (c_int, [c_int]),
    "moe_act_quant": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "moe_fused_experts_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "moe_fused_experts_fp8_rw": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_int, c_void_p, c_int, c_void_p, c_size_t]),
    "moe_fused_experts_fp8": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_int, c_void_p, c_int, c_void_p, c_size_t]),
    "moe_gemm1_swiglu": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_gemm2": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                          c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_weighted_reduce": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "moe_fused_experts_bf16_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "moe_fused_experts_bf16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                       c_void_p, c_int, c_void_p, c_int, c_void_p, c_size_t]),
    "moe_fused_experts_w8a16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                        c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_size_t]),
    "moe_layer_fp8_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "moe_layer_fp8": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                     c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_size_t]),
    "moe_set_shared_overlap": (c_int, [c_int]),
    "moe_hip_init": (c_int, []),
    "moe_static_scratch_address": (c_int, [ctypes.POINTER(c_void_p)]),
    "moe_layer_fp8_static": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                     c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "moe_router_logits_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "moe_router_logits": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_size_t]),
    "moe_mm_fp8_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "moe_mm_fp8": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_size_t]),
    "moe_mm_bf16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p]),
    "moe_mm_w8a16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "moe_mlp_fp8_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "moe_mlp_fp8": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                            c_void_p, c_void_p, c_size_t]),
}


class MoeHipError(RuntimeError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python {os.path.join(HERE, 'build.py')}` "
            "(hipcc, gfx950). There is no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is absent
        fn.restype = res
        fn.argtypes = args
    if lib.moe_hip_version() < MIN_VERSION:
        raise ImportError(f"{LIB_PATH} is version {lib.moe_hip_version()}, this package needs >= {MIN_VERSION} "
                          "(the weight layout of the GEMM entry points changed): rebuild it")
    return lib


lib = _load()


def check(rc: int, what: str):
    if rc != 0:
        raise MoeHipError(f"{what}: {lib.moe_hip_strerror(rc).decode()} (code {rc})")
