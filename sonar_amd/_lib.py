"""ctypes binding of the C ABI in include/sonar_marlin.h.

Loading fails loudly when the HIP library has not been built: there is no
fallback path."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libsonar_marlin.so")

DTYPE_F16 = 0
DTYPE_BF16 = 1
DTYPE_F32 = 2
LAYOUT_GFX950 = 0
ADTYPE_INT8 = 0
ADTYPE_FP8 = 1
TYPE_UINT4B8 = 1125899907892224
TYPE_UINT4 = 1125899906843648
TYPE_UINT8B128 = 1125899923621888
TYPE_FLOAT8_E4M3FN = 2814749767172868
TYPE_FLOAT4_E2M1F = 562949953487106

OK = 0
E_INVALID = -1
E_UNSUPPORTED = -2
E_RUNTIME = -3

# name -> (restype, argtypes); must list every symbol include/sonar_marlin.h declares
PROTOTYPES = {
    "sonar_marlin_last_error": (c_char_p, []),
    "sonar_marlin_version": (c_char_p, []),
    "sonar_marlin_last_decode_launch": (c_int, [c_void_p, c_int]),
    "sonar_debug_tile_schedule": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64]),
    "sonar_debug_moe_tile_schedule": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_int64]),
    "sonar_gptq_marlin_repack": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "sonar_awq_marlin_repack": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "sonar_marlin_to_gfx950": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_gfx950_to_marlin": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_marlin8_to_gfx950": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_gfx950_to_marlin8": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_gptq_marlin_repack_a8": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "sonar_awq_marlin_repack_a8": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "sonar_marlin_a8_to_gfx950": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_gfx950_to_marlin_a8": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_marlin_int4_fp8_preprocess": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "sonar_per_token_quant_int8": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_per_token_quant_fp8": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "sonar_marlin_gemm_a8_scratch_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "sonar_marlin_gemm_a8": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int64, c_int64, c_int64,
                                     c_int64, c_int64, c_void_p]),
    "sonar_moe_wna16_marlin_gemm_a8": (c_int, [
        c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
        c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int64, c_int, c_int64, c_int64, c_int64, c_int64,
        c_int64, c_void_p]),
    "sonar_marlin_dequant": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                     c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "sonar_marlin_gemm_scratch_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "sonar_marlin_gemm": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_size_t,
                                  c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int,
                                  c_int, c_void_p]),
    "sonar_marlin_gemm_nvfp4": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int64, c_void_p, c_size_t,
                                        c_int, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "sonar_marlin_gemm_noalloc": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                          c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int,
                                          c_int, c_void_p]),
    "sonar_moe_marlin_gemm_scratch_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "sonar_moe_wna16_marlin_gemm": (c_int, [
        c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        c_void_p, c_int64, c_void_p, c_size_t, c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
        c_int64, c_int64, c_int, c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_int64,
        c_int, c_int, c_int, c_void_p]),
    "sonar_moe_wna16_marlin_gemm_nvfp4": (c_int, [
        c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_int64,
        c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int64, c_int, c_int64, c_int64, c_int64, c_int64,
        c_void_p]),
    "sonar_moe_align_block_size": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p,
                                           c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sonar_silu_and_mul": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "sonar_moe_activation": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_float, c_float, c_float, c_int,
                                     c_void_p]),
    "sonar_moe_sum": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
}

_lib = None


class SonarMarlinError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} is missing: build it with `python -m sonar_amd.build` "
            "(hipcc --offload-arch=gfx950); there is no fallback implementation")
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != OK:
        msg = load().sonar_marlin_last_error().decode("utf-8", "replace")
        if rc == E_UNSUPPORTED:
            raise NotImplementedError(msg)
        raise SonarMarlinError(rc, msg)
