"""ctypes binding of libngpt_fp8.so.  The library is the only compute path: if it is missing
or a call fails, an exception is raised -- there is no fallback implementation."""
from __future__ import annotations

import ctypes
import pathlib
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

LIB_PATH = pathlib.Path(__file__).resolve().parent / "lib" / "libngpt_fp8.so"
# the same sources compiled with -DNGPT_BENCH_BUILD: adds the timing aids that measurements use and nothing else needs
BENCH_LIB_PATH = LIB_PATH.with_name("libngpt_fp8_bench.so")
BENCH_SIGNATURES = {
    "ngpt_bench_kstep_rate": (c_int, [c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
}

E4M3, E5M2 = 0, 1
W_OUT_IN, W_IN_OUT = 0, 1
K_CONTIGUOUS, K_ROWS = 0, 1
MAX_PREDICT = 4

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float

# name -> (restype, argtypes); mirrors include/ngpt_fp8.h declaration by declaration
SIGNATURES = {
    "ngpt_abi_version": (_I, []),
    "ngpt_last_error": (c_char_p, []),
    "ngpt_num_cus": (_I, []),
    "ngpt_profile_enable": (_I, [_I]),
    "ngpt_profile_read": (_I, [_I, _P, _P]),
    "ngpt_quant_fp8": (_I, [_P, _P, _L, _F, _I, _P]),
    "ngpt_quant_fp8_2d": (_I, [_P, _I, _I, _F, _I, _P, _P, _P]),
    "ngpt_transpose_u8": (_I, [_P, _I, _I, _P, _P]),
    "ngpt_transpose_copy": (_I, [_P, _I, _I, _P, _I, _P]),
    "ngpt_gemm_fp8_tn": (_I, [_P, _I, _L, _P, _I, _L, _I, _I, _I, _F, _P, _L, _I, _P]),
    "ngpt_gemm_fp8_scaled_workspace_bytes": (_L, [_I, _I, _I]),
    "ngpt_gemm_fp8_scaled": (_I, [_P, _I, _L, _P, _I, _L, _I, _I, _I, _P, _P, _P, _L, _P, _L, _P]),
    "ngpt_mm_fwd_workspace_bytes": (_L, [_I, _I, _I, _I]),
    "ngpt_mm_fwd": (_I, [_P, _P, _I, _I, _I, _F, _F, _P, _P, _P, _I, _P, _L, _P]),
    "ngpt_mm_bwd_workspace_bytes": (_L, [_I, _I, _I, _I]),
    "ngpt_mm_bwd": (_I, [_P, _P, _P, _I, _I, _I, _F, _F, _F, _P, _P, _I, _P, _L, _P]),
    "ngpt_fc_relu2_fwd": (_I, [_P, _P, _P, _I, _I, _I, _P, _P, _P, _P, _I, _P]),
    "ngpt_fc_relu2_fwd_workspace_bytes": (_L, [_I, _I, _I]),
    "ngpt_fc_relu2_fwd_ws": (_I, [_P, _P, _P, _I, _I, _I, _P, _P, _P, _P, _I, _P, _L, _P]),
    "ngpt_linear_relu2_bf16": (_I, [_P, _P, _I, _I, _I, _P, _P]),
    "ngpt_fc_relu2_bwd_dpre": (_I, [_P, _P, _P, _I, _I, _I, _P, _P]),
    "ngpt_gemm_bf16_workspace_bytes": (_L, [_I, _I, _I]),
    "ngpt_gemm_bf16": (_I, [_P, _I, _L, _P, _I, _L, _I, _I, _I, _P, _L, _P, _L, _P]),
    "ngpt_reduce_scales": (_I, [_P, _L, _I, _I, _F, _P, _P]),
    "ngpt_quant_transpose_down": (_I, [_P, _I, _I, _I, _L, _P, _P, _P, _P, _P]),
    "ngpt_mlp_input_quant_workspace_bytes": (_L, []),
    "ngpt_mlp_input_quant": (_I, [_P, _I, _I, _P, _P, _P, _P, _P, _L, _P]),
    "ngpt_rmsnorm_bwd": (_I, [_P, _P, _I, _I, _P, _P]),
    "ngpt_quant_up_weights_workspace_bytes": (_L, [_I]),
    "ngpt_quant_up_weights": (_I, [_P, _I, _L, _P, _P, _P, _L, _P]),
    "ngpt_transpose_add": (_I, [_P, _I, _I, _P, _I, _P]),
    "ngpt_softcap_supported": (_I, [_F, _F, _F]),
    "ngpt_ce_fwd_bwd_workspace_bytes": (_L, []),
    "ngpt_ce_fwd_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _F, _F, _F, _F, _F, _P, _L, _P]),
    "ngpt_lmhead_ce_fwd_workspace_bytes": (_L, [_I, _I, _I, _I]),
    "ngpt_lmhead_ce_fwd_min_workspace_bytes": (_L, [_I, _I, _I, _I]),
    "ngpt_lmhead_ce_fwd": (_I, [_P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _F, _F, _F, _F, _F,
                                _P, _P, _P, _P, _P, _I, _P, _L, _P]),
    "ngpt_lmhead_ce_fwd_static_max_rows": (_I, []),
    "ngpt_lmhead_ce_fwd_static": (_I, [_P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _F, _F, _F, _F, _F,
                                       _P, _P, _P, _P, _P, _I, _P]),
    "ngpt_lmhead_ce_bwd_workspace_bytes": (_L, [_I, _I, _I, _I]),
    "ngpt_lmhead_ce_bwd": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _F, _F, _F, _F,
                                _F, _F, _F, _P, _P, _I, _P, _L, _P]),
    "ngpt_lmhead_ce_codes_bytes": (_L, [_I, _I]),
    "ngpt_lmhead_ce_fwd_codes": (_I, [_P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _F, _F, _F, _F, _F,
                                      _P, _P, _P, _P, _P, _P, _I, _P, _L, _P]),
    "ngpt_lmhead_ce_bwd_codes": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _F, _F, _F, _F,
                                      _F, _F, _F, _P, _P, _I, _P, _L, _P]),
}

_lib = None
_bench_lib = None


class NgptError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the library (once) and declare every entry point; raises if it is not built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise NgptError(
                f"{LIB_PATH} is not built; run `python -m modded_nanogpt_amd.build` "
                "(there is no fallback path)")
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)          # AttributeError if the symbol is missing
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def load_bench() -> ctypes.CDLL:
    """The measurement build of the library (every entry point of the default one plus the timing aids)."""
    global _bench_lib
    if _bench_lib is None:
        if not BENCH_LIB_PATH.exists():
            raise NgptError(f"{BENCH_LIB_PATH} is not built; run `python -m modded_nanogpt_amd.build`")
        lib = ctypes.CDLL(str(BENCH_LIB_PATH))
        for name, (res, args) in {**SIGNATURES, **BENCH_SIGNATURES}.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _bench_lib = lib
    return _bench_lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().ngpt_last_error()
        raise NgptError(f"{what} failed with code {code}: {msg.decode() if msg else ''}")
