import ctypes
import pathlib
import subprocess
import sys

import numpy as np
import pytest
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_dir():
    return ROOT / "tests" / "golden"


@pytest.fixture(scope="session")
def fp8_tables(golden_dir):
    """(e4m3fn, e5m2) code tables indexed by bf16 bit pattern."""
    e4 = np.frombuffer((golden_dir / "bf16_to_e4m3fn.bin").read_bytes(), dtype=np.uint8)
    e5 = np.frombuffer((golden_dir / "bf16_to_e5m2.bin").read_bytes(), dtype=np.uint8)
    assert e4.size == 65536 and e5.size == 65536
    return e4, e5


@pytest.fixture(scope="session")
def oracle_c():
    """ctypes handle on the C part of the oracle (built on demand; CPU only)."""
    so = ROOT / "oracle" / "libngpt_oracle.so"
    src = ROOT / "oracle" / "fp8_codec.c"
    if not so.exists() or (src.exists() and src.stat().st_mtime > so.stat().st_mtime):
        subprocess.check_call(["make", "-C", str(ROOT / "oracle")])
    lib = ctypes.CDLL(str(so))
    u8, u16, f32 = ctypes.c_uint8, ctypes.c_uint16, ctypes.c_float
    for name, res, args in (
        ("ngpt_oracle_f32_to_bf16", u16, [f32]),
        ("ngpt_oracle_bf16_to_f32", f32, [u16]),
        ("ngpt_oracle_f32_to_e4m3fn", u8, [f32]),
        ("ngpt_oracle_f32_to_e5m2", u8, [f32]),
        ("ngpt_oracle_f32_to_e5m2_sat", u8, [f32]),
        ("ngpt_oracle_e4m3fn_to_f32", f32, [u8]),
        ("ngpt_oracle_e5m2_to_f32", f32, [u8]),
    ):
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    vp = ctypes.c_void_p
    lib.ngpt_oracle_quant_bf16.restype = None
    lib.ngpt_oracle_quant_bf16.argtypes = [vp, vp, ctypes.c_int64, f32, ctypes.c_int]
    lib.ngpt_oracle_encode_f32.restype = None
    lib.ngpt_oracle_encode_f32.argtypes = [vp, vp, ctypes.c_int64, ctypes.c_int]
    lib.ngpt_oracle_gemm_tn_codes.restype = None
    lib.ngpt_oracle_gemm_tn_codes.argtypes = [vp, vp, vp] + [ctypes.c_int] * 5 + [ctypes.c_double]
    lib.ngpt_oracle_mlp_input_quant.restype = None
    lib.ngpt_oracle_mlp_input_quant.argtypes = [vp, ctypes.c_int64, f32, vp, vp]
    lib.ngpt_oracle_quant_up_weights.restype = None
    lib.ngpt_oracle_quant_up_weights.argtypes = [vp, ctypes.c_int, ctypes.c_int64, vp, vp]
    return lib


@pytest.fixture(scope="session")
def oracle():
    from oracle import nanogpt_fp8_oracle
    return nanogpt_fp8_oracle


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """Frobenius-relative error ||a-b|| / ||b|| in fp64."""
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def max_rel_to_peak(a: torch.Tensor, b: torch.Tensor) -> float:
    """max |a-b| / max |b|."""
    a, b = a.double(), b.double()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-300))
