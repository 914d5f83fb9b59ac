"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol the
header declares, the torch.library operators carry the reference's schemas, their fake
implementations reproduce shapes / dtypes / strides, and nothing computes without a GPU."""
import ctypes
import pathlib
import re

import pytest
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "ngpt_fp8.h"
E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2


@pytest.fixture(scope="module")
def amd():
    import modded_nanogpt_amd
    if not modded_nanogpt_amd._lib.LIB_PATH.exists():
        from modded_nanogpt_amd.build import build
        build(verbose=False)
    return modded_nanogpt_amd


def declared_symbols(bench_only=False):
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    bench = "".join(re.findall(r"#ifdef NGPT_BENCH_BUILD(.*?)#endif", text, flags=re.S))
    if bench_only:
        text = bench
    else:
        text = re.sub(r"#ifdef NGPT_BENCH_BUILD.*?#endif", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ngpt_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(amd):
    names = declared_symbols()
    assert len(names) >= 15
    lib = ctypes.CDLL(str(amd._lib.LIB_PATH))
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ngpt_fp8.h but not exported"
    assert sorted(amd._lib.SIGNATURES) == names, "ctypes table and header disagree"
    assert amd._lib.load().ngpt_abi_version() == 1


def test_timing_aids_are_in_the_measurement_build_only(amd):
    """The k-step microbenchmark and the discarding epilogue are measurement aids: the shipped library must not export
    or accept them; the measurement build (same sources, -DNGPT_BENCH_BUILD) has them on top."""
    aids = declared_symbols(bench_only=True)
    assert aids == sorted(amd._lib.BENCH_SIGNATURES) and "ngpt_bench_kstep_rate" in aids
    lib = ctypes.CDLL(str(amd._lib.LIB_PATH))
    for n in aids:
        assert not hasattr(lib, n), f"{n} must not be exported by the default library"
    # out_kind 3 (discard) is refused by the default build before anything is enqueued
    assert amd._lib.load().ngpt_gemm_fp8_tn(1, 0, 128, 1, 0, 128, 4, 4, 128, 1.0, 1, 4, 3, None) == -1
    if not amd._lib.BENCH_LIB_PATH.exists():
        from modded_nanogpt_amd.build import build
        build(verbose=False, bench=True)
    bench = ctypes.CDLL(str(amd._lib.BENCH_LIB_PATH))
    for n in aids + declared_symbols():
        assert hasattr(bench, n), n


def test_softcap_guard_is_host_only(amd):
    """The CE kernels' lookup tables assume that sigma no longer changes beyond |logit| = 256 and sum exponentials
    relative to the cap: constants that break this are refused (never a silently wrong loss), without a GPU."""
    lib = amd._lib.load()
    assert lib.ngpt_softcap_supported(23.0, 5.0, 7.5) == 0            # the reference's constants
    assert lib.ngpt_softcap_supported(30.0, 0.0, 7.5) == 0            # 15 * tanh(x / 15) + 15
    assert lib.ngpt_softcap_supported(23.0, 5.0, 1000.0) == -4        # sigma far from saturated at |l| = 256
    assert b"outside what the lookup tables cover" in lib.ngpt_last_error()
    assert lib.ngpt_softcap_supported(200.0, 5.0, 7.5) == -4          # exp(-A) underflows
    assert lib.ngpt_softcap_supported(23.0, 5.0, 0.0) == -4 and lib.ngpt_softcap_supported(float("nan"), 5.0, 7.5) == -4
    assert lib.ngpt_softcap_supported(23.0, -300.0, 7.5) == -4        # shifted so far that sigma(255) has not reached 1
    # the entry points apply the same check before they enqueue anything
    assert lib.ngpt_ce_fwd_bwd(1, 1, 1, None, None, 1, 1, 4, 64, 1, 23.0, 5.0, 1000.0, 1.0, 1.0, 1, 1 << 20, None) == -4


def test_argument_errors_do_not_need_a_gpu(amd):
    lib = amd._lib.load()
    assert lib.ngpt_quant_fp8(None, None, 8, 1.0, 0, None) == -1
    assert lib.ngpt_quant_fp8(1, 1, 7, 1.0, 0, None) == -2
    assert b"multiple of 8" in lib.ngpt_last_error()
    assert lib.ngpt_gemm_fp8_tn(1, 0, 100, 1, 0, 100, 4, 4, 100, 1.0, 1, 4, 0, None) == -2     # K % 128
    assert lib.ngpt_mm_bwd(1, 1, 1, 128, 128, 128, 1.0, 1.0, 1.0, 1, 1, 0, 1, 16, None) == -3   # workspace
    assert lib.ngpt_ce_fwd_bwd(1, 1, 1, None, None, 1, 1, 4, 64, 9, 23.0, 5.0, 7.5, 1.0, 1.0, 1, 1 << 20, None) == -4
    assert lib.ngpt_mm_bwd_workspace_bytes(1024, 3072, 768, 0) >= 2 * 1024 * 3072 + 768 * 1024 + 768 * 3072
    # the bf16 products of the MLP: contraction a multiple of 64, rows / columns multiples of 8 -- refused, never sent elsewhere
    assert lib.ngpt_gemm_bf16(1, 1, 768, 1, 1, 768, 768, 768, 1000, 1, 768, 1, 1 << 30, None) == -2
    assert b"K % 64" in lib.ngpt_last_error()
    assert lib.ngpt_gemm_bf16(1, 0, 64, 1, 0, 64, 12, 768, 64, 1, 768, 1, 1 << 30, None) == -2
    assert lib.ngpt_linear_relu2_bf16(1, 1, 64, 100, 64, 1, None) == -2
    assert lib.ngpt_gemm_fp8_scaled(1, 0, 128, 1, 0, 128, 64, 64, 128, None, None, 1, 64, 1, 1 << 20, None) == -1      # scales are required
    # c_fc with a workspace: same argument checks as without one, whichever kernel the workspace would select
    assert lib.ngpt_fc_relu2_fwd_ws(1, 1, None, 8192, 3072, 768, 1, None, None, None, 0, None, 0, None) == -1
    assert lib.ngpt_fc_relu2_fwd_ws(1, 1, 1, 8192, 3072, 768, 1, 1, None, None, 0, None, 0, None) == -1               # e4m3 copy without its scale
    assert lib.ngpt_fc_relu2_fwd_ws(1, 1, 1, 8192, 3000, 768, 1, None, None, None, 0, None, 0, None) == -2 and b"N=3000" in lib.ngpt_last_error()
    assert lib.ngpt_fc_relu2_fwd_workspace_bytes(8192, 3000, 768) == 0 and lib.ngpt_fc_relu2_fwd_workspace_bytes(8192, 3072, 100) == 0
    with pytest.raises(amd._lib.NgptError):
        amd._lib.check(-2, "probe")


def test_mlp_function_states_its_alignment_limits(amd):
    """FusedLinearReLUSquareFunction has no PyTorch fallback: shapes its kernels cannot take are refused with a message
    that names the limit, before any tensor is touched."""
    x = torch.zeros(1, 100, 768, dtype=torch.bfloat16, requires_grad=True)
    w1, w2 = torch.zeros(3072, 768, dtype=torch.bfloat16), torch.zeros(3072, 768, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="multiple of 8"):
        amd.ReLUSqrdMLP(x, w1, w2)
    with pytest.raises(AssertionError, match="multiples of 64"):
        amd.ReLUSqrdMLP(torch.zeros(1, 128, 100, dtype=torch.bfloat16), torch.zeros(3072, 100, dtype=torch.bfloat16), w2)


def test_operator_schemas_match_the_reference(amd):
    want = {
        "mm": "nanogpt::mm(Tensor x, Tensor w, float x_s, float w_s, float grad_s) -> (Tensor, Tensor, Tensor)",
        "mm_backward": "nanogpt::mm_backward(Tensor g, Tensor x_f8, Tensor w_f8, float x_s, float w_s, float grad_s) -> (Tensor, Tensor)",
        "mm_t": "nanogpt::mm_t(Tensor x, Tensor w, float x_s, float w_s, float grad_s) -> (Tensor, Tensor, Tensor)",
        "mm_t_backward": "nanogpt::mm_t_backward(Tensor g, Tensor x_f8, Tensor w_f8, float x_s, float w_s, float grad_s) -> (Tensor, Tensor)",
        "ce_fwd_bwd": "nanogpt::ce_fwd_bwd(Tensor logits, Tensor targets, Tensor mtp_weights, Tensor prefix_targets, "
                      "Tensor prefix_weight, Tensor(a5!) losses, Tensor(a6!) grad_input, SymInt n_rows, SymInt n_predict, "
                      "float A, float B, float C, float grad_s, float grad_scale) -> ()",
    }
    for name, schema in want.items():
        got = str(getattr(torch.ops.nanogpt, name).default._schema)
        assert got == schema, got


def test_fake_implementations_shapes_dtypes_strides(amd):
    M, N, K = 256, 384, 128
    x = torch.empty(M, K, dtype=torch.bfloat16, device="meta")
    w = torch.empty(N, K, dtype=torch.bfloat16, device="meta")
    out, x_f8, w_f8 = torch.ops.nanogpt.mm(x, w, 1.0, 1.0, 1.0)
    assert out.shape == (M, N) and out.dtype == torch.bfloat16
    assert x_f8.shape == (M, K) and x_f8.dtype == E4M3 and w_f8.shape == (N, K) and w_f8.dtype == E4M3
    g = torch.empty(M, N, dtype=torch.bfloat16, device="meta")
    dx, dw = torch.ops.nanogpt.mm_backward(g, x_f8, w_f8, 1.0, 1.0, 1.0)
    assert dx.shape == (M, K) and dx.dtype == torch.bfloat16
    assert dw.shape == (N, K) and dw.dtype == torch.float32 and dw.stride() == (1, N)
    wt = torch.empty(K, N, dtype=torch.bfloat16, device="meta")
    out, x_f8, wt_f8 = torch.ops.nanogpt.mm_t(x, wt, 1.0, 1.0, 1.0)
    assert out.shape == (M, N) and wt_f8.shape == (K, N)
    dx, dw = torch.ops.nanogpt.mm_t_backward(g, x_f8, wt_f8, 1.0, 1.0, 1.0)
    assert dw.shape == (K, N) and dw.is_contiguous()
    with pytest.raises(Exception):
        torch.ops.nanogpt.mm(x, wt, 1.0, 1.0, 1.0)          # inner dimensions differ
    t = torch.empty(M, dtype=torch.int64, device="meta")
    f1 = torch.empty(1, dtype=torch.float32, device="meta")
    losses, lse, sig, xq, wq = torch.ops.nanogpt.lmhead_ce_fwd(x, w, t, f1, t, f1, 1.0, 1.0, 23.0, 5.0, 7.5, False)
    assert losses.shape == (M,) and lse.shape == (M,) and sig.shape == (5, M) and wq.shape == (N, K)
    dx, dw = torch.ops.nanogpt.lmhead_ce_bwd(xq, wq, t, f1, t, f1, lse, sig, 1.0, 1.0, 1.0, 1.0, 23.0, 5.0, 7.5, True)
    assert dx.shape == (M, K) and dw.shape == (K, N)
    post = torch.ops.nanogpt.fc_relu2_fwd(x_f8, w_f8, f1)
    assert post.shape == (M, N) and post.dtype == torch.bfloat16


def test_autograd_contract_of_mm_under_fake_tensors(amd):
    """setup_context / backward wiring of nanogpt::mm traced with fake tensors (what dynamo does)."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        x = torch.empty(128, 256, dtype=torch.bfloat16, requires_grad=True)
        w = torch.empty(384, 256, dtype=torch.bfloat16, requires_grad=True)
        out = torch.ops.nanogpt.mm(x, w, 0.5, 0.25, 0.125)[0]
        assert out.requires_grad and out.shape == (128, 384)
        out.backward(torch.empty_like(out))
        assert x.grad.shape == x.shape and x.grad.dtype == torch.bfloat16
        assert w.grad.shape == w.shape


def test_no_cpu_fallback(amd):
    x = torch.randn(128, 128).bfloat16()
    w = torch.randn(128, 128).bfloat16()
    with pytest.raises(RuntimeError, match="GPU only"):
        torch.ops.nanogpt.mm(x, w, 1.0, 1.0, 1.0)
    with pytest.raises(RuntimeError, match="GPU only"):
        amd.quant_fp8(x, 1.0)
    with pytest.raises(RuntimeError, match="GPU only"):
        amd.FusedSoftcappedCrossEntropy.apply(x, torch.zeros(128, dtype=torch.int64), None, None, None, w,
                                              1.0, 1.0, 1.0, 1.0)


def test_package_never_imports_the_oracle():
    """The shipped package must not reference the oracle in any form."""
    for p in (ROOT / "modded-nanogpt_amd").rglob("*"):
        if p.suffix in (".py", ".hip", ".h") and p.is_file():
            assert "oracle" not in p.read_text(), p


def test_bench_uses_the_oracle_only_as_the_cpu_baseline():
    """In bench.py the oracle may be imported by the cpu_baseline* functions (the timed CPU leg) and nowhere else."""
    import ast
    tree = ast.parse((ROOT / "bench.py").read_text())
    def imports_oracle(node):
        for n in ast.walk(node):
            if isinstance(n, ast.ImportFrom) and n.module and n.module.split(".")[0] == "oracle":
                return True
            if isinstance(n, ast.Import) and any(a.name.split(".")[0] == "oracle" for a in n.names):
                return True
        return False
    for node in tree.body:
        if isinstance(node, ast.FunctionDef) and node.name.startswith("cpu_baseline"):
            assert imports_oracle(node)
        else:
            assert not imports_oracle(node), getattr(node, "name", node)


def test_shipped_gemm_kernels_do_not_spill(amd, tmp_path):
    """The 8-wave GEMM kernels must fit 256 VGPRs without spilling: one scratch reload inside the
    k-loop makes the compiler wait for all outstanding operand loads and serialises them."""
    import re
    import subprocess
    from modded_nanogpt_amd import build as b
    src = b.CSRC / "ce.hip"
    cmd = [b.hipcc_path(), *[f for f in b.HIPCC_FLAGS if f != "-shared"], "-I", str(ROOT / "include"),
           "-S", "--cuda-device-only", "-o", str(tmp_path / "ce.s"), str(src)]
    subprocess.run(cmd, check=True, capture_output=True)
    text = (tmp_path / "ce.s").read_text()
    seen = 0
    for block in text.split("- .agpr_count:")[1:]:
        name = re.search(r"\.name:\s+(\S+)", block).group(1)
        if "gemm_tn_kernel" in name and "Li256ELi256ELi4ELi2ELi128ELi2ELi1" in name:
            spills = int(re.search(r"\.vgpr_spill_count:\s+(\d+)", block).group(1))
            vgprs = int(re.search(r"\.vgpr_count:\s+(\d+)", block).group(1))
            assert spills == 0 and vgprs <= 256, (name, vgprs, spills)
            seen += 1
    assert seen >= 2          # fused CE forward + dlogits kernels
