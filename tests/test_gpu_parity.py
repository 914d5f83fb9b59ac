"""Parity of the HIP path (through the C ABI / torch.library ops) against the CPU oracle.

Tolerances (from the path's specification):
  fp8 quantisation ............ bit-exact
  GEMM outputs ................ <= 2e-2 relative (Frobenius, and max-abs against the peak)
  per-token / mean loss ....... <= 1e-3 absolute
  e5m2 dlogits codes .......... equal except where an fp32 rounding of the gradient straddles an
                                e5m2 rounding boundary (<= 1 code apart, <= 0.1 % of elements)
"""
import math

import numpy as np
import pytest
import torch

from conftest import max_rel_to_peak, rel_err

pytestmark = pytest.mark.gpu

E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2
GEMM_TOL = 2e-2
LOSS_TOL = 1e-3


@pytest.fixture(scope="module")
def amd():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import modded_nanogpt_amd
    modded_nanogpt_amd._lib.load()          # fail loudly if the HIP library is not built
    return modded_nanogpt_amd


def dev(t):
    return t.cuda()


def assert_close_gemm(got, ref, tol=GEMM_TOL):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert got.shape == ref.shape
    assert torch.isfinite(got).all()
    assert rel_err(got, ref) <= tol, f"rel {rel_err(got, ref)}"
    assert max_rel_to_peak(got, ref) <= tol, f"peak-rel {max_rel_to_peak(got, ref)}"


def u8(t):
    return t.contiguous().view(torch.uint8).cpu()


# ------------------------------------------------------------------------------------------ quantisers
@pytest.mark.parametrize("dt,tab", [(E4M3, 0), (E5M2, 1)])
def test_quant_exhaustive_bf16(amd, fp8_tables, dt, tab):
    """All 65536 bf16 bit patterns, scale 1: the GPU quantiser equals the golden table."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.uint16)
    x = bits.view(torch.bfloat16)
    got = u8(amd.quant_fp8(dev(x), 1.0, dt)).numpy()
    want = fp8_tables[tab]
    nan = torch.isnan(x.float()).numpy()
    assert np.array_equal(got[~nan], want[~nan])
    if dt == E4M3:
        assert np.all((got[nan] & 0x7f) == 0x7f)
    else:
        assert np.all((got[nan] & 0x7f) > 0x7c)


@pytest.mark.parametrize("s", [1.0, 1 / 32, 100 / 448, 1.6 / 448, 0.75 / 448])
@pytest.mark.parametrize("dt", [E4M3, E5M2])
def test_quant_scaled_bit_exact(amd, oracle, s, dt):
    g = torch.Generator().manual_seed(21)
    x = (torch.randn(256, 384, generator=g) * (3.0 if dt == E4M3 else 1e-2)).bfloat16()
    ref = (oracle.quant_e4m3 if dt == E4M3 else oracle.quant_e5m2)(x, s)
    got = amd.quant_fp8(dev(x), s, dt)
    assert torch.equal(u8(got), u8(ref))
    rm, tr = amd.quant_fp8_2d(dev(x), s, dt)
    assert torch.equal(u8(rm), u8(ref)) and torch.equal(u8(tr), u8(ref.T.contiguous()))
    _, tr_only = amd.quant_fp8_2d(dev(x), s, dt, want_rowmajor=False)
    assert torch.equal(u8(tr_only), u8(ref.T.contiguous()))


@pytest.mark.parametrize("s", [0.99999994, 1.9999999, -0.5, 3.0e-5, 7.0e3, 1.0e-39, 2.0e38])
@pytest.mark.parametrize("dt", [E4M3, E5M2])
def test_quant_awkward_scales_all_patterns(amd, dt, s):
    """Scales for which the quantiser must leave its reciprocal-multiply path (significand all ones, negative,
    subnormal, reciprocal subnormal) or whose quotients overflow / underflow for most inputs: every bf16
    pattern against torch's own division and casts."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    ref = x.div(s).to(dt)
    got = amd.quant_fp8(dev(x), s, dt).cpu()
    r, g = u8(ref).numpy(), u8(got).numpy()
    nan = np.isnan(ref.float().numpy())
    assert np.array_equal(g[~nan], r[~nan])
    assert np.all(np.isnan(got.float().numpy()[nan]))


def test_transpose_copy_bytes(amd):
    g = torch.Generator().manual_seed(22)
    for (R, C) in [(64, 64), (16, 48), (208, 1040), (768, 1024)]:
        src = torch.randint(0, 256, (R, C), generator=g, dtype=torch.uint8).view(E5M2)
        dst = torch.empty((C, R), dtype=E5M2, device="cuda")
        amd.transpose_copy(dev(src), dst)
        assert torch.equal(u8(dst), u8(src.T.contiguous()))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32, torch.uint8])
def test_transpose_copy_wider_elements_and_ragged_shapes(amd, dt):
    """The optimizer transposes the bf16 tied embedding / lm_head weights (train_gpt.py:808-810): [768, 50304]."""
    g = torch.Generator().manual_seed(23)
    for (R, C) in [(768, 50304), (100, 36), (65, 129)]:
        src = torch.randn(R, C, generator=g).mul(40).to(dt)
        dst = torch.empty((C, R), dtype=dt, device="cuda")
        amd.transpose_copy(dev(src), dst)
        assert torch.equal(dst.cpu(), src.T.contiguous())


# ------------------------------------------------------------------------------------------ raw GEMM
@pytest.mark.parametrize("R,C,K", [(32, 32, 128), (256, 256, 256), (300, 200, 384), (1000, 520, 768), (64, 1100, 128)])
@pytest.mark.parametrize("fa,fb", [(E4M3, E4M3), (E5M2, E4M3), (E4M3, E5M2)])
def test_gemm_tn_all_formats_and_ragged_tiles(amd, R, C, K, fa, fb):
    g = torch.Generator().manual_seed(R * 7 + C)
    a = torch.randn(R, K, generator=g).to(fa)
    b = torch.randn(C, K, generator=g).to(fb)
    ref = (a.double() @ b.double().T) * 0.125
    got32 = amd.gemm_fp8_tn(dev(a), dev(b), 0.125, out_dtype=torch.float32)
    assert rel_err(got32.cpu(), ref) < 1e-4          # exact products, MFMA-internal accumulation (a little below fp32)
    got16 = amd.gemm_fp8_tn(dev(a), dev(b), 0.125, out_dtype=torch.bfloat16)
    assert_close_gemm(got16, ref, 5e-3)
    acc = got32.clone()
    amd.gemm_fp8_tn(dev(a), dev(b), 0.125, out=acc, accumulate=True)
    assert rel_err(acc.cpu(), 2 * ref) < 1e-4


def test_gemm_operand_orientation(amd):
    """A one-hot probe: element (r, c) of the result must pair row r of A with row c of B and the
    same contraction position in both (a transposed tile or a wrong k-permutation fails this)."""
    K = 256
    a = torch.zeros(96, K)
    b = torch.zeros(160, K)
    for r in range(96):
        a[r, (r * 37) % K] = 1 + (r % 5)
    for c in range(160):
        b[c, (c * 11) % K] = 2 + (c % 3)
    ref = a @ b.T
    got = amd.gemm_fp8_tn(dev(a.to(E4M3)), dev(b.to(E4M3)), 1.0, out_dtype=torch.float32).cpu()
    assert torch.equal(got, ref)


# ------------------------------------------------------------------------------------------ nanogpt::mm
def test_mm_forward_config1(amd, oracle):
    """Benchmark configuration 1: x [1024,768], W [3072,768], x_s=1, w_s=1/32, seed 0."""
    x, w, x_s, w_s = oracle.make_cfg1(seed=0)
    out_ref, xf_ref, wf_ref = oracle.mm_fwd(x, w, x_s, w_s)
    out, x_f8, w_f8 = torch.ops.nanogpt.mm(dev(x), dev(w), x_s, w_s, 1.0)
    assert out.dtype == torch.bfloat16 and x_f8.dtype == E4M3 and w_f8.dtype == E4M3
    assert torch.equal(u8(x_f8), u8(xf_ref)) and torch.equal(u8(w_f8), u8(wf_ref))
    assert_close_gemm(out, out_ref)
    # fp32 accumulation agrees with the oracle far inside one bf16 ulp, so almost every element is bit-equal
    assert (out.cpu() == out_ref).float().mean() > 0.98


@pytest.mark.parametrize("M,N,K", [(256, 384, 128), (1024, 3072, 768)])
def test_mm_backward_and_autograd(amd, oracle, M, N, K):
    x, w, _, _ = oracle.make_cfg1(seed=3, M=M, N=N, K=K)
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448
    go = (torch.randn(M, N, generator=torch.Generator().manual_seed(4)) * 1e-3).bfloat16()
    _, xf_ref, wf_ref = oracle.mm_fwd(x, w, x_s, w_s)
    dx_ref, dw_ref = oracle.mm_bwd(go, xf_ref, wf_ref, x_s, w_s, grad_s)
    dx, dw = torch.ops.nanogpt.mm_backward(dev(go), dev(xf_ref), dev(wf_ref), x_s, w_s, grad_s)
    assert dx.shape == (M, K) and dx.dtype == torch.bfloat16
    assert dw.shape == (N, K) and dw.dtype == torch.float32 and dw.stride() == (1, N)
    assert_close_gemm(dx, dx_ref)
    assert_close_gemm(dw, dw_ref)
    # the autograd contract of the op
    xg, wg = dev(x).requires_grad_(), dev(w).requires_grad_()
    out = torch.ops.nanogpt.mm(xg, wg, x_s, w_s, grad_s)[0]
    out.backward(dev(go))
    assert_close_gemm(xg.grad, dx_ref)
    assert_close_gemm(wg.grad, dw_ref)


@pytest.mark.parametrize("rem", [1, 70, 100, 200])
def test_mm_backward_remainder_tiles_split_along_the_contraction(amd, rem):
    """dx of mm_backward with 256 + rem output tiles on a 256-workgroup grid: the remainder tiles are cut
    into 4, 3, 2 or 1 jobs along the contraction and meet in fp32; dW here is 16 tiles cut 16 ways.
    Reference: the fp32 product of the same fp8 operands on the GPU."""
    M, N, K = 256 * (256 + rem), 4096, 256
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448
    gen = torch.Generator(device="cuda").manual_seed(100 + rem)
    x_f8 = torch.randn(M, K, device="cuda", generator=gen).mul_(4).to(E4M3)
    w_f8 = torch.randn(N, K, device="cuda", generator=gen).mul_(4).to(E4M3)
    go = torch.randn(M, N, device="cuda", generator=gen).mul_(1e-3).bfloat16()
    dx, dw = torch.ops.nanogpt.mm_backward(go, x_f8, w_f8, x_s, w_s, grad_s)
    g_f8 = amd.quant_fp8(go, grad_s, E5M2).float()
    dx_ref = (g_f8 @ w_f8.float()) * (grad_s * w_s)
    dw_ref = (g_f8.T @ x_f8.float()) * (x_s * grad_s)
    assert rel_err(dx.float(), dx_ref) <= 5e-3          # bf16 output
    assert rel_err(dw.float(), dw_ref) <= 1e-4          # fp32 output, fp32 partial sums
    # no tile left out or written twice: the row blocks of dx compare equally well everywhere
    blocks = (dx.float() - dx_ref).view(-1, 256, K).norm(dim=(1, 2)) / dx_ref.view(-1, 256, K).norm(dim=(1, 2))
    assert float(blocks.max()) <= 5e-3


def test_mm_t_matches_mm(amd, oracle):
    x, w, _, _ = oracle.make_cfg1(seed=5, M=512, N=640, K=256)
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448
    wt = w.T.contiguous()
    go = (torch.randn(512, 640, generator=torch.Generator().manual_seed(6)) * 1e-3).bfloat16()
    out_ref, xf_ref, wtf_ref = oracle.mm_t_fwd(x, wt, x_s, w_s)
    out, x_f8, w_f8 = torch.ops.nanogpt.mm_t(dev(x), dev(wt), x_s, w_s, grad_s)
    assert w_f8.shape == wt.shape
    assert torch.equal(u8(x_f8), u8(xf_ref)) and torch.equal(u8(w_f8), u8(wtf_ref))
    assert_close_gemm(out, out_ref)
    dx_ref, dw_ref = oracle.mm_t_bwd(go, xf_ref, wtf_ref, x_s, w_s, grad_s)
    dx, dw = torch.ops.nanogpt.mm_t_backward(dev(go), x_f8, w_f8, x_s, w_s, grad_s)
    assert dw.shape == wt.shape and dw.is_contiguous()
    assert_close_gemm(dx, dx_ref)
    assert_close_gemm(dw, dw_ref)


def test_ops_reject_cpu_tensors_and_bad_shapes(amd, oracle):
    x, w, x_s, w_s = oracle.make_cfg1(seed=0, M=64, N=64, K=128)
    with pytest.raises(RuntimeError):
        torch.ops.nanogpt.mm(x, w, x_s, w_s, 1.0)
    with pytest.raises(Exception):
        torch.ops.nanogpt.mm(dev(x), dev(w[:, :64].contiguous()), x_s, w_s, 1.0)       # inner dims differ
    with pytest.raises(Exception):
        torch.ops.nanogpt.mm(dev(x)[:, :100].contiguous(), dev(w)[:, :100].contiguous(), x_s, w_s, 1.0)  # K % 128


# ------------------------------------------------------------------------------------------ MLP
@pytest.mark.parametrize("M,D,H", [(512, 256, 768), (2048, 768, 3072)])
def test_fc_relu2_forward(amd, oracle, M, D, H):
    x, w_fc, w_proj_t = oracle.make_cfg2(seed=7, M=M, D=D, H=H)
    w_f8, scales = oracle.quantize_up_weights(w_fc[None])
    x_f8, dequant = oracle.mlp_input_quant(x, scales[0:1])
    post_ref = oracle.fc_relu2_fwd(x_f8, w_f8[0], dequant)
    post = torch.ops.nanogpt.fc_relu2_fwd(dev(x_f8), dev(w_f8[0]), dev(dequant))
    assert post.dtype == torch.bfloat16 and (post >= 0).all()
    assert_close_gemm(post, post_ref)
    assert torch.equal(post.cpu() == 0, post_ref == 0) or ((post.cpu() == 0) != (post_ref == 0)).float().mean() < 1e-4
    # whole MLP forward through the autograd function, bf16 down projection
    out_ref, _ = oracle.mlp_fwd(x[None], w_fc, w_proj_t, w_f8[0], dequant, x_f8[None])
    out = amd.ReLUSqrdMLP(dev(x[None]), dev(w_fc), dev(w_proj_t), dev(w_f8[0]), dev(dequant), dev(x_f8[None]))
    assert out.shape == (1, M, D)
    assert_close_gemm(out, out_ref)


def test_fc_relu2_emit_fp8_and_amax(amd, oracle):
    M, D, H = 1024, 256, 1024
    x, w_fc, w_proj_t = oracle.make_cfg2(seed=8, M=M, D=D, H=H)
    w_f8, scales = oracle.quantize_up_weights(w_fc[None])
    x_f8, dequant = oracle.mlp_input_quant(x, scales[0:1])
    post_ref = oracle.fc_relu2_fwd(x_f8, w_f8[0], dequant)
    act = torch.tensor([float(post_ref.float().max()) * 1.8 / 448])
    post_ref, pf8_ref, amax_ref = oracle.fc_relu2_fwd(x_f8, w_f8[0], dequant, act)
    partial = torch.full((256,), -1.0, device="cuda")
    post, post_f8 = torch.ops.nanogpt.fc_relu2_fwd_emit(dev(x_f8), dev(w_f8[0]), dev(dequant), dev(act), partial)
    assert_close_gemm(post, post_ref)
    assert (partial >= 0).all()
    assert abs(float(partial.max()) - float(amax_ref)) <= 2.0 ** -7 * float(amax_ref)
    same = (u8(post_f8) == u8(pf8_ref)).float().mean()
    assert same > 0.99                     # differs only where post differs by a bf16 ulp
    assert_close_gemm(post_f8.float().cpu() * act, pf8_ref.float() * act)


@pytest.mark.parametrize("M,K,N", [(8192, 256, 512), (8320, 768, 3072), (8192 + 48, 1024, 1024)])
def test_fc_relu2_and_mm_forward_kernels_agree(amd, M, K, N):
    """c_fc (with and without the e4m3 copy) and the mm forward on the tile kernel (no workspace) and on the
    token-stationary kernel (workspace with room for the re-ordered weights): every output byte equal.  Both kernels
    contract in ascending order with the same MFMA, so the accumulators agree bit for bit; M, K, N include a ragged
    last token tile and every supported contraction length."""
    lib = amd._lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).bfloat16().cuda()
    w = (torch.randn(N, K, generator=g) / K ** 0.5).bfloat16().cuda()
    x_f8, w_f8 = (x / 0.05).to(E4M3), (w / 0.002).to(E4M3)
    dequant = torch.tensor([0.05 * 0.002], device="cuda")
    act = torch.tensor([0.01], device="cuda")
    nws = lib.ngpt_fc_relu2_fwd_workspace_bytes(M, N, K)
    assert nws >= N * K           # these shapes are covered by the token-stationary kernel
    ws = torch.empty(nws, dtype=torch.uint8, device="cuda")
    ptr = lambda t: t.data_ptr()
    res = {}
    for which in ("tile", "stationary"):
        post = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        post_e = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        post_f8 = torch.zeros((M, N), dtype=torch.uint8, device="cuda")
        partial = torch.full((512,), -1.0, device="cuda")
        wsp, wsn = (None, 0) if which == "tile" else (ptr(ws), nws)
        print(f"c_fc {which} M={M} K={K} N={N}", flush=True)
        rc = lib.ngpt_fc_relu2_fwd_ws(ptr(x_f8), ptr(w_f8), ptr(dequant), M, N, K, ptr(post), None, None, None, 0, wsp, wsn, stream)
        assert rc == 0, lib.ngpt_last_error()
        rc = lib.ngpt_fc_relu2_fwd_ws(ptr(x_f8), ptr(w_f8), ptr(dequant), M, N, K, ptr(post_e), ptr(post_f8), ptr(act), ptr(partial), 512,
                                      wsp, wsn, stream)
        assert rc == 0, lib.ngpt_last_error()
        # mm forward from the bf16 operands
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        xq, wq = torch.zeros((M, K), dtype=torch.uint8, device="cuda"), torch.zeros((N, K), dtype=torch.uint8, device="cuda")
        nmm = lib.ngpt_mm_fwd_workspace_bytes(M, N, K, 0)
        wmm = torch.empty(max(nmm, 1), dtype=torch.uint8, device="cuda")
        print(f"mm forward {which}", flush=True)
        rc = lib.ngpt_mm_fwd(ptr(x), ptr(w), M, N, K, 0.05, 0.002, ptr(out), ptr(xq), ptr(wq), 0,
                             *((None, 0) if which == "tile" else (ptr(wmm), nmm)), stream)
        assert rc == 0, lib.ngpt_last_error()
        torch.cuda.synchronize()
        res[which] = dict(post=post, post_e=post_e, post_f8=post_f8, amax=partial.max().item(), out=out, xq=xq, wq=wq)
        assert (partial >= 0).all()
    a, b = res["tile"], res["stationary"]
    for name in ("post", "post_e", "post_f8", "out", "xq", "wq"):
        assert torch.isfinite(b[name].float()).all() and torch.equal(a[name], b[name]), name
    assert torch.equal(a["post"], a["post_e"]) and a["amax"] == b["amax"] == a["post"].float().max().item()
    assert int((a["post"] > 0).sum()) > 0.3 * M * N and int((a["post_f8"] != 0).sum()) > 0.2 * M * N


def test_mlp_backward(amd, oracle):
    M, D, H = 512, 256, 768
    x, w_fc, w_proj_t = oracle.make_cfg2(seed=9, M=M, D=D, H=H)
    dy = (torch.randn(1, M, D, generator=torch.Generator().manual_seed(10)) * 1e-3).bfloat16()
    w_f8, scales = oracle.quantize_up_weights(w_fc[None])
    x_f8, dequant = oracle.mlp_input_quant(x, scales[0:1])
    out_ref, post_ref = oracle.mlp_fwd(x[None], w_fc, w_proj_t, w_f8[0], dequant, x_f8[None])
    dx_ref, dw1_ref, dw2_ref = oracle.mlp_bwd(dy, x[None], w_fc, w_proj_t, post_ref)
    xg, w1g, w2g = dev(x[None]).requires_grad_(), dev(w_fc).requires_grad_(), dev(w_proj_t).requires_grad_()
    out = amd.ReLUSqrdMLP(xg, w1g, w2g, dev(w_f8[0]), dev(dequant), dev(x_f8[None]))
    out.backward(dev(dy))
    assert_close_gemm(xg.grad, dx_ref)
    assert_close_gemm(w1g.grad, dw1_ref)
    assert_close_gemm(w2g.grad, dw2_ref)


# ------------------------------------------------------------------------------------------ CE on logits
def _codes_close(got, ref, frac=1e-3):
    g, r = u8(got).to(torch.int16), u8(ref).to(torch.int16)
    diff = (g != r)
    assert diff.float().mean() <= frac, f"{diff.float().mean()} of codes differ"
    assert ((g - r).abs()[diff] <= 1).all()


@pytest.mark.parametrize("M,V,n_predict,prefix", [(64, 1024, 1, False), (96, 50304, 1, False), (80, 2048, 3, True),
                                                   (300, 40000, 2, True),     # more rows than workgroups, 4 + 4 register pieces
                                                   (12, 66048, 1, False),     # rows too long for the register-resident kernel
                                                   (40, 256, 4, True)])       # 4 + prefix candidates per row, colliding often
def test_ce_fwd_bwd_on_logits(amd, oracle, M, V, n_predict, prefix):
    g = torch.Generator().manual_seed(M + V)
    logits = (torch.randn(M, V, generator=g) * 4).bfloat16()
    targets = torch.randint(0, V, (M,), generator=g)
    targets[3] = -1                                       # invalid targets are skipped
    w = torch.tensor([1.0, 0.5, 0.25, 0.125][:n_predict])
    pt = torch.randint(-1, V, (M,), generator=g) if prefix else torch.full((M,), -1)
    if prefix:
        pt[5] = targets[5]                                # prefix lands on the same column as a target
    pw = torch.tensor([0.3 if prefix else 0.0])
    grad_s, grad_scale = 0.75 / 448, 1.0
    l_ref, dl_ref, _ = oracle.ce_fwd_bwd(logits, targets, w, pt, pw, M, n_predict, 23.0, 5.0, 7.5, grad_s, grad_scale)
    losses = torch.empty(M, device="cuda")
    dl = torch.empty((M, V), dtype=E5M2, device="cuda")
    torch.ops.nanogpt.ce_fwd_bwd(dev(logits), dev(targets), dev(w), dev(pt), dev(pw), losses, dl, M, n_predict,
                                 23.0, 5.0, 7.5, grad_s, grad_scale)
    assert (losses.cpu() - l_ref).abs().max() <= LOSS_TOL
    _codes_close(dl, dl_ref)
    assert_close_gemm(dl.float().cpu(), dl_ref.float())


# ------------------------------------------------------------------------------------------ fused lm_head + CE
def _fused_case(oracle, M, K, V, seed, n_predict=1, prefix=False):
    x, w, t, sc = oracle.make_cfg3(seed=seed, M=M, K=K, V=V, n_tok=V - 47)
    g = torch.Generator().manual_seed(seed + 100)
    mtp = torch.tensor([1.0, 0.5, 0.25, 0.125][:n_predict])
    pt = torch.randint(-1, V, (M,), generator=g) if prefix else None
    pw = torch.tensor([0.3]) if prefix else None
    return x, w, t, sc, mtp, pt, pw


@pytest.mark.parametrize("layout", ["out_in", "in_out"])
@pytest.mark.parametrize("M,K,V,n_predict,prefix", [
    (256, 128, 512, 1, False),         # a single tile in each direction
    (640, 256, 2432, 1, False),        # ragged tiles, 8 vocabulary splits of unequal size
    (384, 768, 5120, 3, True),         # multi-token prediction + prefix targets
    (256, 128, 1024, 4, True),         # the most candidates a row can have (4 + prefix); some collide in 1024 columns
])
def test_fused_lmhead_ce(amd, oracle, layout, M, K, V, n_predict, prefix):
    x, w, t, sc, mtp, pt, pw = _fused_case(oracle, M, K, V, seed=M + V, n_predict=n_predict, prefix=prefix)
    t[7] = -5
    wl = w if layout == "out_in" else w.T.contiguous()
    l_ref, ctx = oracle.lm_head_ce_fwd(x, t, mtp, pt, pw, wl, sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"],
                                       w_layout=layout)
    dx_ref, dw_ref = oracle.lm_head_ce_bwd(ctx)
    xg, wg = dev(x).requires_grad_(), dev(wl).requires_grad_()
    losses = amd.FusedSoftcappedCrossEntropy.apply(
        xg, dev(t), dev(mtp), None if pt is None else dev(pt), None if pw is None else dev(pw), wg,
        sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"], 23.0, 5.0, 7.5, layout)
    assert losses.shape == (M,) and losses.dtype == torch.float32
    assert abs(float(losses.detach().mean().cpu() - l_ref.mean())) <= LOSS_TOL
    # autograd wiring (the engine casts the fp32 weight gradient to the bf16 leaf's dtype)
    losses.sum().backward()
    assert xg.grad.shape == x.shape and xg.grad.dtype == torch.bfloat16 and wg.grad.shape == wl.shape
    assert_close_gemm(xg.grad, dx_ref)
    assert_close_gemm(wg.grad, dw_ref)
    # the operators themselves: dW is fp32 in the weight's own layout
    n = M
    ptd = dev(pt) if pt is not None else torch.full((n,), -1, dtype=torch.int64, device="cuda")
    pwd = dev(pw) if pw is not None else torch.zeros(1, device="cuda")
    l2, lse, sig, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(dev(x), dev(wl), dev(t), dev(mtp), ptd, pwd,
                                                               sc["x_s"], sc["w_s"], 23.0, 5.0, 7.5, layout == "in_out")
    # the autograd function's forward also wrote the sigma codes: its table entries carry the code in their low
    # mantissa bits (2^-16 relative per term, either sign), otherwise it is this same kernel
    assert (l2 - losses.detach()).abs().max().item() <= 1e-4
    # Per-token losses.  The MFMA sums a logit in another order than the oracle's matmul, so a logit that sits on a
    # bf16 rounding boundary may round the other way, which moves the bf16 sigma at a target column by one unit in
    # its last place (z by 23 * 2^-8 or less).  Nothing else may differ: every row's loss must equal the oracle's
    # once exactly that one-unit difference of the saved sigmas is accounted for, such rows must be rare, and a
    # sigma may never be more than one unit off (a wrong column or a wrong row would be).
    rows_i = torch.arange(M)
    sig_ref_all = oracle.softcap_sigma(ctx["logits"], 5.0, 7.5)
    cands = [(float(mtp[k]), torch.cat([t[k:], torch.full((k,), -1, dtype=t.dtype)])) for k in range(n_predict)]
    if pt is not None:
        cands.append((float(pw), pt))
    predicted = torch.zeros(M)
    flipped = torch.zeros(M, dtype=torch.bool)
    dlse = lse.cpu() - ctx["lse"]
    for c, (wc, tc) in enumerate(cands):
        valid = (tc >= 0) & (tc < V)
        s_ref = sig_ref_all[rows_i, tc.clamp(0, V - 1)]
        dsig = torch.where(valid, sig.cpu()[c] - s_ref, torch.zeros(()))
        ulp = torch.where(s_ref > 0, torch.exp2(torch.floor(torch.log2(s_ref.clamp_min(1e-30))) - 7), torch.zeros(()))
        assert (dsig.abs() <= ulp).all(), "a saved sigma is more than one bf16 unit from the oracle's"
        flipped |= dsig != 0
        predicted += torch.where(valid, wc * (dlse - 23.0 * dsig), torch.zeros(()))
    err = losses.detach().cpu() - l_ref
    assert (err - predicted).abs().max() <= 1e-4
    assert (err.abs() > LOSS_TOL).sum() <= flipped.sum() and flipped.float().mean() < 0.02
    assert (err[~flipped].abs() <= LOSS_TOL).all()
    assert torch.equal(u8(x_f8), u8(ctx["x_f8"]))
    assert torch.equal(u8(w_f8), u8(ctx["w_f8"] if layout == "out_in" else ctx["w_f8"].T.contiguous()))
    assert (lse.cpu() - ctx["lse"]).abs().max() < LOSS_TOL
    dx, dw = torch.ops.nanogpt.lmhead_ce_bwd(x_f8, w_f8, dev(t), dev(mtp), ptd, pwd, lse, sig, sc["x_s"], sc["w_s"],
                                             sc["grad_s"], sc["grad_scale"], 23.0, 5.0, 7.5, layout == "in_out")
    assert dw.dtype == torch.float32 and dw.shape == wl.shape and dw.is_contiguous()
    assert_close_gemm(dx, dx_ref)
    assert_close_gemm(dw, dw_ref)


@pytest.mark.parametrize("codes", [False, True])
@pytest.mark.parametrize("M,K,V,n_predict,prefix", [
    (80, 256, 640, 1, False),           # fewer tokens than one token tile
    (640, 256, 2432, 1, False),         # five token tiles, the last 256-row code block half used; 38 vocabulary units
    (384, 768, 5120, 3, True),          # multi-token prediction + prefix targets
    (1024, 512, 4096, 4, True),
    (2048, 1024, 8192, 1, False),       # the longest contraction the token slab has room for
])
def test_lmhead_ce_forward_kernels_agree(amd, oracle, M, K, V, n_predict, prefix, codes):
    """Two kernels serve the fused forward: the token-stationary one (activations resident in LDS, weights streamed
    from a fragment-ordered copy in the workspace) and the tile kernel, which a workspace of the minimum size selects.
    Same logits bit for bit, hence equal codes, sigmas and fp8 copies; the sums of exponentials are taken in a
    different order, so lse and the losses agree to rounding."""
    lib = amd._lib.load()
    x, w, t, sc, mtp, pt, pw = _fused_case(oracle, M, K, V, seed=M + V + K, n_predict=n_predict, prefix=prefix)
    t[M // 2] = -3
    xd, wd, td, mtpd = dev(x), dev(w), dev(t), dev(mtp)
    ptd = dev(pt) if pt is not None else None
    pwd = dev(pw) if pw is not None else None
    stream = torch.cuda.current_stream().cuda_stream
    ptr = lambda a: None if a is None else a.data_ptr()
    Vp, Mp = -(-V // 256) * 256, -(-M // 256) * 256

    def run(nbytes):
        o = dict(losses=torch.full((M,), float("nan"), device="cuda"), lse=torch.full((M,), float("nan"), device="cuda"),
                 sig=torch.zeros((5, M), device="cuda"), x_f8=torch.zeros((M, K), dtype=torch.uint8, device="cuda"),
                 w_f8=torch.zeros((V, K), dtype=torch.uint8, device="cuda"),
                 codes=torch.zeros(lib.ngpt_lmhead_ce_codes_bytes(M, V), dtype=torch.uint8, device="cuda"))
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        head = (ptr(xd), ptr(wd), ptr(td), ptr(mtpd), n_predict, ptr(ptd), ptr(pwd), M, K, V, sc["x_s"], sc["w_s"], 23.0, 5.0, 7.5,
                ptr(o["losses"]), ptr(o["lse"]), ptr(o["sig"]), ptr(o["x_f8"]), ptr(o["w_f8"]))
        if codes:
            rc = lib.ngpt_lmhead_ce_fwd_codes(*head, ptr(o["codes"]), 0, ptr(ws), nbytes, stream)
        else:
            rc = lib.ngpt_lmhead_ce_fwd(*head, 0, ptr(ws), nbytes, stream)
        assert rc == 0, lib.ngpt_last_error()
        torch.cuda.synchronize()
        return o

    full, least = lib.ngpt_lmhead_ce_fwd_workspace_bytes(M, K, V, 0), lib.ngpt_lmhead_ce_fwd_min_workspace_bytes(M, K, V, 0)
    assert full == least + V * K                  # this shape is one the token-stationary kernel takes
    a, b = run(full), run(least)
    for name in ("sig", "x_f8", "w_f8"):
        assert torch.equal(a[name], b[name]), name
    assert torch.isfinite(a["lse"]).all() and (a["lse"] - b["lse"]).abs().max().item() <= 1e-5
    assert (a["losses"] - b["losses"]).abs().max().item() <= 1e-5
    if codes:     # blocks [token tile][vocabulary / 128] of 256 tokens x 128 codes; tokens past M and entries past V are not defined
        ca, cb = a["codes"].view(Mp // 256, Vp // 128, 8, 256, 16), b["codes"].view(Mp // 256, Vp // 128, 8, 256, 16)
        # inside a block: [8 groups of 16 codes][256 tokens][16 codes]
        tok = (torch.arange(Mp, device="cuda").view(Mp // 256, 1, 1, 256, 1) < M)
        voc = (torch.arange(Vp // 16, device="cuda").view(1, Vp // 128, 8, 1, 1) * 16 + torch.arange(16, device="cuda").view(1, 1, 1, 1, 16)) < V
        keep = tok & voc
        assert torch.equal(ca[keep.expand_as(ca)], cb[keep.expand_as(cb)])
        assert int((ca[keep.expand_as(ca)] != 0).sum()) > 0.99 * M * V
    # and against the oracle
    l_ref, ctx = oracle.lm_head_ce_fwd(x, t, mtp, pt, pw, w, sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"], w_layout="out_in")
    assert (a["lse"].cpu() - ctx["lse"]).abs().max() < LOSS_TOL
    assert abs(float(a["losses"].mean().cpu() - l_ref.mean())) <= LOSS_TOL


@pytest.mark.parametrize("grad_scale", [3.0e5, 3.0e7])
def test_fused_lmhead_ce_gradient_saturates(amd, oracle, grad_scale):
    """Row factors large enough for the e5m2 gradient to clamp at +-57344 (the recompute kernel then takes
    its clamping epilogue for those token tiles); M = 640 also leaves half of the last token tile as padding.
    At 3e5 only part of the entries clamp, at 3e7 nearly all."""
    M, K, V = 640, 256, 2432
    x, w, t, sc, mtp, pt, pw = _fused_case(oracle, M, K, V, seed=5)
    l_ref, ctx = oracle.lm_head_ce_fwd(x, t, mtp, pt, pw, w, sc["x_s"], sc["w_s"], sc["grad_s"], grad_scale, w_layout="out_in")
    dx_ref, dw_ref = oracle.lm_head_ce_bwd(ctx)
    clamped = (ctx["dl_f8"].float().abs() == 57344.0).float().mean()
    assert clamped > (0.5 if grad_scale > 1e7 else 0.0) and (grad_scale > 1e7 or clamped < 0.5)
    ptd = torch.full((M,), -1, dtype=torch.int64, device="cuda")
    pwd = torch.zeros(1, device="cuda")
    _, lse, sig, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(dev(x), dev(w), dev(t), dev(mtp), ptd, pwd,
                                                              sc["x_s"], sc["w_s"], 23.0, 5.0, 7.5, False)
    dx, dw = torch.ops.nanogpt.lmhead_ce_bwd(x_f8, w_f8, dev(t), dev(mtp), ptd, pwd, lse, sig, sc["x_s"], sc["w_s"],
                                             sc["grad_s"], grad_scale, 23.0, 5.0, 7.5, False)
    assert torch.isfinite(dx.float()).all() and torch.isfinite(dw).all()
    assert_close_gemm(dx, dx_ref)
    assert_close_gemm(dw, dw_ref)


def _codes_case(oracle, M, K, V, seed, n_predict, prefix, below_window):
    x, w, t, sc, mtp, pt, pw = _fused_case(oracle, M, K, V, seed=seed, n_predict=n_predict, prefix=prefix)
    if below_window:
        # some vocabulary rows far below zero for the first tokens: sigma under the 255 codes' range (logits < -13);
        # a negative count puts them into the last (ragged) vocabulary tile instead of the first
        cold = slice(0, 64) if below_window > 0 else slice(V - 64, V)
        if below_window >= 10 ** 6:      # ... every vocabulary row
            cold, below_window = slice(0, V), below_window - 10 ** 6
            w[64:128] = w[64:128].abs().clamp(min=0.02)
        below_window = abs(below_window)
        w[cold] = -w[64:128].abs().repeat(-(-V // 64), 1)[: cold.stop - cold.start] * 3
        x[:below_window] = x[:below_window].abs().clamp(max=2.0) * 2
    ptd = dev(pt) if pt is not None else torch.full((M,), -1, dtype=torch.int64, device="cuda")
    pwd = dev(pw) if pw is not None else torch.zeros(1, device="cuda")
    return x, w, t, sc, mtp, ptd, pwd


@pytest.mark.parametrize("M,K,V,n_predict,prefix,in_out,below_window,grad_scale", [
    (256, 128, 512, 1, False, False, 0, 1.0),        # one tile
    (640, 256, 2432, 1, False, False, 0, 1.0),       # ragged token and vocabulary tiles (rows / columns of clamped duplicates)
    (384, 768, 5120, 3, True, True, 0, 1.0),         # multi-token prediction + prefix targets, (in, out) weight
    (512, 512, 1024, 2, False, False, 0, 1.0),       # the other two contraction lengths of the token-stationary kernels
    (640, 1024, 1536, 1, True, False, 0, 1.0),       # (K = 1024: gradient bytes stored from the registers, no LDS staging)
    (1024, 256, 2048, 1, False, False, 300, 1.0),    # sigmas below the code window in two of four token tiles, first vocabulary tile: those two tiles are recomputed
    (1024, 256, 2048, 2, True, True, 1024, 1.0),     # ... in every token tile
    (1024, 256, 2048, 1, False, False, 300, 0.01),   # ... with row factors so small that those gradients are exact zeros: nothing is recomputed
    (1024, 256, 2048, 1, False, False, 300, 0.5),    # ... around the limit between the two (some rows on either side)
    (640, 256, 2432, 1, False, False, -640, 16.0),    # ... in the last, half-filled vocabulary tile of every token tile, the last one ragged
    (1024, 256, 2048, 1, False, False, 10 ** 6 + 512, 1.0),   # ... in every vocabulary tile of half of the token tiles: the sample of
                                                              # the codes finds too many, the whole panel is recomputed instead
])
def test_lmhead_ce_backward_from_sigma_codes(amd, oracle, M, K, V, n_predict, prefix, in_out, below_window, grad_scale):
    """The backward that rebuilds the e5m2 gradient from the forward's sigma codes gives bit for bit what the
    recomputing backward gives from the same row statistics; the forward that writes the codes agrees with the plain
    one (its table entries carry the code in their low mantissa bits: relative error 2^-16 per term, either sign)."""
    x, w, t, sc, mtp, ptd, pwd = _codes_case(oracle, M, K, V, M + V + n_predict, n_predict, prefix, below_window)
    wl = w.T.contiguous() if in_out else w
    fwd = (dev(x), dev(wl), dev(t), dev(mtp), ptd, pwd, sc["x_s"], sc["w_s"], 23.0, 5.0, 7.5, in_out)
    l0, lse0, sig0, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(*fwd)
    l1, lse1, sig1, x_f8c, w_f8c, codes = torch.ops.nanogpt.lmhead_ce_fwd_codes(*fwd)
    assert torch.equal(u8(x_f8), u8(x_f8c)) and torch.equal(u8(w_f8), u8(w_f8c)) and torch.equal(sig0, sig1)
    assert (lse0 - lse1).abs().max().item() <= 2e-5 and (l0 - l1).abs().max().item() <= 1e-4
    assert codes.numel() == -(-M // 256) * 256 * (-(-V // 256) * 256)
    # code panel: blocks [token tile][vocabulary / 128] of [8 groups of 16 codes][256 tokens][16 bytes]; count zero
    # codes inside the matrix
    blocks = codes.view(-(-M // 256), -(-V // 256) * 2, 8, 256, 16)[:, : V // 128]
    valid = blocks.permute(0, 3, 1, 2, 4).reshape(-1, V)[:M]
    assert bool((valid == 0).any()) == (below_window != 0)
    bwd = (x_f8, w_f8, dev(t), dev(mtp), ptd, pwd, lse1, sig1)
    tail = (sc["x_s"], sc["w_s"], sc["grad_s"], grad_scale, 23.0, 5.0, 7.5, in_out)
    dx0, dw0 = torch.ops.nanogpt.lmhead_ce_bwd(*bwd, *tail)
    dx1, dw1 = torch.ops.nanogpt.lmhead_ce_bwd_codes(*bwd, codes, *tail)
    assert torch.isfinite(dw0).all() and dw0.abs().max() > 0
    if below_window and not prefix:
        # rows with a sigma below the window, and their factor coef * S_w * exp(A - lse) against the limit
        # 2^-17 / D(largest sigma below the window) = 1138 under which those gradients are exact zeros
        rows0 = (valid == 0).any(dim=1)
        rowf = grad_scale * (23.0 / 7.5) / sc["grad_s"] * float(mtp.sum()) * torch.exp(23.0 - lse1[rows0])
        if grad_scale == 0.01:
            assert (rowf < 1100).all()        # nothing is recomputed
        if grad_scale >= 1.0:
            assert (rowf > 1200).any()        # some tile is
    assert torch.equal(dx0, dx1) and torch.equal(dw0, dw1)


@pytest.mark.parametrize("mode", ["codes", "recompute"])
def test_lmhead_ce_backward_in_several_passes(amd, oracle, mode):
    """More than 65536 tokens: the backward works through them in passes of 65536 tokens and dW accumulates over
    the passes.  Checked against the backward of the two parts on their own (one pass each, the case every other
    test covers): a row's gradient depends on its own statistics only, so dx is the parts' dx and dW their sum."""
    M0, K, V = 65536, 256, 512
    M = M0 + 512
    x, w, t, sc, mtp, ptd, pwd = _codes_case(oracle, M, K, V, 77, 1, False, 0)
    fwd = (dev(x), dev(w), dev(t), dev(mtp), ptd, pwd, sc["x_s"], sc["w_s"], 23.0, 5.0, 7.5, False)
    tail = (sc["x_s"], sc["w_s"], sc["grad_s"], 1.0, 23.0, 5.0, 7.5, False)
    if mode == "codes":
        _, lse, sig, x_f8, w_f8, codes = torch.ops.nanogpt.lmhead_ce_fwd_codes(*fwd)
        run = lambda lo, hi, cd: torch.ops.nanogpt.lmhead_ce_bwd_codes(x_f8[lo:hi], w_f8, dev(t)[lo:hi], dev(mtp), ptd[lo:hi], pwd, lse[lo:hi],
                                                                        sig[:, lo:hi].contiguous(), cd, *tail)
        # the code panel is made of blocks of 256 tokens, M0 is a multiple of 256: the parts' panels are slices of it
        per_tile = codes.numel() // (-(-M // 256))
        dx, dw = run(0, M, codes)
        dx_a, dw_a = run(0, M0, codes[: per_tile * (M0 // 256)])
        dx_b, dw_b = run(M0, M, codes[per_tile * (M0 // 256):])
    else:
        _, lse, sig, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(*fwd)
        run = lambda lo, hi: torch.ops.nanogpt.lmhead_ce_bwd(x_f8[lo:hi], w_f8, dev(t)[lo:hi], dev(mtp), ptd[lo:hi], pwd, lse[lo:hi],
                                                             sig[:, lo:hi].contiguous(), *tail)
        dx, dw = run(0, M)
        dx_a, dw_a = run(0, M0)
        dx_b, dw_b = run(M0, M)
    assert torch.isfinite(dx.float()).all() and torch.isfinite(dw).all() and dw.abs().max() > 0
    # the last token of a part has no successor inside the part: with n_predict = 1 the target of row m is targets[m] alone,
    # so the parts see exactly the rows' own targets
    assert_close_gemm(dx[:M0], dx_a, tol=2e-3)
    assert_close_gemm(dx[M0:], dx_b, tol=2e-3)
    assert_close_gemm(dw, dw_a + dw_b, tol=2e-3)


def test_fused_lmhead_ce_backward_modes(amd, oracle, monkeypatch):
    """FusedSoftcappedCrossEntropy in both settings of fused.CE_BACKWARD against the oracle."""
    M, K, V = 512, 256, 3072
    x, w, t, sc, mtp, pt, pw = _fused_case(oracle, M, K, V, seed=321, n_predict=2, prefix=True)
    l_ref, ctx = oracle.lm_head_ce_fwd(x, t, mtp, pt, pw, w, sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"], w_layout="out_in")
    dx_ref, dw_ref = oracle.lm_head_ce_bwd(ctx)
    grads = {}
    for mode in ("codes", "recompute"):
        monkeypatch.setattr(amd.fused, "CE_BACKWARD", mode)
        xg, wg = dev(x).requires_grad_(), dev(w).float().requires_grad_()
        losses = amd.FusedSoftcappedCrossEntropy.apply(xg, dev(t), dev(mtp), dev(pt), dev(pw), wg.bfloat16(), sc["x_s"], sc["w_s"],
                                                       sc["grad_s"], sc["grad_scale"], 23.0, 5.0, 7.5, "out_in")
        assert abs(float(losses.detach().mean().cpu() - l_ref.mean())) <= LOSS_TOL
        losses.sum().backward()
        assert_close_gemm(xg.grad, dx_ref)
        assert_close_gemm(wg.grad, dw_ref)
        grads[mode] = (xg.grad.clone(), wg.grad.clone())
    # the two modes differ only through the last bits of lse (sum of exponentials), i.e. in a few e5m2 roundings
    assert_close_gemm(grads["codes"][0], grads["recompute"][0], tol=2e-3)
    assert_close_gemm(grads["codes"][1], grads["recompute"][1], tol=2e-3)


def test_fused_lmhead_ce_reduces_to_cross_entropy(amd, oracle):
    """Independent of the oracle's kernel restatement: n_predict = 1, no prefix => the closed form
    F.cross_entropy(23*sigmoid((l+5)/7.5)) on the dequantised operands."""
    M, K, V = 512, 256, 3072
    x, w, t, sc, *_ = _fused_case(oracle, M, K, V, seed=77)
    losses = amd.FusedSoftcappedCrossEntropy.apply(dev(x), dev(t), None, None, None, dev(w), sc["x_s"], sc["w_s"],
                                                   sc["grad_s"], sc["grad_scale"], 23.0, 5.0, 7.5, "out_in")
    xq = oracle.quant_e4m3(x, sc["x_s"]).double() * sc["x_s"]
    wq = oracle.quant_e4m3(w, sc["w_s"]).double() * sc["w_s"]
    ref = oracle.softcap_ce_closed_form((xq @ wq.T).float(), t)
    assert abs(float(losses.mean().cpu() - ref.mean())) < 5e-3
    assert (losses.cpu() - ref).abs().max() < 0.15


@pytest.mark.parametrize("A,B,C", [(30.0, 0.0, 7.5), (15.0, -2.0, 5.0)])
def test_softcap_constants_other_than_the_defaults(amd, oracle, A, B, C):
    """The lookup tables are built from the A, B, C of the call: 30 * sigmoid(l / 7.5) is the 15 * tanh(l / 15) + 15
    form that train_gpt.py:1683-1684 describes.  Both CE paths against the oracle, logits up to |l| ~ 40."""
    assert amd._lib.load().ngpt_softcap_supported(A, B, C) == 0
    M, V = 96, 4096
    g = torch.Generator().manual_seed(41)
    logits = (torch.randn(M, V, generator=g) * 10).bfloat16()
    targets = torch.randint(0, V, (M,), generator=g)
    w, pt, pw = torch.tensor([1.0, 0.5]), torch.randint(-1, V, (M,), generator=g), torch.tensor([0.25])
    grad_s, grad_scale = 0.75 / 448, 1.0
    l_ref, dl_ref, _ = oracle.ce_fwd_bwd(logits, targets, w, pt, pw, M, 2, A, B, C, grad_s, grad_scale)
    losses = torch.empty(M, device="cuda")
    dl = torch.empty((M, V), dtype=E5M2, device="cuda")
    torch.ops.nanogpt.ce_fwd_bwd(dev(logits), dev(targets), dev(w), dev(pt), dev(pw), losses, dl, M, 2, A, B, C, grad_s, grad_scale)
    assert (losses.cpu() - l_ref).abs().max() <= LOSS_TOL
    _codes_close(dl, dl_ref)
    # fused path
    Mf, K, Vf = 384, 256, 2432
    x, wt, t, sc, mtp, ptf, pwf = _fused_case(oracle, Mf, K, Vf, seed=43)
    l_ref, ctx = oracle.lm_head_ce_fwd(x, t, mtp, ptf, pwf, wt, sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"], A, B, C, "out_in")
    dx_ref, dw_ref = oracle.lm_head_ce_bwd(ctx)
    xg, wg = dev(x).requires_grad_(), dev(wt).requires_grad_()
    lf = amd.FusedSoftcappedCrossEntropy.apply(xg, dev(t), None, None, None, wg, sc["x_s"], sc["w_s"], sc["grad_s"],
                                               sc["grad_scale"], A, B, C, "out_in")
    lf.sum().backward()
    assert abs(float(lf.detach().mean().cpu() - l_ref.mean())) <= LOSS_TOL
    assert_close_gemm(xg.grad, dx_ref)
    assert_close_gemm(wg.grad, dw_ref)


def test_softcap_constants_outside_the_tables_are_refused(amd):
    """C = 1000 leaves sigma far from saturated at |logit| = 256: an error, not a wrong loss."""
    M, V = 16, 256
    logits = torch.zeros(M, V, dtype=torch.bfloat16, device="cuda")
    t = torch.zeros(M, dtype=torch.int64, device="cuda")
    losses, dl = torch.empty(M, device="cuda"), torch.empty((M, V), dtype=E5M2, device="cuda")
    one, pw = torch.ones(1, device="cuda"), torch.zeros(1, device="cuda")
    with pytest.raises(RuntimeError, match="lookup tables"):
        torch.ops.nanogpt.ce_fwd_bwd(logits, t, one, t, pw, losses, dl, M, 1, 23.0, 5.0, 1000.0, 1.0, 1.0)
    x = torch.zeros(128, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="lookup tables"):
        amd.FusedSoftcappedCrossEntropy.apply(x, torch.zeros(128, dtype=torch.int64, device="cuda"), None, None, None, x,
                                              1.0, 1.0, 1.0, 1.0, 200.0, 5.0, 7.5)


# ------------------------------------------------------------------------------------------ delayed-scaling helpers
def test_reduce_scales_and_down_weight_requantiser(amd, oracle):
    g = torch.Generator().manual_seed(31)
    L, H, D = 3, 3072, 768
    bank = (torch.randn(L, 2, H, D, generator=g) * 0.02).bfloat16()
    w = bank[:, 1]                                                  # strided view, as the reference passes it
    scales = w.float().abs().amax(dim=(1, 2)) / 448 * torch.tensor([1.0, 0.9, 1.3])
    q_ref, used_ref, next_ref, partial_ref = oracle.quantize_transpose_mlp_down_weights(w, scales, headroom=1.12)
    bank_d = dev(bank)
    out = torch.empty((L, D, H), dtype=E4M3, device="cuda")
    nxt, used = dev(scales.clone()), torch.zeros(L, device="cuda")
    partial = torch.empty((L, (H // 64) * (D // 64)), device="cuda")
    amd.quantize_transpose_mlp_down_weights(bank_d[:, 1], out, nxt, used, partial, headroom=1.12)
    assert torch.equal(u8(out), u8(q_ref))                          # bit-exact, clamped at +-448
    assert torch.equal(used.cpu(), used_ref) and torch.equal(partial.cpu(), partial_ref)
    assert torch.allclose(nxt.cpu(), next_ref, rtol=1e-6)
    p = torch.rand(11, 256, generator=g)
    p[3] = 0
    s = torch.zeros(12, device="cuda")
    amd.reduce_mlp_activation_scales(dev(p), s, headroom=1.80)
    assert torch.allclose(s[:11].cpu(), oracle.reduce_mlp_activation_scales(p, 1.80), rtol=1e-6) and s[11] == 0


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_transpose_add(amd, dt):
    g = torch.Generator().manual_seed(32)
    for (M, N) in [(64, 64), (100, 36), (768, 1000)]:
        src = torch.randn(M, N, generator=g).to(dt)
        dst = torch.randn(N, M, generator=g).to(dt)
        want = (dst.float() + src.float().T).to(dt)
        d = dev(dst)
        amd.transpose_add(dev(src), d)
        assert torch.equal(d.cpu(), want)


def test_mlp_forward_with_fp8_down_projection(amd, oracle):
    """FusedLinearReLUSquareFunction with W2_f8: EMIT_FP8 epilogue + FP8 down projection (record #89 path)."""
    M, D, H = 1024, 256, 1024
    x, w_fc, w_proj_t = oracle.make_cfg2(seed=33, M=M, D=D, H=H)
    w_f8, scales = oracle.quantize_up_weights(w_fc[None])
    x_f8, dequant = oracle.mlp_input_quant(x, scales[0:1])
    post_ref = oracle.fc_relu2_fwd(x_f8, w_f8[0], dequant)
    act = torch.tensor([float(post_ref.float().max()) * 1.8 / 448])
    w2_scale = w_proj_t.float().abs().max().reshape(1) / 448
    w2q_t, _, _, _ = oracle.quantize_transpose_mlp_down_weights(w_proj_t[None], w2_scale)     # [1, D, H]
    w2_f8 = w2q_t[0].T                                                                        # (H, D) view, H contiguous
    out_ref, _, _ = oracle.mlp_fwd(x[None], w_fc, w_proj_t, w_f8[0], dequant, x_f8[None], w2_f8, w2_scale, act)
    partial = torch.zeros(256, device="cuda")
    out = amd.ReLUSqrdMLP(dev(x[None]), dev(w_fc), dev(w_proj_t), dev(w_f8[0]), dev(dequant), dev(x_f8[None]),
                          dev(w2q_t)[0].T, dev(w2_scale), dev(act), partial)
    assert out.shape == (1, M, D) and out.dtype == torch.bfloat16
    assert_close_gemm(out, out_ref)
    assert float(partial.max()) > 0


@pytest.mark.parametrize("a_k_rows,b_k_rows", [(False, False), (False, True), (True, True), (True, False)])
@pytest.mark.parametrize("R,C,K", [(256, 256, 64), (264, 40, 192), (1000, 520, 768), (3072, 768, 4096), (72, 1104, 128)])
def test_gemm_bf16_layouts_and_ragged_tiles(amd, R, C, K, a_k_rows, b_k_rows):
    """The plain bf16 product in all four operand layouts (contraction contiguous, or the contraction as the
    operand's rows, read through transposing LDS loads) against a double-precision product; ragged edge tiles,
    few tiles with a long contraction (cut along it) and many tiles."""
    g = torch.Generator().manual_seed(R + 3 * C + K)
    a = torch.randn(R, K, generator=g).bfloat16()
    b = torch.randn(C, K, generator=g).bfloat16()
    ref = a.double() @ b.double().T
    ad = dev(a.T.contiguous() if a_k_rows else a)
    bd = dev(b.T.contiguous() if b_k_rows else b)
    got = torch.ops.nanogpt.gemm_bf16(ad, bd, a_k_rows, b_k_rows)
    assert got.shape == (R, C) and got.dtype == torch.bfloat16
    assert_close_gemm(got, ref, 5e-3)
    # fp32 accumulation, one rounding: nearly every element is the correctly rounded bf16 of the exact product
    assert (got.cpu() == ref.float().bfloat16()).float().mean() > 0.97


def test_gemm_bf16_operand_orientation(amd):
    """One-hot probe through the transposing reads: element (r, c) pairs row r of A with row c of B at the same
    contraction position; a swapped half, a wrong swizzle or a permuted contraction fails exactly."""
    K = 192
    a = torch.zeros(304, K)
    b = torch.zeros(264, K)
    for r in range(304):
        a[r, (r * 37) % K] = 1 + (r % 5)
    for c in range(264):
        b[c, (c * 11) % K] = 2 + (c % 3)
    ref = a @ b.T
    for a_k_rows in (False, True):
        for b_k_rows in (False, True):
            ad = dev((a.T.contiguous() if a_k_rows else a).bfloat16())
            bd = dev((b.T.contiguous() if b_k_rows else b).bfloat16())
            got = torch.ops.nanogpt.gemm_bf16(ad, bd, a_k_rows, b_k_rows).float().cpu()
            assert torch.equal(got, ref), (a_k_rows, b_k_rows)


@pytest.mark.parametrize("M", [4096, 49152])
def test_gemm_bf16_token_contraction(amd, M):
    """The weight-gradient shape of the MLP backward: [3072, 768] = a^T b over M tokens, 36 output tiles cut 7 ways
    along the contraction with the partial sums meeting in fp32 (one rounding to bf16)."""
    g = torch.Generator(device="cuda").manual_seed(M)
    a = torch.randn(M, 3072, device="cuda", generator=g).bfloat16()
    b = torch.randn(M, 768, device="cuda", generator=g).bfloat16()
    got = torch.ops.nanogpt.gemm_bf16(a, b, True, True)
    ref = a.float().T @ b.float()
    assert got.shape == (3072, 768)
    assert rel_err(got.float().cpu(), ref.cpu()) <= 4e-3          # the bf16 rounding of the output alone is 2^-9 / sqrt(3)


def test_linear_relu_square_without_fp8_copies(amd, oracle):
    """linear_relu_square(a, b) with no fp8 arguments (the reference's DISABLE_FP8 path) and the MLP function on it."""
    M, D, H = 512, 256, 768
    x, w_fc, w_proj_t = oracle.make_cfg2(seed=12, M=M, D=D, H=H)
    out_ref, post_ref = oracle.mlp_fwd(x[None], w_fc, w_proj_t)
    post = amd.linear_relu_square(dev(x), dev(w_fc))
    assert_close_gemm(post, post_ref)
    assert (post.cpu() == post_ref).float().mean() > 0.97
    dy = (torch.randn(1, M, D, generator=torch.Generator().manual_seed(13)) * 1e-3).bfloat16()
    dx_ref, dw1_ref, dw2_ref = oracle.mlp_bwd(dy, x[None], w_fc, w_proj_t, post_ref)
    xg, w1g, w2g = dev(x[None]).requires_grad_(), dev(w_fc).requires_grad_(), dev(w_proj_t).requires_grad_()
    out = amd.ReLUSqrdMLP(xg, w1g, w2g)
    assert_close_gemm(out, out_ref)
    out.backward(dev(dy))
    assert_close_gemm(xg.grad, dx_ref)
    assert_close_gemm(w1g.grad, dw1_ref)
    assert_close_gemm(w2g.grad, dw2_ref)


@pytest.mark.parametrize("M,D,H", [(256, 64, 256), (1000, 768, 3072), (2048, 1024, 4096)])
def test_dpre_bf16_kernel(amd, oracle, M, D, H):
    """bf16 MFMA GEMM with the 2*c*sqrt(post) epilogue, incl. a token count that is not a tile multiple."""
    g = torch.Generator().manual_seed(M + H)
    dy = (torch.randn(M, D, generator=g) * 1e-2).bfloat16()
    w2 = (torch.randn(H, D, generator=g) / math.sqrt(H)).bfloat16()
    post = (torch.relu(torch.randn(M, H, generator=g)) ** 2).bfloat16()
    ref = oracle.fc_relu2_bwd_dpre(dy, w2, post)
    got = torch.ops.nanogpt.fc_relu2_bwd_dpre(dev(dy), dev(w2), dev(post))
    assert got.dtype == torch.bfloat16 and got.shape == (M, H)
    assert_close_gemm(got, ref)
    assert torch.equal(got.cpu() == 0, ref == 0) or ((got.cpu() == 0) != (ref == 0)).float().mean() < 1e-4
    assert (got.cpu() == ref).float().mean() > 0.97            # fp32 accumulation order only moves bf16 ties


@pytest.mark.parametrize("rows,dim", [(64, 768), (1000, 768), (4096, 1024), (16, 2048)])
def test_mlp_input_quant(amd, oracle, rows, dim):
    """rms-norm + amax + dynamic e4m3 quantisation of the MLP input against the eager formulation."""
    g = torch.Generator().manual_seed(rows + dim)
    x = (torch.randn(rows, dim, generator=g) * torch.rand(rows, 1, generator=g) * 3).bfloat16()
    up_scale = torch.tensor([0.0123], dtype=torch.float32)
    normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(dev(x), dev(up_scale))
    ref_n = oracle.rms_norm(x)
    # the row sum of squares is accumulated in a different order: a few results may land on the other side of a bf16 tie
    n_cpu = normed.cpu()
    assert (n_cpu == ref_n).float().mean() > 0.999
    torch.testing.assert_close(n_cpu.float(), ref_n.float(), rtol=2 ** -7, atol=0)
    # given the kernel's own normed values the quantisation is bit-exact
    ref_f8, ref_dq = oracle.mlp_input_quant(n_cpu, up_scale)
    assert torch.equal(x_f8.cpu().view(torch.uint8), ref_f8.view(torch.uint8))
    assert torch.equal(dequant.cpu(), ref_dq)


def test_mlp_input_quant_rounds_the_reciprocal_like_eager(amd, oracle):
    """`448.0 / amax` with a bf16 amax is amax.reciprocal() * 448.0 in eager, two bf16 roundings; one division rounds
    differently for about a quarter of all amax values.  Many small inputs, bit-exact on all of them, and at least
    one of them must be a case that tells the two apart."""
    up_scale = torch.tensor([0.5], dtype=torch.float32)
    telling = 0
    for seed in range(16):
        g = torch.Generator().manual_seed(300 + seed)
        x = (torch.randn(32, 256, generator=g) * torch.rand(32, 1, generator=g) * (seed + 1)).bfloat16()
        normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(dev(x), dev(up_scale))
        n_cpu = normed.cpu()
        ref_f8, ref_dq = oracle.mlp_input_quant(n_cpu, up_scale)
        assert torch.equal(u8(x_f8), u8(ref_f8)) and torch.equal(dequant.cpu(), ref_dq), seed
        amax = n_cpu.float().abs().max()
        one_division = (n_cpu.float() * (448.0 / amax).bfloat16().float()).bfloat16().to(E4M3)
        telling += int(not torch.equal(u8(one_division), u8(ref_f8)))
    assert telling >= 1


@pytest.mark.parametrize("shape", [(256, 768), (1001, 1024), (2, 37, 2048), (5, 64)])
def test_mlp_input_quant_grad(amd, shape):
    """Gradient through the norm (own kernel) against autograd of F.rms_norm on the CPU."""
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 3).bfloat16()
    xd = dev(x).requires_grad_(True)
    normed, _, _ = torch.ops.nanogpt.mlp_input_quant(xd, torch.ones(1, device="cuda"))
    gy = torch.randn(*shape, generator=g).bfloat16()
    normed.backward(dev(gy))
    xr = x.clone().requires_grad_(True)
    torch.nn.functional.rms_norm(xr, (shape[-1],)).backward(gy)
    assert xd.grad.dtype == torch.bfloat16 and xd.grad.shape == x.shape
    torch.testing.assert_close(xd.grad.cpu().float(), xr.grad.float(), rtol=2e-2, atol=1e-3)


@pytest.mark.parametrize("L,H,D", [(3, 256, 128), (12, 3072, 768)])
def test_quant_up_weights(amd, oracle, L, H, D):
    g = torch.Generator().manual_seed(L)
    w = (torch.randn(L, H, D, generator=g) * torch.logspace(-2, 0, L).view(L, 1, 1)).bfloat16()
    w_f8, scales = torch.ops.nanogpt.quant_up_weights(dev(w))
    ref_f8, ref_s = oracle.quantize_up_weights(w)
    assert torch.equal(scales.cpu(), ref_s)
    assert torch.equal(w_f8.cpu().view(torch.uint8), ref_f8.view(torch.uint8))


def test_path_traces_under_torch_compile_fullgraph(amd, oracle):
    """The reference runs its model under torch.compile(dynamic=False, fullgraph=True) (train_gpt.py:2260):
    dynamo, fake tensors and AOT autograd must get through every operator of the path without a graph
    break, forward and backward, and give what eager calls of the same kernels give."""
    M, D, H, V = 512, 256, 1024, 1024
    g = torch.Generator().manual_seed(71)
    x0 = dev(torch.randn(M, D, generator=g).bfloat16())
    w_fc = dev((torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16())
    w_proj_t = dev((torch.randn(H, D, generator=g) / math.sqrt(H)).bfloat16())
    w_head = dev((torch.randn(D, V, generator=g) / math.sqrt(D)).bfloat16())      # (in, out) as at the reference's HEAD
    w_mm = dev((torch.randn(D, D, generator=g) / math.sqrt(D)).bfloat16())
    targets = dev(torch.randint(0, V, (M,), generator=g))
    w_f8, up_scales = torch.ops.nanogpt.quant_up_weights(w_fc[None].contiguous())
    w2_scale = (w_proj_t.float().abs().max() / 448).reshape(1)
    w2_f8_dh = (w_proj_t.float() / w2_scale).T.contiguous().to(E4M3)               # [D, H]
    act_scale = torch.full((1,), 0.02, device="cuda")
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448

    def step(x, w_mm, w_fc, w_proj_t, w_head, partial, fp8_down):
        h = torch.ops.nanogpt.mm(x, w_mm, x_s=1.0, w_s=1 / 32, grad_s=grad_s)[0]
        normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(h, up_scales[0:1])
        if fp8_down:
            h = h + amd.ReLUSqrdMLP(normed, w_fc, w_proj_t, w_f8[0], dequant, x_f8, w2_f8_dh.T, w2_scale, act_scale, partial)
        else:
            h = h + amd.ReLUSqrdMLP(normed, w_fc, w_proj_t, w_f8[0], dequant, x_f8)
        losses = amd.FusedSoftcappedCrossEntropy.apply(h, targets, None, None, None, w_head, x_s, w_s, grad_s, 1.0)
        return losses.sum()

    for fp8_down in (False, True):
        results = []
        for fn in (step, torch.compile(step, fullgraph=True, dynamic=False, backend="aot_eager")):
            leaves = [t.clone().requires_grad_(True) for t in (x0, w_mm, w_fc, w_proj_t, w_head)]
            partial = torch.zeros(256, device="cuda")
            loss = fn(*leaves, partial, fp8_down)
            loss.backward()
            results.append((loss.detach(), [t.grad for t in leaves], partial))
        (l0, g0, p0), (l1, g1, p1) = results
        assert torch.isfinite(l0) and torch.equal(l0, l1)
        for a, b in zip(g0, g1):
            assert a is not None and b is not None and a.dtype == b.dtype and a.shape == b.shape
            # same kernels in the same order on the same data
            assert rel_err(b.float(), a.float()) <= 1e-5
        assert torch.equal(p0, p1) and (float(p0.max()) > 0) == fp8_down


def test_path_runs_under_the_reference_compile_mode(amd):
    """torch.compile(dynamic=False, fullgraph=True) with the DEFAULT backend, as the reference compiles its model
    (train_gpt.py:2260): the path's operators between ordinary torch operations that the backend fuses into generated
    kernels (residual adds, a norm), forward and backward, against the same function run eagerly.  The generated
    elementwise kernels keep fp32 where eager's separate kernels round to bf16 in between (residual add + norm in one
    kernel); an activation that moves by a bf16 unit changes a few percent of the fp8 codes downstream (the same effect
    as eager against fused quantisation in the reference), so gradients are compared to 5e-2 here, not to 2e-2."""
    M, D, H, V = 512, 256, 1024, 2048
    g = torch.Generator().manual_seed(72)
    x0 = dev(torch.randn(M, D, generator=g).bfloat16())
    w_mm = dev((torch.randn(D, D, generator=g) / math.sqrt(D)).bfloat16())
    w_fc = dev((torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16())
    w_proj_t = dev((torch.randn(H, D, generator=g) / math.sqrt(H)).bfloat16())
    w_head = dev((torch.randn(D, V, generator=g) / math.sqrt(D)).bfloat16())      # (in, out) as at the reference's HEAD
    targets = dev(torch.randint(0, V, (M,), generator=g))
    w_f8, up_scales = torch.ops.nanogpt.quant_up_weights(w_fc[None].contiguous())
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448

    def step(x, w_mm, w_fc, w_proj_t, w_head):
        h = x + torch.ops.nanogpt.mm(x, w_mm, x_s=1.0, w_s=1 / 32, grad_s=grad_s)[0]
        normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(h, up_scales[0:1])
        h = h + amd.ReLUSqrdMLP(normed, w_fc, w_proj_t, w_f8[0], dequant, x_f8)
        h = torch.nn.functional.rms_norm(h, (D,))
        losses = amd.FusedSoftcappedCrossEntropy.apply(h, targets, None, None, None, w_head, x_s, w_s, grad_s, 1.0)
        return losses.sum()

    results = []
    for compiled in (False, True):
        fn = torch.compile(step, fullgraph=True, dynamic=False) if compiled else step
        leaves = [t.clone().requires_grad_(True) for t in (x0, w_mm, w_fc, w_proj_t, w_head)]
        try:
            loss = fn(*leaves)
            loss.backward()
            torch.cuda.synchronize()
        except Exception as e:      # the default backend generates code with a compiler that a box may lack
            if compiled and type(e).__module__.startswith(("torch._dynamo", "torch._inductor", "triton")):
                pytest.skip(f"the default torch.compile backend could not generate code here: {type(e).__name__}: {str(e)[:200]}")
            raise
        results.append((loss.detach(), [t.grad for t in leaves]))
    (l0, g0), (l1, g1) = results
    assert torch.isfinite(l0) and abs(float(l0 - l1)) / M <= LOSS_TOL
    for a, b in zip(g0, g1):
        assert a is not None and b is not None and a.dtype == b.dtype and a.shape == b.shape
        assert rel_err(b.float(), a.float()) <= 5e-2


def test_path_replays_from_a_hip_graph(amd):
    """Launch-bound callers capture the step in a HIP graph: the library neither allocates, nor synchronises, nor
    clears memory through the runtime, so a captured step (mm forward+backward, the MLP function, the fused CE,
    all through autograd) must replay correctly.  Replayed three times on new inputs, with eager work and
    synchronisations in between, each replay against the eager result for the same inputs."""
    M, D, H, V = 512, 256, 1024, 2048
    gen = torch.Generator(device="cuda").manual_seed(9)
    rnd = lambda *s, scale=1.0: (torch.randn(*s, device="cuda", generator=gen) * scale).bfloat16()
    x_in = rnd(M, D)
    w_mm, w_fc, w_pt, w_head = rnd(D, D, scale=D ** -0.5), rnd(H, D, scale=D ** -0.5), rnd(H, D, scale=H ** -0.5), rnd(D, V, scale=D ** -0.5)
    targets = torch.randint(0, V, (M,), device="cuda", generator=gen)
    w_f8, up_scales = torch.ops.nanogpt.quant_up_weights(w_fc[None].contiguous())
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448
    leaves = [t.clone().requires_grad_(True) for t in (w_mm, w_fc, w_pt, w_head)]

    def step(x):
        for t in leaves:
            t.grad = None
        x = x.detach().requires_grad_(True)
        h = torch.ops.nanogpt.mm(x, leaves[0], x_s=1.0, w_s=1 / 32, grad_s=grad_s)[0]
        normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(h, up_scales[0:1])
        h = h + amd.ReLUSqrdMLP(normed, leaves[1], leaves[2], w_f8[0], dequant, x_f8)
        losses = amd.FusedSoftcappedCrossEntropy.apply(h, targets, None, None, None, leaves[3], x_s, w_s, grad_s, 1.0)
        loss = losses.sum()
        loss.backward()
        return [loss.detach().clone(), x.grad.clone()] + [t.grad.clone() for t in leaves]

    side = torch.cuda.Stream()                 # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(x_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(x_in)
    for rep in range(3):
        x_in.copy_(rnd(M, D))
        want = step(x_in)                      # eager, same buffers as the graph reads
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(captured, want):
            assert torch.isfinite(got.float()).all()
            assert rel_err(got.float(), ref.float()) <= 1e-5, f"replay {rep}"


def test_entry_points_are_reentrant_across_host_threads_and_streams(amd):
    """Two host threads, each on its own stream (default priority), issue mm forward+backward and the fused CE
    at the same time; every result must equal the one the same call gives alone."""
    import threading
    M, N, K, V = 512, 640, 256, 1024
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448

    def make(seed):
        g = torch.Generator(device="cuda").manual_seed(seed)
        r = lambda *s, scale=1.0: (torch.randn(*s, device="cuda", generator=g) * scale).bfloat16()
        return dict(x=r(M, K), w=r(N, K, scale=K ** -0.5), go=r(M, N, scale=1e-3), wh=r(K, V, scale=K ** -0.5),
                    t=torch.randint(0, V, (M,), device="cuda", generator=g))

    def work(d):
        out, x_f8, w_f8 = torch.ops.nanogpt.mm(d["x"], d["w"], x_s, w_s, grad_s)
        dx, dw = torch.ops.nanogpt.mm_backward(d["go"], x_f8, w_f8, x_s, w_s, grad_s)
        xr, wr = d["x"].clone().requires_grad_(True), d["wh"].clone().requires_grad_(True)
        losses = amd.FusedSoftcappedCrossEntropy.apply(xr, d["t"], None, None, None, wr, x_s, w_s, grad_s, 1.0)
        losses.sum().backward()
        return [out, dx, dw.contiguous(), losses.detach(), xr.grad, wr.grad]

    data = [make(1), make(2)]
    alone = [work(d) for d in data]
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def run(i):
        try:
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.default_stream())
            with torch.cuda.stream(s):
                for _ in range(20):
                    results[i] = work(data[i])
            s.synchronize()
        except Exception as e:      # surfaced below, in the main thread
            errors.append(e)

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for got, ref in zip(results, alone):
        for a, b in zip(got, ref):
            # same kernels on the same data, each call with its own workspace
            assert rel_err(a.float(), b.float()) <= 1e-5
