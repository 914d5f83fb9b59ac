"""Full-size runs of the fused lm_head + cross-entropy (benchmark configurations 3 and 5) on the GPU.

The CPU oracle cannot process 49152 x 50304 logits in seconds, so parity at this size is checked on what
the problem's structure allows: rows are independent in the forward and in dx (row subsets against the
oracle), dW is checked on a subset of vocabulary rows against the oracle's gradient formula, and as a
sum over the token halves (additivity of the whole path, including the balanced walk's split tiles)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

LOSS_TOL = 1e-3
GEMM_TOL = 2e-2


@pytest.fixture(scope="module")
def amd():
    import modded_nanogpt_amd as m
    m._lib.load()
    assert torch.cuda.is_available()
    return m


def _rel(got, ref):
    return ((got.float() - ref.float()).norm() / ref.float().norm().clamp_min(1e-30)).item()


def _run_gpu(x, w, t, sc, mode="recompute"):
    """Forward + backward through the operators; `mode` = where the backward takes the gradient of the logits from:
    "recompute" (second logits GEMM) or "codes" (one code byte per logit kept by the forward, the default of the
    autograd function and what bench.py times)."""
    d = "cuda"
    M = x.shape[0]
    mtp = torch.tensor([1.0], device=d)
    pt = torch.full((M,), -1, dtype=torch.int64, device=d)
    pw = torch.zeros(1, device=d)
    xd, wd, td = x.to(d), w.to(d), t.to(d)
    fwd_args = (xd, wd, td, mtp, pt, pw, sc["x_s"], sc["w_s"], sc["A"], sc["B"], sc["C"], False)
    tail = (sc["x_s"], sc["w_s"], sc["grad_s"], sc["grad_scale"], sc["A"], sc["B"], sc["C"], False)
    if mode == "codes":
        losses, lse, sig, x_f8, w_f8, codes = torch.ops.nanogpt.lmhead_ce_fwd_codes(*fwd_args)
        dx, dw = torch.ops.nanogpt.lmhead_ce_bwd_codes(x_f8, w_f8, td, mtp, pt, pw, lse, sig, codes, *tail)
    else:
        losses, lse, sig, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(*fwd_args)
        dx, dw = torch.ops.nanogpt.lmhead_ce_bwd(x_f8, w_f8, td, mtp, pt, pw, lse, sig, *tail)
    torch.cuda.synchronize()
    return losses, lse, x_f8, w_f8, dx, dw


def _check_fp8_copies_and_lse(oracle, x, w, sc, lse, x_f8, w_f8):
    """The fp8 copies equal the oracle's quantiser on every byte, and EVERY row's lse equals an fp32 reference taken on
    the GPU in row chunks from those verified copies (logits as bf16(acc * x_s * w_s), the oracle's softcap, logsumexp
    in fp32 -- reference train_gpt.py:1689-1692), so nothing that later checks build on rests on the kernel's own statistics."""
    assert torch.equal(x_f8.view(torch.uint8).cpu(), oracle.quant_e4m3(x, sc["x_s"]).view(torch.uint8))
    assert torch.equal(w_f8.view(torch.uint8).cpu(), oracle.quant_e4m3(w, sc["w_s"]).view(torch.uint8))
    wf = w_f8.float()
    scale = torch.tensor(sc["x_s"], dtype=torch.float32) * torch.tensor(sc["w_s"], dtype=torch.float32)
    worst = 0.0
    for r0 in range(0, x_f8.shape[0], 2048):
        logits = ((x_f8[r0:r0 + 2048].float() @ wf.T) * scale.item()).bfloat16()
        z = sc["A"] * oracle.softcap_sigma(logits, sc["B"], sc["C"])
        worst = max(worst, (torch.logsumexp(z, dim=1) - lse[r0:r0 + 2048]).abs().max().item())
    assert worst <= LOSS_TOL, worst


def _check_rows(oracle, x, w, t, sc, rows, losses, dx):
    one = torch.tensor([1.0])
    l_ref, ctx = oracle.lm_head_ce_fwd(x[rows], t[rows], one, None, None, w, sc["x_s"], sc["w_s"], sc["grad_s"],
                                       sc["grad_scale"], sc["A"], sc["B"], sc["C"], "out_in")
    dx_ref, _ = oracle.lm_head_ce_bwd(ctx)
    assert (losses.cpu()[rows] - l_ref).abs().max().item() <= LOSS_TOL
    assert _rel(dx.cpu()[rows], dx_ref) <= GEMM_TOL


def _check_dw_columns(oracle, t, sc, cols, lse, x_f8, w_f8, dw):
    xf = x_f8.cpu().float()
    logits = ((xf @ w_f8.cpu()[cols].float().T) * (sc["x_s"] * sc["w_s"])).bfloat16()
    dl = oracle.ce_grad_columns(logits, cols, lse.cpu(), t, sc["A"], sc["B"], sc["C"], sc["grad_s"], sc["grad_scale"])
    dw_ref = (dl.float().T @ xf) * (sc["x_s"] * sc["grad_s"])
    assert _rel(dw.cpu()[cols], dw_ref) <= GEMM_TOL


@pytest.mark.parametrize("mode", ["codes", "recompute"])
def test_config3_full_size(amd, oracle, mode):
    x, w, t, sc = oracle.make_cfg3(seed=0)
    M, V = x.shape[0], w.shape[0]
    losses, lse, x_f8, w_f8, dx, dw = _run_gpu(x, w, t, sc, mode)
    assert torch.isfinite(losses).all() and torch.isfinite(dx.float()).all() and torch.isfinite(dw).all()
    _check_fp8_copies_and_lse(oracle, x, w, sc, lse, x_f8, w_f8)
    # row subset (first / middle / last tiles, tile edges) against the oracle
    rows = torch.cat([torch.arange(0, M, 997), torch.arange(M - 64, M), torch.arange(255, M, 8192)]).unique()
    _check_rows(oracle, x, w, t, sc, rows, losses, dx)
    # softmax normaliser bounds: z in (0, A)  =>  ln V < lse < A + ln V
    assert (lse > math.log(V)).all() and (lse < sc["A"] + math.log(V)).all()
    # vocabulary subset of dW (some target columns, first / last rows of the matrix) against the oracle's formula
    cols = torch.cat([t[:16], torch.arange(0, 8), torch.arange(V - 8, V), torch.tensor([255, 256, 25151, 50047])]).unique()
    _check_dw_columns(oracle, t, sc, cols, lse, x_f8, w_f8, dw)
    # additivity over the token halves
    h = M // 2
    la, _, _, _, dxa, dwa = _run_gpu(x[:h], w, t[:h], sc, mode)
    lb, _, _, _, dxb, dwb = _run_gpu(x[h:], w, t[h:], sc, mode)
    assert (torch.cat([la, lb]) - losses).abs().max().item() <= 1e-5
    assert _rel(torch.cat([dxa, dxb]), dx) <= 1e-3
    assert _rel(dwa + dwb, dw) <= 1e-4


def test_config5_shape(amd, oracle):
    """Medium-track dimensions: K = 1024 (8 k-steps per tile), M = 65536 (the largest single pass)."""
    g = torch.Generator().manual_seed(5)
    M, K, V = 65536, 1024, 50304
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16()
    t = torch.randint(0, 50257, (M,), generator=g)
    sc = dict(x_s=100 / 448, w_s=1.6 / 448, grad_s=0.75 / 448, grad_scale=1.0, A=23.0, B=5.0, C=7.5)
    losses, lse, x_f8, w_f8, dx, dw = _run_gpu(x, w, t, sc, "codes")
    _check_fp8_copies_and_lse(oracle, x, w, sc, lse, x_f8, w_f8)
    rows = torch.cat([torch.arange(0, M, 2039), torch.arange(M - 32, M)]).unique()
    _check_rows(oracle, x, w, t, sc, rows, losses, dx)
    cols = torch.cat([t[:8], torch.arange(V - 4, V)]).unique()
    _check_dw_columns(oracle, t, sc, cols, lse, x_f8, w_f8, dw)


def test_mtp_and_prefix_targets_at_training_shape(amd, oracle):
    """Stage-1 shape of the reference's schedule (train_gpt.py:1980-1983): M = 16384 tokens, three predicted
    tokens per position with weights, prefix targets, (in, out) weight as at HEAD, through the autograd function.
    Contiguous row blocks against the oracle; inside a block the last two rows look ahead past the block's
    end, so only the final block (the true end of the batch, where the look-ahead stops) is compared whole."""
    g = torch.Generator().manual_seed(16)
    M, K, V = 16384, 768, 50304
    x = torch.randn(M, K, generator=g).bfloat16()
    w_kv = (torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16().T.contiguous()      # (in, out)
    t = torch.randint(0, 50257, (M,), generator=g)
    t[5] = -100                                                                            # an ignored position
    mtp = torch.tensor([1.0, 0.5, 0.25])
    pt = torch.where(torch.rand(M, generator=g) < 0.3, torch.randint(0, 50257, (M,), generator=g), torch.full((M,), -1))
    pw = torch.tensor([0.4])
    x_s, w_s, grad_s, grad_scale = 100 / 448, 1.6 / 448, 0.75 / 448, 2.0
    d = "cuda"
    xd, wd = x.to(d).requires_grad_(True), w_kv.to(d).requires_grad_(True)
    losses = amd.FusedSoftcappedCrossEntropy.apply(xd, t.to(d), mtp.to(d), pt.to(d), pw.to(d), wd, x_s, w_s, grad_s, grad_scale)
    losses.sum().backward()
    torch.cuda.synchronize()
    assert wd.grad.shape == (K, V) and xd.grad.dtype == torch.bfloat16     # (autograd casts the fp32 dW to the leaf's dtype)
    n_ahead = mtp.numel() - 1
    for lo, hi in ((0, 96), (8100, 8292), (M - 96, M)):
        rows = slice(lo, hi)
        l_ref, ctx = oracle.lm_head_ce_fwd(x[rows], t[rows], mtp, pt[rows], pw, w_kv, x_s, w_s, grad_s, grad_scale)
        dx_ref, _ = oracle.lm_head_ce_bwd(ctx)
        keep = (hi - lo) if hi == M else (hi - lo - n_ahead)
        assert (losses.detach().cpu()[rows][:keep] - l_ref[:keep]).abs().max().item() <= LOSS_TOL
        assert _rel(xd.grad.cpu()[rows][:keep], dx_ref[:keep]) <= GEMM_TOL


def test_two_passes(amd, oracle):
    """More tokens than one pass of the backward holds (65536): dW accumulates over the passes."""
    g = torch.Generator().manual_seed(7)
    M, K, V = 65536 + 2048, 256, 2048
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16()
    t = torch.randint(0, V, (M,), generator=g)
    sc = dict(x_s=100 / 448, w_s=1.6 / 448, grad_s=0.75 / 448, grad_scale=1.0, A=23.0, B=5.0, C=7.5)
    losses, lse, x_f8, w_f8, dx, dw = _run_gpu(x, w, t, sc)
    rows = torch.cat([torch.arange(0, M, 1021), torch.arange(65536 - 8, 65536 + 8), torch.arange(M - 8, M)]).unique()
    _check_rows(oracle, x, w, t, sc, rows, losses, dx)
    _check_dw_columns(oracle, t, sc, torch.arange(0, V, 37), lse, x_f8, w_f8, dw)


@pytest.mark.parametrize("M,K,V", [(49152, 768, 50304), (65536 + 2048, 256, 2048)])
def test_backward_from_sigma_codes_full_size(amd, M, K, V):
    """Config 3, and more tokens than one pass of the backward holds: the gradients rebuilt from the forward's sigma
    codes equal the recomputed ones bit for bit (same row statistics), and the code-writing forward agrees with the
    plain one."""
    g = torch.Generator().manual_seed(11)
    d = "cuda"
    x = torch.randn(M, K, generator=g).bfloat16().to(d)
    w = (torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16().to(d)
    t = torch.randint(0, V, (M,), generator=g).to(d)
    mtp = torch.tensor([1.0], device=d)
    pt = torch.full((M,), -1, dtype=torch.int64, device=d)
    pw = torch.zeros(1, device=d)
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448
    fwd = (x, w, t, mtp, pt, pw, x_s, w_s, 23.0, 5.0, 7.5, False)
    l0, lse0, sig0, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(*fwd)
    l1, lse1, sig1, _, _, codes = torch.ops.nanogpt.lmhead_ce_fwd_codes(*fwd)
    assert torch.equal(sig0, sig1) and (lse0 - lse1).abs().max().item() <= 2e-5 and (l0 - l1).abs().max().item() <= 1e-4
    assert abs(float(l0.mean() - l1.mean())) <= 1e-5
    tail = (x_s, w_s, grad_s, 1.0, 23.0, 5.0, 7.5, False)
    dx0, dw0 = torch.ops.nanogpt.lmhead_ce_bwd(x_f8, w_f8, t, mtp, pt, pw, lse1, sig1, *tail)
    dx1, dw1 = torch.ops.nanogpt.lmhead_ce_bwd_codes(x_f8, w_f8, t, mtp, pt, pw, lse1, sig1, codes, *tail)
    assert torch.equal(dx0, dx1)
    if M <= 65536:
        assert torch.equal(dw0, dw1)
    else:   # dW of several passes is accumulated with floating-point atomics: the order of the additions varies from run to run
        assert _rel(dw1, dw0) <= 1e-5


def test_config2_mlp_forward_full_size(amd, oracle):
    """FP8 MLP forward at M = 49152: norm + quantise producers, c_fc with the ReLU^2 epilogue, down projection."""
    g = torch.Generator().manual_seed(2)
    M, D, H = 49152, 768, 3072
    x_raw = (torch.randn(M, D, generator=g) * 2).bfloat16()
    w_fc = (torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16()
    w_proj_t = (torch.randn(D, H, generator=g) / math.sqrt(H)).bfloat16().T.contiguous()
    d = "cuda"
    w_f8, scales = torch.ops.nanogpt.quant_up_weights(w_fc[None].to(d))
    w_f8_ref, scales_ref = oracle.quantize_up_weights(w_fc[None])
    assert torch.equal(w_f8.cpu().view(torch.uint8), w_f8_ref.view(torch.uint8)) and torch.equal(scales.cpu(), scales_ref)
    normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(x_raw.to(d), scales[0:1])
    # the quantisation is exact given the kernel's own normed values (global amax: needs the whole tensor)
    x_f8_ref, dequant_ref = oracle.mlp_input_quant(normed.cpu(), scales_ref[0:1])
    assert torch.equal(x_f8.cpu().view(torch.uint8), x_f8_ref.view(torch.uint8)) and torch.equal(dequant.cpu(), dequant_ref)
    assert (normed.cpu() == oracle.rms_norm(x_raw)).float().mean() > 0.999
    post = torch.ops.nanogpt.fc_relu2_fwd(x_f8, w_f8[0], dequant)
    out = amd.ReLUSqrdMLP(normed[None], w_fc.to(d), w_proj_t.to(d), w_f8[0], dequant, x_f8[None])
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, M, 1531), torch.arange(M - 16, M)]).unique()
    post_ref = oracle.fc_relu2_fwd(x_f8_ref[rows], w_f8_ref[0], dequant_ref)
    assert _rel(post.cpu()[rows], post_ref) <= GEMM_TOL
    out_ref = (post_ref.float() @ w_proj_t.float()).bfloat16()
    assert _rel(out.cpu()[0, rows], out_ref) <= GEMM_TOL


@pytest.mark.parametrize("M,D,H", [(49152, 768, 3072), (65536, 1024, 4096)])
def test_config4_mlp_backward_full_size(amd, oracle, M, D, H):
    """FP8 MLP forward + bf16 backward at M = 49152 (one layer of benchmark configuration 4) and at the medium-track
    shape M = 65536, D = 1024, H = 4096 (the MLP half of configuration 5).  dpre and dx are
    row-local: a row sample against the oracle.  The weight gradients contract over all tokens: against an
    fp32 product of the kernel's own post / dpre on the GPU (the plain reference for a floating-point
    contraction), and as the sum of the gradients of the two token halves (additivity, which also
    exercises the sliced contraction at a second size)."""
    g = torch.Generator().manual_seed(4)
    d = "cuda"
    x_raw = torch.randn(M, D, generator=g).bfloat16()
    w_fc = (torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16()
    w_proj_t = (torch.randn(D, H, generator=g) / math.sqrt(H)).bfloat16().T.contiguous()
    dy = (torch.randn(M, D, generator=g) * 1e-3).bfloat16()
    w_f8, scales = torch.ops.nanogpt.quant_up_weights(w_fc[None].to(d))
    normed_all, x_f8_all, dequant = torch.ops.nanogpt.mlp_input_quant(x_raw.to(d), scales[0:1])

    def run(rows):   # forward + backward on a slice of the tokens, same quantised input as the whole
        normed = normed_all[rows].detach().clone().requires_grad_(True)
        x_f8 = x_f8_all[rows].contiguous()
        w1 = w_fc.to(d).requires_grad_(True)
        w2 = w_proj_t.to(d).requires_grad_(True)
        out = amd.ReLUSqrdMLP(normed[None], w1, w2, w_f8[0], dequant, x_f8[None])
        out.backward(dy[rows].to(d)[None])
        post = torch.ops.nanogpt.fc_relu2_fwd(x_f8, w_f8[0], dequant)
        return normed, post, normed.grad, w1.grad, w2.grad

    everything = slice(0, M)
    normed, post, dx, dw1, dw2 = run(everything)
    dyd = dy.to(d)
    dpre = torch.ops.nanogpt.fc_relu2_bwd_dpre(dyd, w_proj_t.to(d), post)
    torch.cuda.synchronize()
    # row-local parts on a sample of rows: the forward's post against the oracle's on the same fp8 operands, then the backward
    rows = torch.cat([torch.arange(0, M, 1531), torch.arange(M - 16, M)]).unique()
    post_ref = oracle.fc_relu2_fwd(x_f8_all.cpu()[rows], w_f8.cpu()[0], dequant.cpu())
    assert _rel(post.cpu()[rows], post_ref) <= GEMM_TOL
    dpre_ref = oracle.fc_relu2_bwd_dpre(dy[rows], w_proj_t, post.cpu()[rows])
    assert _rel(dpre.cpu()[rows], dpre_ref) <= GEMM_TOL
    dx_ref = (dpre_ref.float() @ w_fc.float()).bfloat16()
    assert _rel(dx.cpu()[rows], dx_ref) <= GEMM_TOL
    # weight gradients against an fp32 contraction of the same operands
    dw2_ref = post.float().T @ dyd.float()
    dw1_ref = dpre.float().T @ normed.detach().float()
    assert dw1.shape == (H, D) and dw2.shape == (H, D)
    assert _rel(dw2, dw2_ref) <= GEMM_TOL and _rel(dw1, dw1_ref) <= GEMM_TOL
    # additivity over the token halves (each half's bf16 result carries its own rounding)
    del dw1_ref, dw2_ref
    _, _, _, dw1_a, dw2_a = run(slice(0, M // 2))
    _, _, _, dw1_b, dw2_b = run(slice(M // 2, M))
    assert _rel(dw2_a.float() + dw2_b.float(), dw2.float()) <= GEMM_TOL
    assert _rel(dw1_a.float() + dw1_b.float(), dw1.float()) <= GEMM_TOL


def test_config4_twelve_layers_back_to_back(amd):
    """Benchmark configuration 4 as worded: twelve layers with their own weights, forward + backward, enqueued back
    to back on one stream without a synchronisation in between.  Every layer's outputs and gradients must be what
    the same layer gives when it runs alone (the parts of split tiles are summed in a fixed order, so nothing may differ
    beyond what a run of the same kernels on the same data differs by)."""
    g = torch.Generator().manual_seed(12)
    M, D, H, L = 49152, 768, 3072, 12
    d = "cuda"
    x_raw = (torch.randn(M, D, generator=g) * 2).bfloat16().to(d)
    dy = (torch.randn(1, M, D, generator=g) * 1e-3).bfloat16().to(d)
    w_fc = [(torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16().to(d) for _ in range(L)]
    w_pt = [(torch.randn(D, H, generator=g) / math.sqrt(H)).bfloat16().T.contiguous().to(d) for _ in range(L)]
    w_f8, scales = torch.ops.nanogpt.quant_up_weights(torch.stack(w_fc))

    def layer(l):
        x = x_raw.clone().requires_grad_(True)
        w1, w2 = w_fc[l].clone().requires_grad_(True), w_pt[l].clone().requires_grad_(True)
        normed, x_f8, dequant = torch.ops.nanogpt.mlp_input_quant(x, scales[l:l + 1])
        out = amd.ReLUSqrdMLP(normed[None], w1, w2, w_f8[l], dequant, x_f8[None])
        out.backward(dy)
        return [out.detach(), x.grad, w1.grad, w2.grad]

    together = [layer(l) for l in range(L)]          # nothing synchronises between the layers
    torch.cuda.synchronize()
    for l in (0, 5, 11):
        alone = layer(l)
        torch.cuda.synchronize()
        for got, ref in zip(together[l], alone):
            assert torch.isfinite(got.float()).all()
            # split tiles meet in fp32 in any order: a sum next to a bf16 rounding boundary may round the other way
            assert _rel(got, ref) <= 1e-4, f"layer {l}"
    # layers differ from each other (own weights): a result that leaked from a neighbour would not pass the check above
    assert _rel(together[0][2], together[11][2]) > 0.5


@pytest.mark.parametrize("layout", ["out_in", "in_out"])
def test_mm_forward_backward_lm_head_shape(amd, oracle, layout):
    """nanogpt::mm / mm_t forward + backward at an lm_head-sized problem (N = 50304): row / column subsets
    against the oracle's quantise-dequantise-matmul restatement."""
    g = torch.Generator().manual_seed(11)
    M, N, K = 8192, 50304, 768
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    grad = (torch.randn(M, N, generator=g) * 1e-3).bfloat16()
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448 * 1e-2
    d = "cuda"
    if layout == "out_in":
        out, x_f8, w_f8 = torch.ops.nanogpt.mm(x.to(d), w.to(d), x_s, w_s, grad_s)
        dx, dw = torch.ops.nanogpt.mm_backward(grad.to(d), x_f8, w_f8, x_s, w_s, grad_s)
        dw_nk = dw                                   # [N, K] (a transposed view of the [K, N] result)
    else:
        out, x_f8, w_f8 = torch.ops.nanogpt.mm_t(x.to(d), w.T.contiguous().to(d), x_s, w_s, grad_s)
        dx, dw = torch.ops.nanogpt.mm_t_backward(grad.to(d), x_f8, w_f8, x_s, w_s, grad_s)
        dw_nk = dw.T                                 # [K, N] -> [N, K]
    torch.cuda.synchronize()
    xq, wq = oracle.quant_e4m3(x, x_s).float(), oracle.quant_e4m3(w, w_s).float()
    rows = torch.cat([torch.arange(0, M, 509), torch.arange(M - 8, M)]).unique()
    cols = torch.cat([torch.arange(0, N, 3001), torch.arange(N - 8, N)]).unique()
    out_ref = ((xq[rows] @ wq.T) * (x_s * w_s)).bfloat16()
    assert _rel(out.cpu()[rows], out_ref) <= GEMM_TOL
    gq_rows = oracle.quant_e5m2(grad[rows], grad_s).float()
    dx_ref = ((gq_rows @ wq) * (grad_s * w_s)).bfloat16()
    assert _rel(dx.cpu()[rows], dx_ref) <= GEMM_TOL
    gq_cols = oracle.quant_e5m2(grad[:, cols].contiguous(), grad_s).float()
    dw_ref = (gq_cols.T @ xq) * (x_s * grad_s)
    assert _rel(dw_nk.cpu()[cols], dw_ref) <= GEMM_TOL
