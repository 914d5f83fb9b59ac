"""Pins the floating-point part of the oracle against independent statements: a brute-force
triple loop over fp8 codes in double (C), closed forms, torch.autograd, fp64 finite
differences and invariants.  CPU only, small shapes."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import rel_err


def _brute(oracle_c, a_f8, b_f8, scale):
    """C[m,n] = scale * sum_k dec(a[m,k]) dec(b[n,k]) in double, from raw codes."""
    fa = 1 if a_f8.dtype == torch.float8_e5m2 else 0
    fb = 1 if b_f8.dtype == torch.float8_e5m2 else 0
    a = a_f8.contiguous().view(torch.uint8).numpy()
    b = b_f8.contiguous().view(torch.uint8).numpy()
    M, K = a.shape
    N = b.shape[0]
    out = np.empty((M, N), dtype=np.float64)
    oracle_c.ngpt_oracle_gemm_tn_codes(a.ctypes.data, b.ctypes.data, out.ctypes.data, M, N, K, fa, fb, float(scale))
    return torch.from_numpy(out)


@pytest.mark.parametrize("M,N,K", [(16, 16, 32), (5, 7, 13), (33, 20, 200)])
def test_mm_fwd_bwd_vs_brute_force(oracle, oracle_c, M, N, K):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    go = (torch.randn(M, N, generator=g) * 1e-3).bfloat16()
    x_s, w_s, grad_s = 100 / 448, 1.6 / 448, 0.75 / 448
    out, x_f8, w_f8 = oracle.mm_fwd(x, w, x_s, w_s)
    assert out.dtype == torch.bfloat16 and x_f8.dtype == torch.float8_e4m3fn
    s32 = float(np.float32(x_s) * np.float32(w_s))
    ref = _brute(oracle_c, x_f8, w_f8, s32)
    assert torch.equal(out, ref.float().bfloat16()) or rel_err(out, ref) < 3e-3
    assert rel_err(out, ref) < 3e-3            # bf16 output rounding only

    dx, dw = oracle.mm_bwd(go, x_f8, w_f8, x_s, w_s, grad_s)
    assert dx.shape == (M, K) and dx.dtype == torch.bfloat16
    assert dw.shape == (N, K) and dw.dtype == torch.float32 and dw.stride() == (1, N)
    g_f8 = oracle.quant_e5m2(go, grad_s)
    ref_dx = _brute(oracle_c, g_f8, w_f8.T.contiguous(), float(np.float32(grad_s) * np.float32(w_s)))
    ref_dw = _brute(oracle_c, g_f8.T.contiguous(), x_f8.T.contiguous(), float(np.float32(x_s) * np.float32(grad_s)))
    assert rel_err(dx, ref_dx) < 3e-3
    assert rel_err(dw, ref_dw) < 1e-6


def test_mm_t_is_mm_with_transposed_storage(oracle):
    x, w, x_s, w_s = oracle.make_cfg1(seed=4, M=64, N=48, K=96)
    go = torch.randn(64, 48, generator=torch.Generator().manual_seed(5)).bfloat16() * 1e-3
    out, x_f8, w_f8 = oracle.mm_fwd(x, w, x_s, w_s)
    out_t, x_f8_t, w_f8_t = oracle.mm_t_fwd(x, w.T.contiguous(), x_s, w_s)
    assert torch.equal(out, out_t) and torch.equal(x_f8.view(torch.uint8), x_f8_t.view(torch.uint8))
    assert torch.equal(w_f8.view(torch.uint8), w_f8_t.T.contiguous().view(torch.uint8))
    dx, dw = oracle.mm_bwd(go, x_f8, w_f8, x_s, w_s, 0.75 / 448)
    dx_t, dw_t = oracle.mm_t_bwd(go, x_f8_t, w_f8_t, x_s, w_s, 0.75 / 448)
    assert torch.equal(dx, dx_t) and dw_t.is_contiguous() and torch.equal(dw, dw_t.T)


def test_mm_cfg1_matches_fp32_linear_within_quantisation(oracle):
    """Config 1 (power-of-two scales): fp8 result is close to the unquantised bf16 linear;
    a transposed or unscaled operand would be off by O(1)."""
    x, w, x_s, w_s = oracle.make_cfg1(seed=0, M=128, N=96, K=768)
    out, _, _ = oracle.mm_fwd(x, w, x_s, w_s)
    ref = x.float() @ w.float().T
    assert rel_err(out, ref) < 0.06


def test_fc_relu2_invariants_and_value(oracle):
    g = torch.Generator().manual_seed(6)
    x = oracle.rms_norm(torch.randn(96, 64, generator=g).bfloat16())
    w = (torch.randn(3, 80, 64, generator=g) / 8).bfloat16()
    w_f8, scales = oracle.quantize_up_weights(w)
    assert w_f8.shape == w.shape and scales.shape == (3,)
    assert torch.allclose(scales, w.float().abs().amax(dim=(1, 2)) / 448, rtol=1e-2)
    assert float(w_f8[1].float().abs().max()) == 448.0
    x_f8, dequant = oracle.mlp_input_quant(x, scales[1:2])
    assert float(x_f8.float().abs().max()) == 448.0
    post = oracle.fc_relu2_fwd(x_f8, w_f8[1], dequant)
    pre = x.float() @ w[1].float().T
    assert post.dtype == torch.bfloat16 and (post >= 0).all()
    assert rel_err(post, torch.relu(pre) ** 2) < 0.08
    # post == 0 exactly where the bf16-rounded pre-activation is <= 0
    c = ((x_f8.float() @ w_f8[1].float().T) * dequant).bfloat16()
    assert torch.equal(post, (torch.relu(c.float()) ** 2).bfloat16())
    assert ((c <= 0) <= (post == 0)).all()
    # EMIT_FP8 variant
    act = torch.tensor([float(post.float().max()) * 1.25 / 448])
    post2, post_f8, amax = oracle.fc_relu2_fwd(x_f8, w_f8[1], dequant, act)
    assert torch.equal(post, post2) and float(amax) == float(post.float().max())
    assert rel_err(post_f8.float() * act, post) < 0.05
    assert float(post_f8.float().max()) <= 448.0


def test_mlp_backward_matches_autograd(oracle):
    g = torch.Generator().manual_seed(7)
    M, D, H = 64, 32, 96
    x = torch.randn(M, D, generator=g).bfloat16()
    w1 = (torch.randn(H, D, generator=g) / math.sqrt(D)).bfloat16()
    w2 = (torch.randn(H, D, generator=g) / math.sqrt(H)).bfloat16()
    dy = (torch.randn(M, D, generator=g) * 1e-2).bfloat16()
    out, post = oracle.mlp_fwd(x, w1, w2)
    dx, dw1, dw2 = oracle.mlp_bwd(dy, x, w1, w2, post)
    xf, w1f, w2f = (t.double().requires_grad_() for t in (x, w1, w2))
    ref = torch.relu(xf @ w1f.T) ** 2 @ w2f
    assert rel_err(out, ref.detach()) < 1e-2
    ref.backward(dy.double())
    assert rel_err(dx, xf.grad) < 2e-2
    assert rel_err(dw1, w1f.grad) < 2e-2
    assert rel_err(dw2, w2f.grad) < 2e-2
    # 2*c*sqrt(post) == 2*c*relu(pre) up to bf16 rounding of post
    dpre = oracle.fc_relu2_bwd_dpre(dy, w2, post)
    pre = x.double() @ w1.double().T
    assert rel_err(dpre, 2 * (dy.double() @ w2.double().T) * torch.relu(pre)) < 1e-2


def _ce_inputs(M=48, V=320, seed=8, scale=4.0):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(M, V, generator=g) * scale).bfloat16()
    targets = torch.randint(0, V, (M,), generator=g)
    return logits, targets


def test_ce_reduces_to_cross_entropy(oracle):
    logits, targets = _ce_inputs()
    M, V = logits.shape
    one, nopre, pw = torch.tensor([1.0]), torch.full((M,), -1), torch.zeros(1)
    losses, dl, lse = oracle.ce_fwd_bwd(logits, targets, one, nopre, pw, M, 1, 23.0, 5.0, 7.5, 0.75 / 448, 1.0)
    ref = oracle.softcap_ce_closed_form(logits, targets)
    # bf16 rounding of sigma moves a single softcapped logit by <= 23 * 2^-9
    assert (losses - ref).abs().max() < 23 * 2.0 ** -8
    assert abs(float(losses.mean() - ref.mean())) < 1e-2
    z = 23 * oracle.softcap_sigma(logits, 5.0, 7.5)
    assert ((z > 0) & (z < 23)).all()
    assert (lse > z.max(1).values).all() and (lse <= z.max(1).values + math.log(V) + 1e-5).all()
    assert torch.allclose(torch.exp(z - lse[:, None]).sum(1), torch.ones(M), atol=1e-5)
    # exact agreement with cross_entropy on the *rounded* sigma
    assert torch.allclose(losses, F.cross_entropy(z, targets, reduction="none"), atol=2e-6)


def test_ce_equal_logits_gives_log_v(oracle):
    M, V = 4, 1000
    logits = torch.full((M, V), 0.75).bfloat16()
    t = torch.tensor([0, 5, 999, 17])
    losses, dl, _ = oracle.ce_fwd_bwd(logits, t, torch.tensor([1.0]), torch.full((M,), -1), torch.zeros(1),
                                      M, 1, 23.0, 5.0, 7.5, 1.0, 1.0)
    assert torch.allclose(losses, torch.full((M,), math.log(V)), atol=1e-5)


def test_ce_gradient_vs_autograd_and_finite_differences(oracle):
    logits, targets = _ce_inputs(M=12, V=40, seed=9)
    M, V = logits.shape
    grad_s, grad_scale = 2.0 ** -12, 3.0
    losses, dl, _ = oracle.ce_fwd_bwd(logits, targets, torch.tensor([1.0]), torch.full((M,), -1), torch.zeros(1),
                                      M, 1, 23.0, 5.0, 7.5, grad_s, grad_scale)
    lf = logits.double().requires_grad_()
    (oracle.softcap_ce_closed_form(lf, targets).sum() * grad_scale).backward()
    got = dl.float().double() * grad_s
    # against the analytic gradient evaluated in fp64 on the bf16-rounded sigma: only the
    # e5m2 rounding remains (2 mantissa bits: <= 2^-3 relative, plus the subnormal quantum)
    sig = oracle.softcap_sigma(logits, 5.0, 7.5).double()
    z = 23.0 * sig
    p = torch.softmax(z, dim=1)
    want = grad_scale * (23.0 / 7.5) * (p - F.one_hot(targets, V)) * sig * (1 - sig)
    assert ((got - want).abs() <= 0.126 * want.abs() + grad_s * 2.0 ** -17).all()
    # against autograd of the un-rounded closed form: sigma rounding adds a few percent
    assert rel_err(got, lf.grad) < 0.1
    assert (torch.sign(got) == torch.sign(lf.grad))[got != 0].all()
    # finite differences in fp64 on the closed form
    eps = 1e-6
    base = float(oracle.softcap_ce_closed_form(logits.double(), targets).sum())
    for (i, j) in [(0, int(targets[0])), (3, 7), (11, 39)]:
        pert = logits.double().clone()
        pert[i, j] += eps
        fd = (float(oracle.softcap_ce_closed_form(pert, targets).sum()) - base) / eps * grad_scale
        assert abs(fd - float(lf.grad[i, j])) < 1e-4 * max(1.0, abs(fd))


def test_ce_mtp_prefix_and_invalid_targets(oracle):
    logits, targets = _ce_inputs(M=40, V=200, seed=10)
    M, V = logits.shape
    w = torch.tensor([1.0, 0.5, 0.25])
    nopre = torch.full((M,), -1)
    losses, dl, lse = oracle.ce_fwd_bwd(logits, targets, w, nopre, torch.zeros(1), M, 3, 23.0, 5.0, 7.5, 2.0 ** -10, 1.0)
    ref = oracle.softcap_ce_mtp_closed_form(logits, targets, w)
    assert (losses - ref).abs().max() < 3 * 23 * 2.0 ** -8
    # prefix term == an extra CE against prefix_targets with weight pw, where valid
    pt = torch.randint(-1, V, (M,), generator=torch.Generator().manual_seed(11))
    pw = torch.tensor([0.3])
    l2, dl2, _ = oracle.ce_fwd_bwd(logits, targets, w, pt, pw, M, 3, 23.0, 5.0, 7.5, 2.0 ** -10, 1.0)
    z = 23 * oracle.softcap_sigma(logits, 5.0, 7.5)
    extra = torch.where(pt >= 0, 0.3 * (lse - z[torch.arange(M), pt.clamp(0)]), torch.zeros(()))
    assert torch.allclose(l2, losses + extra, atol=1e-5)
    # out-of-range targets contribute nothing to the loss
    t_bad = targets.clone()
    t_bad[5], t_bad[6] = -3, V + 4
    l3, _, _ = oracle.ce_fwd_bwd(logits, t_bad, torch.tensor([1.0]), nopre, torch.zeros(1), M, 1, 23.0, 5.0, 7.5, 2.0 ** -10, 1.0)
    assert l3[5] == 0 and l3[6] == 0 and l3[7] != 0
    # gradient rows: sum_j dl/(coef*sigma') == S_w - sum of matched target weights (softmax sums to one)
    sig = oracle.softcap_sigma(logits, 5.0, 7.5)
    _, dl1, lse1 = oracle.ce_fwd_bwd(logits, targets, torch.tensor([1.0]), nopre, torch.zeros(1), M, 1, 23.0, 5.0, 7.5, 2.0 ** -10, 1.0)
    p = torch.exp(z - lse1[:, None])
    tgt = F.one_hot(targets, V).float()
    want = (23 / 7.5) / 2.0 ** -10 * (p - tgt) * sig * (1 - sig)
    assert rel_err(dl1.float(), want) < 0.08


def test_lm_head_ce_backward_matches_autograd(oracle):
    x, w, t, sc = oracle.make_cfg3(seed=12, M=96, K=64, V=384, n_tok=380)
    for layout in ("out_in", "in_out"):
        wl = w if layout == "out_in" else w.T.contiguous()
        losses, ctx = oracle.lm_head_ce_fwd(x, t, None, None, None, wl, sc["x_s"], sc["w_s"], sc["grad_s"],
                                            sc["grad_scale"], w_layout=layout)
        dx, dw = oracle.lm_head_ce_bwd(ctx)
        assert dw.shape == wl.shape and dw.is_contiguous() and dw.dtype == torch.float32
        xq = (ctx["x_f8"].double() * sc["x_s"]).requires_grad_()
        wq = (ctx["w_f8"].double() * sc["w_s"]).requires_grad_()
        logits = xq @ (wq.T if layout == "out_in" else wq)
        ref = oracle.softcap_ce_closed_form(logits, t)
        assert (losses - ref.detach()).abs().max() < 0.12     # bf16 logits + bf16 sigma
        assert abs(float(losses.mean() - ref.mean())) < 2e-2
        ref.sum().backward()
        # x_f8/w_f8 already carry the quantisation, so only e5m2(dl) and bf16 rounding remain
        assert rel_err(dx, xq.grad) < 0.06
        assert rel_err(dw, wq.grad) < 0.06
    # chunked evaluation == whole evaluation
    l_c, dx_c, dw_c, n = oracle.lm_head_ce_chunked(x, t, w, **sc, rows_per_chunk=40)
    losses, ctx = oracle.lm_head_ce_fwd(x, t, None, None, None, w, sc["x_s"], sc["w_s"], sc["grad_s"],
                                        sc["grad_scale"], w_layout="out_in")
    dx, dw = oracle.lm_head_ce_bwd(ctx)
    assert n == 96 and torch.allclose(l_c, losses, atol=1e-6) and torch.equal(dx_c, dx)
    assert rel_err(dw_c, dw) < 1e-6


def test_down_projection_requantiser_oracle(oracle):
    """quantize_transpose_mlp_down_weights / reduce_mlp_activation_scales against element-wise statements."""
    g = torch.Generator().manual_seed(13)
    L, H, D = 3, 192, 128
    w = (torch.randn(L, H, D, generator=g) * 0.02).bfloat16()
    scales = w.float().abs().amax(dim=(1, 2)) / 448 * 0.9          # a stale (too small) scale: some values clamp
    q_t, used, nxt, partial = oracle.quantize_transpose_mlp_down_weights(w, scales, headroom=1.12)
    assert q_t.shape == (L, D, H) and partial.shape == (L, 3 * 2) and torch.equal(used, scales)
    for l, h, d in [(0, 0, 0), (1, 100, 77), (2, 191, 127)]:
        want = max(-448.0, min(448.0, float(w[l, h, d]) / float(scales[l])))
        assert float(q_t[l, d, h]) == float(torch.tensor(want).to(torch.float8_e4m3fn))
    assert float(q_t.float().abs().max()) == 448.0                 # clamped, not NaN
    assert torch.isfinite(q_t.float()).all()
    assert torch.allclose(partial.amax(dim=1), w.float().abs().amax(dim=(1, 2)))
    assert torch.allclose(nxt, w.float().abs().amax(dim=(1, 2)) * 1.12 / 448)
    p = torch.tensor([[0.0, 3.0, 1.0], [0.0, 0.0, 0.0]])
    s = oracle.reduce_mlp_activation_scales(p, headroom=1.8)
    assert torch.allclose(s, torch.tensor([3.0 * 1.8 / 448, 1e-12 * 1.8 / 448]))


def test_ce_grad_columns_is_a_column_slice_of_ce_fwd_bwd(oracle):
    """ce_grad_columns (the checker of the full-size dW tests) must store exactly the codes ce_fwd_bwd stores
    in those columns -- target columns included -- given the rows' log-sum-exp."""
    for seed, scale, grad_s, grad_scale in ((14, 4.0, 0.75 / 448, 1.0), (15, 1.0, 2.0 ** -14, 3.0)):
        logits, targets = _ce_inputs(M=64, V=512, seed=seed, scale=scale)
        M, V = logits.shape
        targets[3], targets[9] = -1, V + 5                      # invalid targets contribute nothing
        losses, dl, lse = oracle.ce_fwd_bwd(logits, targets, torch.tensor([1.0]), torch.full((M,), -1), torch.zeros(1),
                                            M, 1, 23.0, 5.0, 7.5, grad_s, grad_scale)
        g = torch.Generator().manual_seed(seed)
        cols = torch.unique(torch.cat([torch.randperm(V, generator=g)[:96], targets[(targets >= 0) & (targets < V)][:40]]))
        hits = int((targets.unsqueeze(1) == cols.unsqueeze(0)).sum())
        assert hits >= 40                                        # the subset does contain target columns
        sub = oracle.ce_grad_columns(logits[:, cols].contiguous(), cols, lse, targets, 23.0, 5.0, 7.5, grad_s, grad_scale)
        assert sub.dtype == torch.float8_e5m2
        assert torch.equal(sub.view(torch.uint8), dl[:, cols].contiguous().view(torch.uint8))
        # a dropped one-hot term would change exactly the target entries
        wrong = oracle.ce_grad_columns(logits[:, cols].contiguous(), cols, lse, torch.full_like(targets, -1), 23.0, 5.0, 7.5,
                                       grad_s, grad_scale)
        assert int((wrong.view(torch.uint8) != sub.view(torch.uint8)).sum()) >= hits // 2


def _bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_mlp_quantisers_round_where_eager_rounds(oracle, oracle_c):
    """mlp_input_quant and quantize_up_weights are torch expressions; the scalar C restatement writes every rounding
    out (448.0 / amax is reciprocal() * 448 in eager, each bf16 operation rounds).  They must agree bit for bit, and
    the inputs are chosen so that the plausible mistakes (one division, no intermediate rounding) do change codes."""
    import ctypes
    differs_single_div = differs_no_round = 0
    for seed in range(12):
        g = torch.Generator().manual_seed(100 + seed)
        normed = oracle.rms_norm((torch.randn(64, 96, generator=g) * (1 + seed)).bfloat16())
        if seed == 11:
            normed = torch.zeros(8, 16).bfloat16()               # amax clamps to bf16(1e-12)
        up_scale = torch.tensor([0.0123 * (seed + 1)])
        x_f8, dequant = oracle.mlp_input_quant(normed, up_scale)
        n = normed.numel()
        out = np.empty(n, dtype=np.uint8)
        dq = ctypes.c_float(0)
        oracle_c.ngpt_oracle_mlp_input_quant(_bf16_bits(normed).ctypes.data, n, float(up_scale), out.ctypes.data, ctypes.byref(dq))
        assert np.array_equal(out, x_f8.view(torch.uint8).numpy().ravel()), seed
        assert dq.value == float(dequant), seed
        # the two mistakes this guards against
        amax = normed.float().abs().max().clamp(min=1e-12)
        one_div = (normed.float() * (448.0 / amax).bfloat16().float()).bfloat16().to(torch.float8_e4m3fn)
        no_round = (normed.float() * (448.0 / amax)).to(torch.float8_e4m3fn)
        differs_single_div += int(not torch.equal(one_div.view(torch.uint8), x_f8.view(torch.uint8)))
        differs_no_round += int(not torch.equal(no_round.view(torch.uint8), x_f8.view(torch.uint8)))
    assert differs_single_div >= 1 and differs_no_round >= 1

    g = torch.Generator().manual_seed(200)
    w = (torch.randn(5, 48, 64, generator=g) * torch.tensor([0.02, 0.5, 3.0, 1e-3, 0.0]).view(5, 1, 1)).bfloat16()
    w_f8, scales = oracle.quantize_up_weights(w)
    out = np.empty(w.numel(), dtype=np.uint8)
    sc = np.empty(5, dtype=np.float32)
    oracle_c.ngpt_oracle_quant_up_weights(_bf16_bits(w).ctypes.data, 5, 48 * 64, out.ctypes.data, sc.ctypes.data)
    assert np.array_equal(out, w_f8.view(torch.uint8).numpy().ravel())
    assert np.array_equal(sc, scales.numpy())
    no_round = (w.float() / (w.float().reshape(5, -1).abs().amax(1).clamp(min=1e-12) / 448).view(5, 1, 1)).to(torch.float8_e4m3fn)
    assert not torch.equal(no_round.view(torch.uint8), w_f8.view(torch.uint8))
