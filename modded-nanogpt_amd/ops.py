"""`torch.library` operators of the FP8 contraction path, under the reference's own names and
schemas, backed by libngpt_fp8.so (hand-written HIP for gfx950) through its C ABI.

    nanogpt::mm, nanogpt::mm_backward          reference train_gpt_medium.py:40-116
    nanogpt::mm_t, nanogpt::mm_t_backward      reference train_gpt.py:70-162
    nanogpt::ce_fwd_bwd                        reference triton_kernels.py:1182-1206
    nanogpt::lmhead_ce_fwd / _bwd              the fused lm_head + softcapped CE behind
                                               FusedSoftcappedCrossEntropy (no reference op: the
                                               reference materialises the logits instead)
    nanogpt::fc_relu2_fwd                      linear_relu_square(..., a_f8=, b_f8=), triton_kernels.py:576-665

Scales are Python floats in the schema (graph constants under torch.compile), every op has a
fake implementation reproducing shapes, dtypes and strides, and `mm` / `mm_t` carry the
reference's autograd contract (saved x_f8 / w_f8, `set_materialize_grads(False)`).
All tensors must live on the GPU: there is no CPU implementation behind these ops.
"""
from __future__ import annotations

import torch
from torch import Tensor

from . import _lib

E4M3 = torch.float8_e4m3fn
E5M2 = torch.float8_e5m2
MAX_PREDICT = _lib.MAX_PREDICT


def _gpu(*tensors: Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("nanogpt FP8 ops run on the GPU only (got a CPU tensor); "
                               "there is no CPU fallback")


def _p(t: Tensor | None):
    return None if t is None else t.data_ptr()


def _stream(t: Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _workspace(nbytes: int, device) -> Tensor:
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------------------------------------
# nanogpt::mm  (weight stored (out, in))

@torch.library.custom_op("nanogpt::mm", mutates_args=())
def mm_op(x: Tensor, w: Tensor, x_s: float, w_s: float, grad_s: float) -> tuple[Tensor, Tensor, Tensor]:
    assert x.is_contiguous() and w.is_contiguous()
    assert x.ndim == w.ndim == 2 and x.shape[1] == w.shape[1]
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    _gpu(x, w)
    lib = _lib.load()
    M, K = x.shape
    N = w.shape[0]
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    x_f8 = torch.empty((M, K), dtype=E4M3, device=x.device)
    w_f8 = torch.empty((N, K), dtype=E4M3, device=x.device)
    nws = lib.ngpt_mm_fwd_workspace_bytes(M, N, K, _lib.W_OUT_IN)      # 0 for shapes that stay on the tile kernel
    ws = _workspace(nws, x.device) if nws else None
    _lib.check(lib.ngpt_mm_fwd(_p(x), _p(w), M, N, K, x_s, w_s, _p(out), _p(x_f8), _p(w_f8),
                               _lib.W_OUT_IN, _p(ws) if nws else None, nws, _stream(x)), "ngpt_mm_fwd")
    return out, x_f8, w_f8


@mm_op.register_fake
def _(x: Tensor, w: Tensor, *_):
    assert x.ndim == w.ndim == 2
    assert x.shape[1] == w.shape[1]
    assert x.device == w.device
    assert x.is_contiguous() and w.is_contiguous()
    return x @ w.T, x.to(E4M3), w.to(E4M3)


@torch.library.custom_op("nanogpt::mm_backward", mutates_args=())
def mm_backward_op(g: Tensor, x_f8: Tensor, w_f8: Tensor, x_s: float, w_s: float, grad_s: float) -> tuple[Tensor, Tensor]:
    assert g.is_contiguous()
    _gpu(g, x_f8, w_f8)
    lib = _lib.load()
    M, N = g.shape
    K = x_f8.shape[1]
    assert x_f8.shape == (M, K) and w_f8.shape == (N, K)
    dx = torch.empty((M, K), dtype=torch.bfloat16, device=g.device)
    dw_kn = torch.empty((K, N), dtype=torch.float32, device=g.device)
    ws = _workspace(lib.ngpt_mm_bwd_workspace_bytes(M, N, K, _lib.W_OUT_IN), g.device)
    x_f8, w_f8 = x_f8.contiguous(), w_f8.contiguous()     # bound to names: the copies outlive the launch
    _lib.check(lib.ngpt_mm_bwd(_p(g), _p(x_f8), _p(w_f8), M, N, K, x_s, w_s, grad_s,
                               _p(dx), _p(dw_kn), _lib.W_OUT_IN, _p(ws), ws.numel(), _stream(g)), "ngpt_mm_bwd")
    return dx, dw_kn.T


@mm_backward_op.register_fake
def _(g: Tensor, x_f8: Tensor, w_f8: Tensor, *_):
    return x_f8.to(torch.bfloat16), w_f8.T.contiguous().T.to(torch.float32)


def _mm_backward(ctx, grad_out: Tensor, *_):
    x_f8, w_f8 = ctx.saved_tensors
    x_s, w_s, grad_s = ctx.scales
    grad_x, grad_w = torch.ops.nanogpt.mm_backward(grad_out, x_f8, w_f8, x_s, w_s, grad_s)
    return grad_x, grad_w, None, None, None


def _mm_setup_context(ctx: torch.autograd.function.FunctionCtx, inputs, output):
    *_, x_s, w_s, grad_s = inputs
    _, x_f8, w_f8 = output
    ctx.save_for_backward(x_f8, w_f8)
    ctx.scales = x_s, w_s, grad_s
    ctx.set_materialize_grads(False)


mm_op.register_autograd(_mm_backward, setup_context=_mm_setup_context)


# ------------------------------------------------------------------------------------------------
# nanogpt::mm_t  (weight stored (in, out))

@torch.library.custom_op("nanogpt::mm_t", mutates_args=())
def mm_t_op(x: Tensor, w: Tensor, x_s: float, w_s: float, grad_s: float) -> tuple[Tensor, Tensor, Tensor]:
    """Computes y = x @ w with F8 weights stored as (in_features, out_features)."""
    assert x.is_contiguous() and w.is_contiguous()
    assert x.ndim == w.ndim == 2 and x.shape[1] == w.shape[0]
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    _gpu(x, w)
    lib = _lib.load()
    M, K = x.shape
    N = w.shape[1]
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    x_f8 = torch.empty((M, K), dtype=E4M3, device=x.device)
    w_f8 = torch.empty((K, N), dtype=E4M3, device=x.device)
    ws = _workspace(lib.ngpt_mm_fwd_workspace_bytes(M, N, K, _lib.W_IN_OUT), x.device)
    _lib.check(lib.ngpt_mm_fwd(_p(x), _p(w), M, N, K, x_s, w_s, _p(out), _p(x_f8), _p(w_f8),
                               _lib.W_IN_OUT, _p(ws), ws.numel(), _stream(x)), "ngpt_mm_fwd")
    return out, x_f8, w_f8


@mm_t_op.register_fake
def _(x: Tensor, w: Tensor, *_):
    assert x.ndim == w.ndim == 2
    assert x.shape[1] == w.shape[0]
    assert x.device == w.device
    assert x.is_contiguous() and w.is_contiguous()
    return x @ w, x.to(E4M3), w.to(E4M3)


@torch.library.custom_op("nanogpt::mm_t_backward", mutates_args=())
def mm_t_backward_op(g: Tensor, x_f8: Tensor, w_f8: Tensor, x_s: float, w_s: float, grad_s: float) -> tuple[Tensor, Tensor]:
    assert g.is_contiguous()
    _gpu(g, x_f8, w_f8)
    lib = _lib.load()
    M, N = g.shape
    K = x_f8.shape[1]
    assert x_f8.shape == (M, K) and w_f8.shape == (K, N)
    dx = torch.empty((M, K), dtype=torch.bfloat16, device=g.device)
    dw = torch.empty((K, N), dtype=torch.float32, device=g.device)
    ws = _workspace(lib.ngpt_mm_bwd_workspace_bytes(M, N, K, _lib.W_IN_OUT), g.device)
    x_f8, w_f8 = x_f8.contiguous(), w_f8.contiguous()     # bound to names: the copies outlive the launch
    _lib.check(lib.ngpt_mm_bwd(_p(g), _p(x_f8), _p(w_f8), M, N, K, x_s, w_s, grad_s,
                               _p(dx), _p(dw), _lib.W_IN_OUT, _p(ws), ws.numel(), _stream(g)), "ngpt_mm_bwd")
    return dx, dw


@mm_t_backward_op.register_fake
def _(g: Tensor, x_f8: Tensor, w_f8: Tensor, *_):
    return x_f8.to(torch.bfloat16), w_f8.to(torch.float32)


def _mm_t_backward(ctx, grad_out: Tensor, *_):
    x_f8, w_f8 = ctx.saved_tensors
    x_s, w_s, grad_s = ctx.scales
    grad_x, grad_w = torch.ops.nanogpt.mm_t_backward(grad_out, x_f8, w_f8, x_s, w_s, grad_s)
    return grad_x, grad_w, None, None, None


mm_t_op.register_autograd(_mm_t_backward, setup_context=_mm_setup_context)


# ------------------------------------------------------------------------------------------------
# nanogpt::ce_fwd_bwd  (logits materialised by the caller)

@torch.library.custom_op("nanogpt::ce_fwd_bwd", mutates_args={"losses", "grad_input"})
def ce_fwd_bwd(
    logits: Tensor,
    targets: Tensor,
    mtp_weights: Tensor,
    prefix_targets: Tensor,
    prefix_weight: Tensor,
    losses: Tensor,
    grad_input: Tensor,
    n_rows: int,
    n_predict: int,
    A: float,
    B: float,
    C: float,
    grad_s: float,
    grad_scale: float,
) -> None:
    _gpu(logits, targets, mtp_weights, prefix_targets, prefix_weight, losses, grad_input)
    assert logits.dtype == torch.bfloat16 and logits.is_contiguous() and logits.ndim == 2
    assert logits.shape[0] == n_rows and grad_input.shape == logits.shape
    assert targets.dtype == torch.int64 and prefix_targets.dtype == torch.int64
    assert mtp_weights.dtype == torch.float32 and mtp_weights.numel() >= n_predict
    assert losses.dtype == torch.float32 and grad_input.dtype == E5M2 and grad_input.is_contiguous()
    lib = _lib.load()
    ws = _workspace(lib.ngpt_ce_fwd_bwd_workspace_bytes(), logits.device)
    _lib.check(lib.ngpt_ce_fwd_bwd(_p(logits), _p(targets), _p(mtp_weights), _p(prefix_targets),
                                   _p(prefix_weight), _p(losses), _p(grad_input), n_rows, logits.shape[1],
                                   n_predict, A, B, C, grad_s, grad_scale, _p(ws), ws.numel(),
                                   _stream(logits)), "ngpt_ce_fwd_bwd")


@ce_fwd_bwd.register_fake
def _(logits, targets, mtp_weights, prefix_targets, prefix_weight, losses, grad_input, *_):
    return None


# ------------------------------------------------------------------------------------------------
# Fused lm_head + softcapped CE (the logits are never stored)

@torch.library.custom_op("nanogpt::lmhead_ce_fwd", mutates_args=())
def lmhead_ce_fwd(x: Tensor, w: Tensor, targets: Tensor, mtp_weights: Tensor, prefix_targets: Tensor,
                  prefix_weight: Tensor, x_s: float, w_s: float, A: float, B: float, C: float,
                  w_in_out: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    """-> (losses [M] f32, lse [M] f32, saved_sigma [MAX_PREDICT+1, M] f32, x_f8 [M,K], w_f8 [V,K])."""
    _gpu(x, w, targets, mtp_weights, prefix_targets, prefix_weight)
    assert x.is_contiguous() and w.is_contiguous() and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    assert targets.dtype == torch.int64 and prefix_targets.dtype == torch.int64
    lib = _lib.load()
    M, K = x.shape
    V = w.shape[1] if w_in_out else w.shape[0]
    assert (w.shape[0] if w_in_out else w.shape[1]) == K
    n_predict = mtp_weights.shape[0]
    dev = x.device
    losses = torch.empty(M, dtype=torch.float32, device=dev)
    lse = torch.empty(M, dtype=torch.float32, device=dev)
    saved_sigma = torch.empty((MAX_PREDICT + 1, M), dtype=torch.float32, device=dev)     # zeroed by the library
    x_f8 = torch.empty((M, K), dtype=E4M3, device=dev)
    w_f8 = torch.empty((V, K), dtype=E4M3, device=dev)
    layout = _lib.W_IN_OUT if w_in_out else _lib.W_OUT_IN
    ws = _workspace(lib.ngpt_lmhead_ce_fwd_workspace_bytes(M, K, V, layout), dev)
    _lib.check(lib.ngpt_lmhead_ce_fwd(_p(x), _p(w), _p(targets), _p(mtp_weights), n_predict,
                                      _p(prefix_targets), _p(prefix_weight), M, K, V, x_s, w_s, A, B, C,
                                      _p(losses), _p(lse), _p(saved_sigma), _p(x_f8), _p(w_f8), layout,
                                      _p(ws), ws.numel(), _stream(x)), "ngpt_lmhead_ce_fwd")
    return losses, lse, saved_sigma, x_f8, w_f8


@lmhead_ce_fwd.register_fake
def _(x, w, targets, mtp_weights, prefix_targets, prefix_weight, x_s, w_s, A, B, C, w_in_out):
    M, K = x.shape
    V = w.shape[1] if w_in_out else w.shape[0]
    f32 = dict(dtype=torch.float32, device=x.device)
    return (torch.empty(M, **f32), torch.empty(M, **f32), torch.empty((MAX_PREDICT + 1, M), **f32),
            torch.empty((M, K), dtype=E4M3, device=x.device), torch.empty((V, K), dtype=E4M3, device=x.device))


@torch.library.custom_op("nanogpt::lmhead_ce_bwd", mutates_args=())
def lmhead_ce_bwd(x_f8: Tensor, w_f8: Tensor, targets: Tensor, mtp_weights: Tensor, prefix_targets: Tensor,
                  prefix_weight: Tensor, lse: Tensor, saved_sigma: Tensor, x_s: float, w_s: float,
                  grad_s: float, grad_scale: float, A: float, B: float, C: float,
                  w_in_out: bool) -> tuple[Tensor, Tensor]:
    """-> (dx [M,K] bf16, dW fp32 in the weight's layout)."""
    _gpu(x_f8, w_f8, targets, lse, saved_sigma)
    lib = _lib.load()
    M, K = x_f8.shape
    V = w_f8.shape[0]
    dev = x_f8.device
    dx = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    dw = torch.empty((K, V) if w_in_out else (V, K), dtype=torch.float32, device=dev)
    layout = _lib.W_IN_OUT if w_in_out else _lib.W_OUT_IN
    ws = _workspace(lib.ngpt_lmhead_ce_bwd_workspace_bytes(M, K, V, layout), dev)
    _lib.check(lib.ngpt_lmhead_ce_bwd(_p(x_f8), _p(w_f8), _p(targets), _p(mtp_weights), mtp_weights.shape[0],
                                      _p(prefix_targets), _p(prefix_weight), _p(lse), _p(saved_sigma),
                                      M, K, V, x_s, w_s, grad_s, grad_scale, A, B, C, _p(dx), _p(dw), layout,
                                      _p(ws), ws.numel(), _stream(x_f8)), "ngpt_lmhead_ce_bwd")
    return dx, dw


@lmhead_ce_bwd.register_fake
def _(x_f8, w_f8, targets, mtp_weights, prefix_targets, prefix_weight, lse, saved_sigma,
      x_s, w_s, grad_s, grad_scale, A, B, C, w_in_out):
    M, K = x_f8.shape
    V = w_f8.shape[0]
    return (torch.empty((M, K), dtype=torch.bfloat16, device=x_f8.device),
            torch.empty((K, V) if w_in_out else (V, K), dtype=torch.float32, device=x_f8.device))


# The same pair with the softcap's output kept between forward and backward instead of recomputed: one byte per
# logit, the 8-bit code of bf16(sigmoid(..)) -- the reference keeps one byte per logit too, its e5m2 gradient
# (triton_kernels.py:1231-1253) -- and never the logits.  The backward rebuilds the e5m2 gradient from the codes,
# bit-identical to the recomputed one, and skips the second logits GEMM.

@torch.library.custom_op("nanogpt::lmhead_ce_fwd_codes", mutates_args=())
def lmhead_ce_fwd_codes(x: Tensor, w: Tensor, targets: Tensor, mtp_weights: Tensor, prefix_targets: Tensor,
                        prefix_weight: Tensor, x_s: float, w_s: float, A: float, B: float, C: float,
                        w_in_out: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor]:
    """-> (losses, lse, saved_sigma, x_f8, w_f8 as lmhead_ce_fwd, sigma_codes uint8 [ceil256(M) * ceil256(V)])."""
    _gpu(x, w, targets, mtp_weights, prefix_targets, prefix_weight)
    assert x.is_contiguous() and w.is_contiguous() and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    assert targets.dtype == torch.int64 and prefix_targets.dtype == torch.int64
    lib = _lib.load()
    M, K = x.shape
    V = w.shape[1] if w_in_out else w.shape[0]
    assert (w.shape[0] if w_in_out else w.shape[1]) == K
    n_predict = mtp_weights.shape[0]
    dev = x.device
    losses = torch.empty(M, dtype=torch.float32, device=dev)
    lse = torch.empty(M, dtype=torch.float32, device=dev)
    saved_sigma = torch.empty((MAX_PREDICT + 1, M), dtype=torch.float32, device=dev)     # zeroed by the library
    x_f8 = torch.empty((M, K), dtype=E4M3, device=dev)
    w_f8 = torch.empty((V, K), dtype=E4M3, device=dev)
    codes = torch.empty(lib.ngpt_lmhead_ce_codes_bytes(M, V), dtype=torch.uint8, device=dev)
    layout = _lib.W_IN_OUT if w_in_out else _lib.W_OUT_IN
    ws = _workspace(lib.ngpt_lmhead_ce_fwd_workspace_bytes(M, K, V, layout), dev)
    _lib.check(lib.ngpt_lmhead_ce_fwd_codes(_p(x), _p(w), _p(targets), _p(mtp_weights), n_predict,
                                            _p(prefix_targets), _p(prefix_weight), M, K, V, x_s, w_s, A, B, C,
                                            _p(losses), _p(lse), _p(saved_sigma), _p(x_f8), _p(w_f8), _p(codes), layout,
                                            _p(ws), ws.numel(), _stream(x)), "ngpt_lmhead_ce_fwd_codes")
    return losses, lse, saved_sigma, x_f8, w_f8, codes


@lmhead_ce_fwd_codes.register_fake
def _(x, w, targets, mtp_weights, prefix_targets, prefix_weight, x_s, w_s, A, B, C, w_in_out):
    M, K = x.shape
    V = w.shape[1] if w_in_out else w.shape[0]
    f32 = dict(dtype=torch.float32, device=x.device)
    ncodes = (-(-M // 256) * 256) * (-(-V // 256) * 256)
    return (torch.empty(M, **f32), torch.empty(M, **f32), torch.empty((MAX_PREDICT + 1, M), **f32),
            torch.empty((M, K), dtype=E4M3, device=x.device), torch.empty((V, K), dtype=E4M3, device=x.device),
            torch.empty(ncodes, dtype=torch.uint8, device=x.device))


@torch.library.custom_op("nanogpt::lmhead_ce_bwd_codes", mutates_args=())
def lmhead_ce_bwd_codes(x_f8: Tensor, w_f8: Tensor, targets: Tensor, mtp_weights: Tensor, prefix_targets: Tensor,
                        prefix_weight: Tensor, lse: Tensor, saved_sigma: Tensor, sigma_codes: Tensor,
                        x_s: float, w_s: float, grad_s: float, grad_scale: float, A: float, B: float, C: float,
                        w_in_out: bool) -> tuple[Tensor, Tensor]:
    """-> (dx [M,K] bf16, dW fp32 in the weight's layout), from the forward's sigma codes."""
    _gpu(x_f8, w_f8, targets, lse, saved_sigma, sigma_codes)
    lib = _lib.load()
    M, K = x_f8.shape
    V = w_f8.shape[0]
    assert sigma_codes.dtype == torch.uint8 and sigma_codes.is_contiguous()
    assert sigma_codes.numel() >= lib.ngpt_lmhead_ce_codes_bytes(M, V)
    dev = x_f8.device
    dx = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    dw = torch.empty((K, V) if w_in_out else (V, K), dtype=torch.float32, device=dev)
    layout = _lib.W_IN_OUT if w_in_out else _lib.W_OUT_IN
    ws = _workspace(lib.ngpt_lmhead_ce_bwd_workspace_bytes(M, K, V, layout), dev)
    _lib.check(lib.ngpt_lmhead_ce_bwd_codes(_p(x_f8), _p(w_f8), _p(targets), _p(mtp_weights), mtp_weights.shape[0],
                                            _p(prefix_targets), _p(prefix_weight), _p(lse), _p(saved_sigma), _p(sigma_codes),
                                            M, K, V, x_s, w_s, grad_s, grad_scale, A, B, C, _p(dx), _p(dw), layout,
                                            _p(ws), ws.numel(), _stream(x_f8)), "ngpt_lmhead_ce_bwd_codes")
    return dx, dw


@lmhead_ce_bwd_codes.register_fake
def _(x_f8, w_f8, targets, mtp_weights, prefix_targets, prefix_weight, lse, saved_sigma, sigma_codes,
      x_s, w_s, grad_s, grad_scale, A, B, C, w_in_out):
    M, K = x_f8.shape
    V = w_f8.shape[0]
    return (torch.empty((M, K), dtype=torch.bfloat16, device=x_f8.device),
            torch.empty((K, V) if w_in_out else (V, K), dtype=torch.float32, device=x_f8.device))


# ------------------------------------------------------------------------------------------------
# FP8 up-projection + ReLU^2

@torch.library.custom_op("nanogpt::fc_relu2_fwd", mutates_args=())
def fc_relu2_fwd(x_f8: Tensor, w_f8: Tensor, dequant_scale: Tensor) -> Tensor:
    """post [M,N] bf16 = relu(bf16(x_f8 . w_f8^T * dequant))^2."""
    _gpu(x_f8, w_f8, dequant_scale)
    assert x_f8.is_contiguous() and w_f8.is_contiguous() and x_f8.dtype == E4M3 and w_f8.dtype == E4M3
    assert dequant_scale.dtype == torch.float32 and dequant_scale.numel() >= 1
    lib = _lib.load()
    M, K = x_f8.shape
    N = w_f8.shape[0]
    post = torch.empty((M, N), dtype=torch.bfloat16, device=x_f8.device)
    ws = _workspace(lib.ngpt_fc_relu2_fwd_workspace_bytes(M, N, K), x_f8.device)
    _lib.check(lib.ngpt_fc_relu2_fwd_ws(_p(x_f8), _p(w_f8), _p(dequant_scale), M, N, K, _p(post), None, None,
                                        None, 0, _p(ws), ws.numel(), _stream(x_f8)), "ngpt_fc_relu2_fwd")
    return post


@fc_relu2_fwd.register_fake
def _(x_f8, w_f8, dequant_scale):
    return torch.empty((x_f8.shape[0], w_f8.shape[0]), dtype=torch.bfloat16, device=x_f8.device)


@torch.library.custom_op("nanogpt::fc_relu2_fwd_emit", mutates_args={"partial_amax"})
def fc_relu2_fwd_emit(x_f8: Tensor, w_f8: Tensor, dequant_scale: Tensor, activation_scale: Tensor,
                      partial_amax: Tensor) -> tuple[Tensor, Tensor]:
    """As fc_relu2_fwd, plus post_f8 = e4m3(min(post / activation_scale, 448)) and the
    per-workgroup running max of post in partial_amax."""
    _gpu(x_f8, w_f8, dequant_scale, activation_scale, partial_amax)
    assert x_f8.is_contiguous() and w_f8.is_contiguous() and partial_amax.is_contiguous()
    assert partial_amax.dtype == torch.float32 and activation_scale.dtype == torch.float32
    lib = _lib.load()
    M, K = x_f8.shape
    N = w_f8.shape[0]
    post = torch.empty((M, N), dtype=torch.bfloat16, device=x_f8.device)
    post_f8 = torch.empty((M, N), dtype=E4M3, device=x_f8.device)
    ws = _workspace(lib.ngpt_fc_relu2_fwd_workspace_bytes(M, N, K), x_f8.device)
    _lib.check(lib.ngpt_fc_relu2_fwd_ws(_p(x_f8), _p(w_f8), _p(dequant_scale), M, N, K, _p(post), _p(post_f8),
                                        _p(activation_scale), _p(partial_amax), partial_amax.numel(),
                                        _p(ws), ws.numel(), _stream(x_f8)), "ngpt_fc_relu2_fwd")
    return post, post_f8


@fc_relu2_fwd_emit.register_fake
def _(x_f8, w_f8, dequant_scale, activation_scale, partial_amax):
    M, N = x_f8.shape[0], w_f8.shape[0]
    return (torch.empty((M, N), dtype=torch.bfloat16, device=x_f8.device),
            torch.empty((M, N), dtype=E4M3, device=x_f8.device))


@torch.library.custom_op("nanogpt::linear_relu2_bf16", mutates_args=())
def linear_relu2_bf16(x: Tensor, w: Tensor) -> Tensor:
    """post [M,N] bf16 = relu(bf16(x @ w.T))^2 for bf16 x [M,K], w [N,K]: linear_relu_square without fp8 copies."""
    _gpu(x, w)
    assert x.dtype == w.dtype == torch.bfloat16 and x.is_contiguous() and w.is_contiguous()
    M, K = x.shape
    N = w.shape[0]
    assert w.shape[1] == K
    post = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _lib.check(_lib.load().ngpt_linear_relu2_bf16(_p(x), _p(w), M, N, K, _p(post), _stream(x)), "ngpt_linear_relu2_bf16")
    return post


@linear_relu2_bf16.register_fake
def _(x, w):
    return torch.empty((x.shape[0], w.shape[0]), dtype=torch.bfloat16, device=x.device)


@torch.library.custom_op("nanogpt::gemm_bf16", mutates_args=())
def gemm_bf16(a: Tensor, b: Tensor, a_k_rows: bool, b_k_rows: bool) -> Tensor:
    """out [R, C] bf16 = sum_k A(r, k) B(c, k) with fp32 accumulation and one rounding.  `a` is stored [R, K], or
    [K, R] when a_k_rows (the contraction index is its row); `b` likewise [C, K] or [K, C].  The four plain products
    of FusedLinearReLUSquareFunction (reference triton_kernels.py:715, 723, 727, 728):
        post @ W2      = gemm_bf16(post, W2, False, True)       dpre @ W1 = gemm_bf16(dpre, W1, False, True)
        post.T @ dY    = gemm_bf16(post, dY, True, True)        dpre.T @ x = gemm_bf16(dpre, x, True, True)"""
    _gpu(a, b)
    assert a.dtype == b.dtype == torch.bfloat16 and a.ndim == b.ndim == 2 and a.stride(1) == 1 and b.stride(1) == 1
    K, R = a.shape if a_k_rows else a.shape[::-1]
    Kb, C = b.shape if b_k_rows else b.shape[::-1]
    assert K == Kb, "contraction lengths differ"
    lib = _lib.load()
    out = torch.empty((R, C), dtype=torch.bfloat16, device=a.device)
    ws = _workspace(lib.ngpt_gemm_bf16_workspace_bytes(R, C, K), a.device)
    _lib.check(lib.ngpt_gemm_bf16(_p(a), _lib.K_ROWS if a_k_rows else _lib.K_CONTIGUOUS, a.stride(0),
                                  _p(b), _lib.K_ROWS if b_k_rows else _lib.K_CONTIGUOUS, b.stride(0),
                                  R, C, K, _p(out), C, _p(ws), ws.numel(), _stream(a)), "ngpt_gemm_bf16")
    return out


@gemm_bf16.register_fake
def _(a, b, a_k_rows, b_k_rows):
    R = a.shape[1] if a_k_rows else a.shape[0]
    C = b.shape[1] if b_k_rows else b.shape[0]
    return a.new_empty((R, C))


@torch.library.custom_op("nanogpt::fc_relu2_bwd_dpre", mutates_args=())
def fc_relu2_bwd_dpre(dy: Tensor, w2: Tensor, post: Tensor) -> Tensor:
    """dpre [M,H] = bf16(2 * bf16(dy @ w2.T) * sqrt(post)) for dy [M,D], w2 [H,D], post [M,H], all bf16."""
    _gpu(dy, w2, post)
    assert dy.dtype == w2.dtype == post.dtype == torch.bfloat16
    assert dy.is_contiguous() and w2.is_contiguous() and post.is_contiguous()
    M, D = dy.shape
    H = w2.shape[0]
    assert w2.shape[1] == D and post.shape == (M, H)
    dpre = torch.empty((M, H), dtype=torch.bfloat16, device=dy.device)
    _lib.check(_lib.load().ngpt_fc_relu2_bwd_dpre(_p(dy), _p(w2), _p(post), M, H, D, _p(dpre), _stream(dy)),
               "ngpt_fc_relu2_bwd_dpre")
    return dpre


@fc_relu2_bwd_dpre.register_fake
def _(dy, w2, post):
    return torch.empty_like(post)


# ------------------------------------------------------------------------------------------------
# MLP input producer (reference train_gpt.py:1643-1647) and the up-projection weight quantiser (:1419-1422)

@torch.library.custom_op("nanogpt::mlp_input_quant", mutates_args=())
def mlp_input_quant(x: Tensor, up_scale: Tensor) -> tuple[Tensor, Tensor, Tensor]:
    """(normed, x_f8, dequant) = (rms_norm(x), e4m3(normed * (448.0 / amax(|normed|))), up_scale * amax / 448) for
    bf16 x [..., D]; dequant is a 1-element fp32 device tensor (what the reference keeps in
    `_mlp_dequant_scale_buf`).  Nothing synchronises with the host."""
    _gpu(x, up_scale)
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    assert up_scale.dtype == torch.float32 and up_scale.numel() >= 1
    dequant = torch.empty(1, dtype=torch.float32, device=x.device)
    dim = x.shape[-1]
    rows = x.numel() // dim
    lib = _lib.load()
    normed = torch.empty_like(x)
    x_f8 = torch.empty(x.shape, dtype=E4M3, device=x.device)
    nbytes = lib.ngpt_mlp_input_quant_workspace_bytes()
    ws = _workspace(nbytes, x.device)
    _lib.check(lib.ngpt_mlp_input_quant(_p(x), rows, dim, _p(up_scale), _p(normed), _p(x_f8), _p(dequant), _p(ws), nbytes,
                                        _stream(x)), "ngpt_mlp_input_quant")
    return normed, x_f8, dequant


@mlp_input_quant.register_fake
def _(x, up_scale):
    return (torch.empty_like(x), torch.empty(x.shape, dtype=E4M3, device=x.device),
            torch.empty(1, dtype=torch.float32, device=x.device))


@torch.library.custom_op("nanogpt::rms_norm_backward", mutates_args=())
def rms_norm_backward(g: Tensor, x: Tensor) -> Tensor:
    """dx of y = F.rms_norm(x, (D,)) for the incoming gradient g: bf16 in and out, fp32 arithmetic."""
    _gpu(g, x)
    assert x.dtype == torch.bfloat16 and g.dtype == torch.bfloat16 and x.shape == g.shape
    x, g = x.contiguous(), g.contiguous()
    dim = x.shape[-1]
    dx = torch.empty_like(x)
    _lib.check(_lib.load().ngpt_rmsnorm_bwd(_p(x), _p(g), x.numel() // dim, dim, _p(dx), _stream(x)), "ngpt_rmsnorm_bwd")
    return dx


@rms_norm_backward.register_fake
def _(g, x):
    return torch.empty_like(x)


def _mlp_input_quant_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[0])
    ctx.set_materialize_grads(False)     # no zero tensors for the fp8 copy and the scale, which carry no gradient


def _mlp_input_quant_backward(ctx, d_normed, d_x_f8, d_dequant):
    # x_f8 and dequant come from detached values in the reference; the gradient flows through the norm only
    (x,) = ctx.saved_tensors
    if d_normed is None:
        return None, None
    return torch.ops.nanogpt.rms_norm_backward(d_normed, x), None


mlp_input_quant.register_autograd(_mlp_input_quant_backward, setup_context=_mlp_input_quant_setup)


@torch.library.custom_op("nanogpt::quant_up_weights", mutates_args=())
def quant_up_weights(w: Tensor) -> tuple[Tensor, Tensor]:
    """Per-layer e4m3 copy of w [L, ...] bf16 with scales[l] = amax(|w[l]|).clamp(1e-12) / 448 (fp32 [L])."""
    _gpu(w)
    assert w.dtype == torch.bfloat16 and w.is_contiguous() and w.ndim >= 2
    layers = w.shape[0]
    per_layer = w.numel() // layers
    lib = _lib.load()
    w_f8 = torch.empty(w.shape, dtype=E4M3, device=w.device)
    scales = torch.empty(layers, dtype=torch.float32, device=w.device)
    nbytes = lib.ngpt_quant_up_weights_workspace_bytes(layers)
    ws = _workspace(nbytes, w.device)
    _lib.check(lib.ngpt_quant_up_weights(_p(w), layers, per_layer, _p(w_f8), _p(scales), _p(ws), nbytes, _stream(w)),
               "ngpt_quant_up_weights")
    return w_f8, scales


@quant_up_weights.register_fake
def _(w):
    return torch.empty(w.shape, dtype=E4M3, device=w.device), torch.empty(w.shape[0], dtype=torch.float32, device=w.device)


# ------------------------------------------------------------------------------------------------
# Building blocks exposed for callers and tests (plain functions, not registered ops)

def quant_fp8(x: Tensor, scale: float, dtype: torch.dtype = E4M3) -> Tensor:
    """`x.div(scale).to(dtype)` for a contiguous bf16 tensor, on the GPU."""
    _gpu(x)
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    fmt = _lib.E4M3 if dtype == E4M3 else _lib.E5M2
    _lib.check(_lib.load().ngpt_quant_fp8(_p(x), _p(out), x.numel(), scale, fmt, _stream(x)), "ngpt_quant_fp8")
    return out


def quant_fp8_2d(x: Tensor, scale: float, dtype: torch.dtype = E4M3, want_rowmajor=True, want_transposed=True):
    _gpu(x)
    assert x.dtype == torch.bfloat16 and x.is_contiguous() and x.ndim == 2
    R, C = x.shape
    out = torch.empty((R, C), dtype=dtype, device=x.device) if want_rowmajor else None
    out_t = torch.empty((C, R), dtype=dtype, device=x.device) if want_transposed else None
    fmt = _lib.E4M3 if dtype == E4M3 else _lib.E5M2
    _lib.check(_lib.load().ngpt_quant_fp8_2d(_p(x), R, C, scale, fmt, _p(out), _p(out_t), _stream(x)),
               "ngpt_quant_fp8_2d")
    return out, out_t


def gemm_fp8_tn(a: Tensor, b: Tensor, scale: float, out_dtype=torch.bfloat16, out: Tensor | None = None,
                accumulate: bool = False) -> Tensor:
    """C[r,c] = scale * sum_k a[r,k] b[c,k] for fp8 a [R,K], b [C,K] (contraction contiguous)."""
    _gpu(a, b)
    fmt = {E4M3: _lib.E4M3, E5M2: _lib.E5M2}
    R, K = a.shape
    Cn = b.shape[0]
    assert b.shape[1] == K and a.stride(1) == 1 and b.stride(1) == 1
    if out is None:
        out = torch.empty((R, Cn), dtype=out_dtype, device=a.device)
    kind = 0 if out.dtype == torch.bfloat16 else (2 if accumulate else 1)
    _lib.check(_lib.load().ngpt_gemm_fp8_tn(_p(a), fmt[a.dtype], a.stride(0), _p(b), fmt[b.dtype], b.stride(0),
                                            R, Cn, K, scale, _p(out), out.stride(0), kind, _stream(a)),
               "ngpt_gemm_fp8_tn")
    return out


@torch.library.custom_op("nanogpt::gemm_fp8_scaled", mutates_args=())
def gemm_fp8_scaled(a: Tensor, b: Tensor, scale_a: Tensor, scale_b: Tensor) -> Tensor:
    """bf16 [R, C] = (a [R, K] fp8) @ (b [C, K] fp8).T * (scale_a * scale_b) with both scales 1-element fp32 device
    tensors read by the kernel: `torch._scaled_mm(post_f8, W2_f8, scale_a=activation_scale, scale_b=W2_scale,
    out_dtype=bf16)`, the FP8 down projection (reference triton_kernels.py:706-713), in one launch."""
    _gpu(a, b, scale_a, scale_b)
    fmt = {E4M3: _lib.E4M3, E5M2: _lib.E5M2}
    R, K = a.shape
    Cn = b.shape[0]
    assert b.shape[1] == K and a.stride(1) == 1 and b.stride(1) == 1
    assert scale_a.dtype == torch.float32 and scale_b.dtype == torch.float32 and scale_a.numel() >= 1 and scale_b.numel() >= 1
    lib = _lib.load()
    out = torch.empty((R, Cn), dtype=torch.bfloat16, device=a.device)
    ws = _workspace(lib.ngpt_gemm_fp8_scaled_workspace_bytes(R, Cn, K), a.device)
    _lib.check(lib.ngpt_gemm_fp8_scaled(_p(a), fmt[a.dtype], a.stride(0), _p(b), fmt[b.dtype], b.stride(0), R, Cn, K,
                                        _p(scale_a), _p(scale_b), _p(out), Cn, _p(ws), ws.numel(), _stream(a)),
               "ngpt_gemm_fp8_scaled")
    return out


@gemm_fp8_scaled.register_fake
def _(a, b, scale_a, scale_b):
    assert a.ndim == 2 and b.ndim == 2 and a.shape[1] == b.shape[1]
    return a.new_empty((a.shape[0], b.shape[0]), dtype=torch.bfloat16)


@torch.library.custom_op("nanogpt::gemm_fp8_tn", mutates_args=())
def gemm_fp8_tn_op(a: Tensor, b: Tensor, scale: float, out_f32: bool) -> Tensor:
    """`gemm_fp8_tn` as a registered operator, for callers that run under `torch.compile(fullgraph=True)`
    (the FP8 down projection inside `FusedLinearReLUSquareFunction`, reference triton_kernels.py:706-713)."""
    return gemm_fp8_tn(a, b, scale, out_dtype=torch.float32 if out_f32 else torch.bfloat16)


@gemm_fp8_tn_op.register_fake
def _(a, b, scale, out_f32):
    assert a.ndim == 2 and b.ndim == 2 and a.shape[1] == b.shape[1]
    return a.new_empty((a.shape[0], b.shape[0]), dtype=torch.float32 if out_f32 else torch.bfloat16)
