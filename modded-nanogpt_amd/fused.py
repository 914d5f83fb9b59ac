"""The two autograd functions the reference model calls, with identical `apply` signatures:

    FusedLinearReLUSquareFunction   reference triton_kernels.py:667-729 (alias ReLUSqrdMLP, train_gpt.py:48)
    FusedSoftcappedCrossEntropy     reference triton_kernels.py:1208-1292

plus the launch wrappers the reference exports beside them (`linear_relu_square`,
`transpose_copy`).  `train_gpt.py:42` imports these names from a module called
`triton_kernels`; this module exports the same names.
"""
from __future__ import annotations

import torch
from torch import Tensor

import os

from . import _lib, ops

E4M3 = torch.float8_e4m3fn

# Where the backward of FusedSoftcappedCrossEntropy takes the e5m2 gradient of the logits from:
#   "codes"      the forward keeps one byte per logit, the 8-bit code of bf16(sigmoid(..)) (the reference keeps one
#                byte per logit as well, the e5m2 gradient itself; the logits are never stored), and the backward
#                rebuilds the gradient from it: three GEMM passes per step;
#   "recompute"  nothing of size [tokens, vocabulary] is kept and the backward runs the logits GEMM again: four passes.
# Given the same row statistics (lse, saved sigmas) both produce the same e5m2 gradient bytes, hence bit-identical dx / dW;
# through this function the two forwards sum the exponentials of a row in different orders and with table entries that
# differ in their last mantissa bits (the code-carrying ones), so lse and with it the gradients agree to about 1e-5 relative.
# Set before the forward runs (module attribute or NGPT_CE_BACKWARD).
CE_BACKWARD = os.environ.get("NGPT_CE_BACKWARD", "codes")
assert CE_BACKWARD in ("codes", "recompute"), f"NGPT_CE_BACKWARD={CE_BACKWARD!r}: expected 'codes' or 'recompute'"


def transpose_copy(src: Tensor, dst: Tensor) -> None:
    """dst (N, M) = src (M, N).T for any element type of 1, 2 or 4 bytes -- reference triton_kernels.py:819-841
    (called on the fp8 operands and, by the optimizer, on the bf16 tied weights, train_gpt.py:808-810)."""
    assert src.ndim == 2 and dst.ndim == 2
    M, N = src.shape
    assert dst.shape == (N, M), f"Expected dst shape ({N}, {M}), got {dst.shape}"
    assert src.is_contiguous() and dst.is_contiguous() and src.dtype == dst.dtype and src.element_size() in (1, 2, 4)
    ops._gpu(src, dst)
    _lib.check(_lib.load().ngpt_transpose_copy(src.data_ptr(), M, N, dst.data_ptr(), src.element_size(),
                                               ops._stream(src)), "ngpt_transpose_copy")


def transpose_add(src: Tensor, dst: Tensor) -> None:
    """dst (N, M) += src (M, N).T -- reference triton_kernels.py:882-903 (tied embedding / lm_head gradients)."""
    assert src.ndim == 2 and dst.ndim == 2
    M, N = src.shape
    assert dst.shape == (N, M), f"Expected dst shape ({N}, {M}), got {dst.shape}"
    assert src.is_contiguous() and dst.is_contiguous() and src.dtype == dst.dtype
    assert src.dtype in (torch.bfloat16, torch.float32)
    ops._gpu(src, dst)
    _lib.check(_lib.load().ngpt_transpose_add(src.data_ptr(), M, N, dst.data_ptr(), src.element_size(),
                                              ops._stream(src)), "ngpt_transpose_add")


def reduce_mlp_activation_scales(partial_amax: Tensor, scales: Tensor, headroom: float = 1.25) -> None:
    """scales[l] = max(partial_amax[l].max(), 1e-12) * headroom / 448 -- reference triton_kernels.py:732-745."""
    num_layers, partial_count = partial_amax.shape
    assert scales.numel() >= num_layers
    assert partial_amax.dtype == torch.float32 and scales.dtype == torch.float32 and partial_amax.stride(1) == 1
    ops._gpu(partial_amax, scales)
    _lib.check(_lib.load().ngpt_reduce_scales(partial_amax.data_ptr(), partial_amax.stride(0), num_layers,
                                              partial_count, headroom, scales.data_ptr(), ops._stream(scales)),
               "ngpt_reduce_scales")


def quantize_transpose_mlp_down_weights(weights: Tensor, output_storage: Tensor, next_scales: Tensor,
                                        used_scales: Tensor, partial_amax: Tensor, headroom: float = 1.12) -> None:
    """Delayed-scale e4m3 copy of the MLP down projections, stored transposed, plus the next step's
    scales -- reference triton_kernels.py:748-779.  weights [L, H, D] bf16 (a strided view of the MLP
    bank is fine), output_storage [L, D, H] e4m3, next_scales / used_scales [L], partial_amax [L, tiles]."""
    num_layers, hidden_dim, model_dim = weights.shape
    assert output_storage.shape == (num_layers, model_dim, hidden_dim)
    num_tiles = -(-hidden_dim // 64) * -(-model_dim // 64)
    assert partial_amax.shape == (num_layers, num_tiles)
    assert weights.dtype == torch.bfloat16 and weights.stride(2) == 1 and weights.stride(1) == model_dim
    assert output_storage.is_contiguous() and partial_amax.is_contiguous()
    ops._gpu(weights, output_storage, next_scales, used_scales, partial_amax)
    _lib.check(_lib.load().ngpt_quant_transpose_down(weights.data_ptr(), num_layers, hidden_dim, model_dim,
                                                     weights.stride(0), next_scales.data_ptr(),
                                                     output_storage.data_ptr(), used_scales.data_ptr(),
                                                     partial_amax.data_ptr(), ops._stream(weights)),
               "ngpt_quant_transpose_down")
    reduce_mlp_activation_scales(partial_amax, next_scales, headroom=headroom)


def linear_relu_square(a, b, aux=None, a_f8=None, b_f8=None, dequant_scale_ptr=None,
                       activation_scale=None, partial_amax=None):
    """Reference launcher triton_kernels.py:576-665.

    Forward (aux is None): post = relu(a @ b.T)^2.  With b_f8: the contraction runs on the e4m3
    copies and is scaled by the 1-element device tensor `dequant_scale_ptr`; with
    `activation_scale` an e4m3 copy of post and per-workgroup amax partials are produced too.
    Backward (aux = post): dpre = 2 * (a @ b.T) * sqrt(post), all bf16."""
    M, K = a.shape
    N, K2 = b.shape
    assert K == K2
    use_fp8 = b_f8 is not None
    emit_fp8 = activation_scale is not None
    if aux is None:
        if use_fp8:
            assert dequant_scale_ptr is not None and a_f8 is not None
            if emit_fp8:
                assert partial_amax is not None
                return ops.fc_relu2_fwd_emit(a_f8, b_f8, dequant_scale_ptr, activation_scale, partial_amax)
            return ops.fc_relu2_fwd(a_f8, b_f8, dequant_scale_ptr)
        return ops.linear_relu2_bf16(a.contiguous(), b.contiguous())
    return ops.fc_relu2_bwd_dpre(a.contiguous(), b.contiguous(), aux.contiguous())


class FusedLinearReLUSquareFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, W1, W2, W1_f8=None, dequant_scale=None, x_f8=None, W2_f8=None, W2_scale=None,
                activation_scale=None, partial_amax=None):
        # saved for the backward: post = relu(x @ W1.T)^2 (the pre-activation never reaches memory)
        x_flat = x.view((-1, x.shape[-1]))
        # There is no PyTorch fallback behind these kernels; say what they need before anything is launched.  The
        # products of the backward contract over the tokens, so the token count is bound by the contraction step too.
        tokens, model_dim, hidden_dim = x_flat.shape[0], x_flat.shape[1], W1.shape[0]
        assert model_dim % 64 == 0 and hidden_dim % 64 == 0, (
            f"FusedLinearReLUSquareFunction: model_dim={model_dim} and hidden_dim={hidden_dim} must be multiples of 64")
        assert tokens % 8 == 0 and (tokens % 64 == 0 or not (x.requires_grad or W1.requires_grad or W2.requires_grad)), (
            f"FusedLinearReLUSquareFunction: {tokens} tokens; the forward needs a multiple of 8, the backward (which "
            "contracts over the tokens) a multiple of 64")
        post_f8 = None
        if W1_f8 is not None:
            assert x_f8 is not None and dequant_scale is not None
            x_f8 = x_f8.view((-1, x_f8.shape[-1]))
            if W2_f8 is not None:
                assert W2_scale is not None and activation_scale is not None
                assert partial_amax is not None
                post, post_f8 = linear_relu_square(x_flat, W1, a_f8=x_f8, b_f8=W1_f8,
                                                   dequant_scale_ptr=dequant_scale,
                                                   activation_scale=activation_scale,
                                                   partial_amax=partial_amax)
            else:
                post = linear_relu_square(x_flat, W1, a_f8=x_f8, b_f8=W1_f8, dequant_scale_ptr=dequant_scale)
        else:
            post = linear_relu_square(x_flat, W1)
        if W2_f8 is not None:
            # W2_f8 is the (H, D) view of a (D, H) row-major e4m3 buffer: the contraction index H
            # is contiguous on both sides, which is what the TN GEMM reads.  The two scales are
            # 1-element device tensors; the GEMM's epilogue multiplies by their product, no host sync.
            w2_dh = W2_f8.T
            assert w2_dh.is_contiguous()
            x3 = ops.gemm_fp8_scaled(post_f8, w2_dh, activation_scale.reshape(-1).to(torch.float32),
                                     W2_scale.reshape(-1).to(torch.float32))
        else:
            x3 = ops.gemm_bf16(post, W2, False, True)          # post @ W2, W2 [H, D] read with the contraction as its rows
        # the backward is all bf16 and needs post and W2 themselves, not the e4m3 copies
        ctx.save_for_backward(x, W1, W2, post)
        return x3.view(x.shape)

    @staticmethod
    def backward(ctx, grad_output):
        x, W1, W2, post = ctx.saved_tensors
        x_flat = x.view((-1, x.shape[-1]))
        g = grad_output.reshape((-1, grad_output.shape[-1]))
        g = g.contiguous()
        dW2 = ops.gemm_bf16(post, g, True, True)               # post.T @ dY: contraction over the tokens
        dpre = linear_relu_square(g, W2, aux=post)
        dW1 = ops.gemm_bf16(dpre, x_flat, True, True)          # dpre.T @ x
        dx = ops.gemm_bf16(dpre, W1, False, True)              # dpre @ W1
        return dx.view(x.shape), dW1, dW2, None, None, None, None, None, None, None


ReLUSqrdMLP = FusedLinearReLUSquareFunction.apply


class FusedSoftcappedCrossEntropy(torch.autograd.Function):
    """lm_head GEMM + 23*sigmoid((l+5)/7.5) softcap + cross-entropy, forward and backward, with the
    [M, V] logits never written to HBM.  `lm_head_weight` is (in, out) as at the reference's HEAD
    (`w_layout="in_out"`); pass `w_layout="out_in"` as a keyword-free 14th argument for the
    (out, in) convention of `nanogpt::mm`."""

    @staticmethod
    def forward(ctx, x, targets, mtp_weights, prefix_targets, prefix_weight, lm_head_weight,
                x_s, w_s, grad_s, grad_scale, A=23.0, B=5.0, C=7.5, w_layout="in_out"):
        assert w_layout in ("in_out", "out_in")
        w_in_out = w_layout == "in_out"
        n_rows = x.shape[0]
        dev = x.device
        if mtp_weights is None:
            mtp_weights = torch.ones(1, device=dev, dtype=torch.float32)   # a fill kernel, not a host copy: legal under graph capture
        mtp_weights = mtp_weights.to(torch.float32).contiguous()
        targets = targets.contiguous()
        if prefix_targets is None:
            prefix_targets = torch.full((n_rows,), -1, dtype=torch.int64, device=dev)
        prefix_targets = prefix_targets.contiguous()
        if prefix_weight is None:
            prefix_weight = torch.zeros(1, dtype=torch.float32, device=dev)
        prefix_weight = prefix_weight.reshape(1).to(torch.float32).contiguous()

        if CE_BACKWARD == "codes" and n_rows % 128 == 0:
            losses, lse, saved_sigma, x_f8, w_f8, codes = torch.ops.nanogpt.lmhead_ce_fwd_codes(
                x.contiguous(), lm_head_weight.contiguous(), targets, mtp_weights, prefix_targets, prefix_weight,
                x_s, w_s, A, B, C, w_in_out)
        else:
            losses, lse, saved_sigma, x_f8, w_f8 = torch.ops.nanogpt.lmhead_ce_fwd(
                x.contiguous(), lm_head_weight.contiguous(), targets, mtp_weights, prefix_targets, prefix_weight,
                x_s, w_s, A, B, C, w_in_out)
            codes = None
        ctx.save_for_backward(targets, mtp_weights, prefix_targets, prefix_weight, lse, saved_sigma, x_f8, w_f8, codes)
        ctx.params = (A, B, C, x_s, w_s, grad_s, grad_scale, w_in_out)
        return losses

    @staticmethod
    def backward(ctx, grad_output):
        # grad_output is ignored: grad_scale is folded into the gradient, as in the reference
        # (triton_kernels.py:1117, 1262).
        targets, mtp_weights, prefix_targets, prefix_weight, lse, saved_sigma, x_f8, w_f8, codes = ctx.saved_tensors
        A, B, C, x_s, w_s, grad_s, grad_scale, w_in_out = ctx.params
        if codes is not None:
            grad_x, grad_w = torch.ops.nanogpt.lmhead_ce_bwd_codes(
                x_f8, w_f8, targets, mtp_weights, prefix_targets, prefix_weight, lse, saved_sigma, codes,
                x_s, w_s, grad_s, grad_scale, A, B, C, w_in_out)
        else:
            grad_x, grad_w = torch.ops.nanogpt.lmhead_ce_bwd(
                x_f8, w_f8, targets, mtp_weights, prefix_targets, prefix_weight, lse, saved_sigma,
                x_s, w_s, grad_s, grad_scale, A, B, C, w_in_out)
        return grad_x, None, None, None, None, grad_w, None, None, None, None, None, None, None, None
