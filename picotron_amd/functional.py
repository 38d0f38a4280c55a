"""autograd.Functions that tie the HIP forward and backward kernels together for the model code."""
from __future__ import annotations

import torch

from . import ops


class RMSNormFunc(torch.autograd.Function):
    """y = rmsnorm(x) * w.  cast_then_scale selects LlamaRMSNorm's rounding order (``model.py:81-86``)."""

    @staticmethod
    def forward(ctx, x, weight, eps, cast_then_scale):
        y, rstd, _ = ops.rmsnorm_fwd(x, weight, eps, cast_then_scale)
        ctx.save_for_backward(x, weight, rstd)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, rstd = ctx.saved_tensors
        dx, dw = ops.rmsnorm_bwd(dy, x, weight, rstd)
        return dx, dw.to(weight.dtype), None, None


class RMSNormResidualFunc(torch.autograd.Function):
    """h = x + residual; returns (rmsnorm(h) * w, h) -- the prenorm form of flash-attn's layer_norm_fn."""

    @staticmethod
    def forward(ctx, x, residual, weight, eps):
        y, rstd, h = ops.rmsnorm_fwd(x, weight, eps, False, residual=residual, want_residual_out=True)
        ctx.save_for_backward(h, weight, rstd)
        return y, h

    @staticmethod
    def backward(ctx, dy, dh):
        h, weight, rstd = ctx.saved_tensors
        dx, dw = ops.rmsnorm_bwd(dy, h, weight, rstd)
        if dh is not None:
            dx = dx + dh
        return dx, dx, dw.to(weight.dtype), None


class RotaryFunc(torch.autograd.Function):
    """Non-interleaved RoPE on [B,H,S,D]; the backward is the rotation by -theta."""

    @staticmethod
    def forward(ctx, x, cos, sin, pos_offset):
        ctx.save_for_backward(cos, sin)
        ctx.pos_offset = pos_offset
        return ops.rope(x, cos, sin, pos_offset, inverse=False)

    @staticmethod
    def backward(ctx, dy):
        cos, sin = ctx.saved_tensors
        return ops.rope(dy, cos, sin, ctx.pos_offset, inverse=True), None, None, None


class SwiGLUFunc(torch.autograd.Function):
    """silu(gate) * up (``model.py:186``)."""

    @staticmethod
    def forward(ctx, gate, up):
        ctx.save_for_backward(gate, up)
        return ops.swiglu_fwd(gate, up)

    @staticmethod
    def backward(ctx, dy):
        gate, up = ctx.saved_tensors
        return ops.swiglu_bwd(dy, gate, up)


class FlashAttnFunc(torch.autograd.Function):
    """Single-chunk causal / dense attention on [B,H,S,D] views; K/V may carry fewer (GQA) heads."""

    @staticmethod
    def forward(ctx, q, k, v, sm_scale, causal):
        out, lse = ops.attn_fwd(q, k, v, sm_scale, causal, 0, out_dtype=q.dtype, bshd_out=True)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.sm_scale, ctx.causal = sm_scale, causal
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        # delta = sum_d dout * out is computed inside the call; gradients come back in the dtype and memory layout of
        # their inputs: no accumulation buffer, no cast pass
        dq, dk, dv = ops.attn_bwd(dout, q, k, v, lse, None, ctx.sm_scale, ctx.causal, 0, dq_dtype=q.dtype, dq_like=q,
                                  dkv_dtype=k.dtype, out=out)
        return dq, dk, dv, None, None


class CrossEntropyFunc(torch.autograd.Function):
    """Mean cross-entropy of [rows, vocab] logits against int64 targets (``train.py:46-49``), fp32 loss.
    The backward writes dlogits in the dtype of the logits in one pass; the upstream gradient and the 1 / count
    factor reach the kernel through a device scalar, so nothing synchronises with the host."""

    @staticmethod
    def forward(ctx, logits, targets, ignore_index=-100):
        loss_rows, lse = ops.cross_entropy_fwd(logits, targets, ignore_index)
        count = (targets != ignore_index).sum().clamp(min=1).to(torch.float32)
        ctx.save_for_backward(logits, targets, lse, count)
        ctx.ignore_index = ignore_index
        return loss_rows.sum() / count

    @staticmethod
    def backward(ctx, grad_out):
        logits, targets, lse, count = ctx.saved_tensors
        scale = (grad_out.to(torch.float32) / count).reshape(1)
        return ops.cross_entropy_bwd(logits, targets, lse, scale, ctx.ignore_index), None, None


def cross_entropy(logits, targets, ignore_index: int = -100):
    """Drop-in for ``F.cross_entropy(logits, targets, reduction='mean')`` on 2-D logits."""
    return CrossEntropyFunc.apply(logits, targets, ignore_index)
