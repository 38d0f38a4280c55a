"""autograd.Functions that tie the HIP forward and backward kernels together for the model code."""
from __future__ import annotations

import os

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
        dx, dw = ops.rmsnorm_bwd(dy, x, weight, rstd, dw_dtype=weight.dtype)
        return dx, dw, None, None


class RMSNormResidualFunc(torch.autograd.Function):
    """h = x + residual; returns (rmsnorm(h) * w, h) -- the prenorm form of flash-attn's layer_norm_fn."""

    @staticmethod
    def forward(ctx, x, residual, weight, eps):
        y, rstd, h = ops.rmsnorm_fwd(x, weight, eps, False, residual=residual, want_residual_out=True)
        ctx.save_for_backward(h, weight, rstd)
        ctx.set_materialize_grads(False)    # the last norm's h has no consumer: no zero tensor is made for it
        return y, h

    @staticmethod
    def backward(ctx, dy, dh):
        h, weight, rstd = ctx.saved_tensors
        if dy is None:
            # only the residual stream carried a gradient: it passes through the add unchanged
            return dh, dh, None, None
        # dh, the gradient that reached h without passing the norm, is added inside the kernel
        dx, dw = ops.rmsnorm_bwd(dy, h, weight, rstd, dresidual=dh, dw_dtype=weight.dtype)
        return dx, dx, dw, None


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
                                  dkv_dtype=k.dtype, out=out, dkv_like=k if k.stride() == v.stride() else None)
        return dq, dk, dv, None, None


class CrossEntropyFunc(torch.autograd.Function):
    """Mean cross-entropy of [rows, vocab] logits against int64 targets (``train.py:46-49``), fp32 loss.
    The backward writes dlogits in the dtype of the logits in one pass; the upstream gradient and the 1 / count
    factor reach the kernel through a device scalar, so nothing synchronises with the host."""

    @staticmethod
    def forward(ctx, logits, targets, ignore_index=-100):
        if os.getenv("PICO_CHECK_TARGETS", "0") == "1":
            # F.cross_entropy asserts on the device for a target outside [0, vocab) (train.py:46-49); the kernels skip such
            # a row instead (they may not index with it), which would hide a tokenizer / vocabulary mismatch.  This
            # opt-in check costs a host synchronisation.
            bad = (targets != ignore_index) & ((targets < 0) | (targets >= logits.size(-1)))
            if bool(bad.any()):
                raise RuntimeError(f"cross_entropy: {int(bad.sum())} targets lie outside [0, {logits.size(-1)}) and are not "
                                   f"ignore_index={ignore_index}")
        loss_rows, lse = ops.cross_entropy_fwd(logits, targets, ignore_index)
        # rows that count: not ignored and a valid index (the kernels skip a target outside [0, vocab) as well)
        count = ((targets != ignore_index) & (targets >= 0) & (targets < logits.size(-1))).sum().clamp(min=1).to(torch.float32)
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


# ---------------------------------------------------------------------------------------------------------------
# Fused projections.  The reference's q_proj / k_proj / v_proj (and gate_proj / up_proj) read the same activation;
# their weights are kept as separate Parameters but laid out back to back in one buffer, so one GEMM produces all
# outputs, one GEMM all weight gradients and one GEMM the (already summed) input gradient.  The pieces below hand
# strided views of those fused buffers to the kernels, which take row pitches / element strides as they are, and
# write the pieces of the fused gradient in place: no concatenation, split or layout copy on either pass.

class FusedLinearFunc(torch.autograd.Function):
    """y = x @ w_fused^T where w_fused is the buffer that the Parameters `parts` (rows of it, in order) alias."""

    @staticmethod
    def forward(ctx, x, w_fused, *parts):
        ctx.save_for_backward(x, w_fused)
        ctx.sizes = [p.size(0) for p in parts]
        return torch.nn.functional.linear(x, w_fused)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.size(-1))
        dx = (dy2 @ w).view(x.shape)
        dw = dy2.t() @ x.reshape(-1, x.size(-1))
        return (dx, None) + tuple(dw.split(ctx.sizes, dim=0))


def _fused_rope() -> bool:
    """RoPE inside the attention kernels (default); PICO_FUSED_ROPE=0 keeps it a launch of its own over q and k."""
    return os.getenv("PICO_FUSED_ROPE", "1") != "0"


class QKVAttentionFunc(torch.autograd.Function):
    """RoPE on the q and k parts of a fused [B,S,(Hq+2Hkv)*D] projection, then causal / dense attention (one chunk);
    returns [B,S,Hq*D].

    Default: q is rotated inside the attention forward (every query once, in the prologue of the workgroup that owns
    it; the kernel leaves the rotated q behind for the backward), only k -- which many workgroups read -- is rotated by a
    launch of its own, and the backward un-rotates dq and dk in the epilogues of its kernels: one small RoPE launch per
    layer in the forward, none in the backward.  The backward writes dq, dk, dv straight into the matching columns of
    one [B,S,(Hq+2Hkv)*D] buffer.  With PICO_FUSED_ROPE=0 q and k are rotated by one launch (they lie side by side in
    the projection) and dq / dk are un-rotated in place by another."""

    @staticmethod
    def forward(ctx, qkv, cos, sin, n_heads, n_kv_heads, head_dim, causal):
        B, S, _ = qkv.shape
        nq, nkv = n_heads * head_dim, n_kv_heads * head_dim
        v = qkv[..., nq + nkv:].view(B, S, n_kv_heads, head_dim).transpose(1, 2)
        sm_scale = 1.0 / (head_dim ** 0.5)
        fused = _fused_rope()
        if fused:
            q_raw = qkv[..., :nq].view(B, S, n_heads, head_dim).transpose(1, 2)
            k_raw = qkv[..., nq:nq + nkv].view(B, S, n_kv_heads, head_dim).transpose(1, 2)
            k = ops.rope(k_raw, cos, sin, 0, out=ops.empty_bshd(B, n_kv_heads, S, head_dim, qkv.dtype, qkv.device))
            out, lse, q = ops.attn_fwd_rope(q_raw, k, v, cos, sin, sm_scale, causal, 0, 0, want_q_rot=True, out_dtype=qkv.dtype)
        else:
            # q and k lie side by side, so one launch rotates both as Hq+Hkv heads into a [B,S,Hq+Hkv,D] copy (the
            # projection output itself stays untouched: v is used as it lies)
            qk = qkv[..., :nq + nkv].view(B, S, n_heads + n_kv_heads, head_dim).transpose(1, 2)
            qk = ops.rope(qk, cos, sin, 0, out=ops.empty_bshd(B, n_heads + n_kv_heads, S, head_dim, qkv.dtype, qkv.device))
            q, k = qk[:, :n_heads], qk[:, n_heads:]
            out, lse = ops.attn_fwd(q, k, v, sm_scale, causal, 0, out_dtype=qkv.dtype, bshd_out=True)
        ctx.save_for_backward(q, k, v, out, lse, cos, sin)
        ctx.meta = (n_heads, n_kv_heads, head_dim, causal, sm_scale, fused)
        return out.transpose(1, 2).reshape(B, S, nq)

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, cos, sin = ctx.saved_tensors
        n_heads, n_kv_heads, head_dim, causal, sm_scale, fused = ctx.meta
        B, S = q.size(0), q.size(2)
        nq, nkv = n_heads * head_dim, n_kv_heads * head_dim
        dqkv = torch.empty(B, S, nq + 2 * nkv, dtype=q.dtype, device=q.device)
        dq = dqkv[..., :nq].view(B, S, n_heads, head_dim).transpose(1, 2)
        dk = dqkv[..., nq:nq + nkv].view(B, S, n_kv_heads, head_dim).transpose(1, 2)
        dv = dqkv[..., nq + nkv:].view(B, S, n_kv_heads, head_dim).transpose(1, 2)
        do = dout.view(B, S, n_heads, head_dim).transpose(1, 2)
        if fused:
            ops.attn_bwd_rope(do, q, k, v, out, lse, cos, sin, sm_scale, causal, dq, dk, dv)
        else:
            ops.attn_bwd(do, q, k, v, lse, None, sm_scale, causal, 0, dq, dk, dv, out=out)
            dqk = dqkv[..., :nq + nkv].view(B, S, n_heads + n_kv_heads, head_dim).transpose(1, 2)
            ops.rope(dqk, cos, sin, 0, inverse=True, out=dqk)
        return dqkv, None, None, None, None, None, None


class SwiGLUFusedFunc(torch.autograd.Function):
    """silu(gate) * up where gate and up are the two halves of one [..., 2I] projection output; the backward writes
    dgate and dup into the halves of one [..., 2I] buffer."""

    @staticmethod
    def forward(ctx, gate_up):
        ctx.save_for_backward(gate_up)
        half = gate_up.size(-1) // 2
        return ops.swiglu_fwd(gate_up[..., :half], gate_up[..., half:])

    @staticmethod
    def backward(ctx, dy):
        (gate_up,) = ctx.saved_tensors
        half = gate_up.size(-1) // 2
        d = torch.empty_like(gate_up)
        ops.swiglu_bwd(dy, gate_up[..., :half], gate_up[..., half:], out=(d[..., :half], d[..., half:]))
        return d
