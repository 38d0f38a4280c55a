"""Oracle (test infrastructure): RoPE, RMSNorm and SwiGLU of ``picotron/model.py`` on the CPU.

* ``get_cos_sin``            <- ``model.py:21-31``
* ``apply_rotary_pos_emb``   <- ``model.py:12-19`` (same maths as the flash branch ``model.py:136-137``:
                                non-interleaved rotation with the first D/2 table columns)
* ``rmsnorm``                <- ``LlamaRMSNorm.forward`` ``model.py:81-86`` (cast, then scale) and the
                                single-rounding fp32 variant used by ``TritonRMSNorm`` ``model.py:51-65``
* ``swiglu``                 <- ``F.silu(gate) * up`` ``model.py:186``

Backward closed forms are written out so the HIP backward kernels can be compared with
something that is not autograd of the same forward; tests check the two agree.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- RoPE
def get_cos_sin(seq_length: int, head_dim: int, base: float = 500000.0, dtype=torch.bfloat16,
                device="cpu"):
    """cos/sin tables [S, D] with the two halves duplicated (``model.py:21-31``).

    theta is computed on the CPU from an int64 arange (:24); the angle pos*theta is formed in
    fp32 (:28-31); the tables are rounded to ``dtype`` (bf16 unless DTYPE says otherwise, :25).
    """
    assert head_dim % 2 == 0
    exponent = torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim
    theta = 1.0 / (base ** exponent)
    pos = torch.arange(seq_length).unsqueeze(1).float().to(device)
    angle = pos * theta.to(device).float()
    return torch.cos(angle).to(dtype).repeat(1, 2), torch.sin(angle).to(dtype).repeat(1, 2)


def apply_rotary_pos_emb(x, cos, sin):
    """x*cos + rotate_half(x)*sin with halves split at D/2 (``model.py:12-19``); x [B,H,S,D]."""
    half = x.size(-1) // 2
    lo, hi = x[..., :half], x[..., half:]
    return x * cos + torch.cat((-hi, lo), dim=-1) * sin


def apply_rotary_pos_emb_backward(dy, cos, sin):
    """Adjoint of the rotation = rotation by -theta: dx = dy*cos - rotate_half(dy*sin)... written per half."""
    half = dy.size(-1) // 2
    c, s = cos[..., :half], sin[..., :half]
    d_lo, d_hi = dy[..., :half], dy[..., half:]
    return torch.cat((d_lo * c + d_hi * s, d_hi * c - d_lo * s), dim=-1)


# --------------------------------------------------------------------------- RMSNorm
def rmsnorm(x, weight, eps: float, cast_then_scale: bool = True):
    """y = w * (x * rsqrt(mean(x^2) + eps)).

    cast_then_scale=True follows ``LlamaRMSNorm`` (:81-86): the normalised value is rounded to
    x.dtype and only then multiplied by the weight.  False is the fused fp32 form with one
    rounding at the end, as flash-attn's ``layer_norm_fn(is_rms_norm=True)`` computes it.
    """
    xf = x.to(torch.float32) if x.dtype != torch.float64 else x
    var = xf.pow(2).mean(-1, keepdim=True)
    xhat = xf * torch.rsqrt(var + eps)
    if cast_then_scale:
        return weight * xhat.to(x.dtype)
    return (xhat * weight.to(xhat.dtype)).to(x.dtype)


def rmsnorm_backward(dy, x, weight, eps: float):
    """Closed form: g = dy*w; dx = r*(g - xhat*mean(g*xhat)); dw = sum_tokens dy*xhat (fp32 maths)."""
    acc = torch.float64 if x.dtype == torch.float64 else torch.float32
    xf, dyf, wf = x.to(acc), dy.to(acc), weight.to(acc)
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    xhat = xf * r
    g = dyf * wf
    dx = r * (g - xhat * (g * xhat).mean(-1, keepdim=True))
    dw = (dyf * xhat).reshape(-1, x.size(-1)).sum(0)
    return dx, dw


# --------------------------------------------------------------------------- SwiGLU
def swiglu(gate, up):
    return F.silu(gate) * up


def swiglu_backward(dy, gate, up):
    """dg = dy*u*sig(g)*(1 + g*(1 - sig(g))); du = dy*silu(g)."""
    acc = torch.float64 if gate.dtype == torch.float64 else torch.float32
    g, u, d = gate.to(acc), up.to(acc), dy.to(acc)
    sg = torch.sigmoid(g)
    return d * u * sg * (1 + g * (1 - sg)), d * g * sg


def cross_entropy(logits: torch.Tensor, targets: torch.Tensor, ignore_index: int = -100):
    """Mean cross-entropy as ``train.py:46-49`` computes it (``F.cross_entropy(..., reduction='mean')``), written out:
    loss_r = logsumexp(logits_r) - logits_r[target_r]; mean over the rows whose target is not ignore_index.
    Returns (loss, per-row logsumexp).  Pinned against ``F.cross_entropy`` in tests/test_oracle_layers.py."""
    x = logits.float()
    lse = torch.logsumexp(x, dim=-1)
    keep = targets != ignore_index
    picked = x.gather(1, targets.clamp(min=0).unsqueeze(1)).squeeze(1)
    rows = torch.where(keep, lse - picked, torch.zeros_like(lse))
    return rows.sum() / keep.sum().clamp(min=1), lse


def cross_entropy_backward(logits: torch.Tensor, targets: torch.Tensor, grad_out: float = 1.0, ignore_index: int = -100):
    """d loss / d logits = (softmax - onehot) * grad_out / count on kept rows, 0 on ignored ones."""
    x = logits.float()
    keep = targets != ignore_index
    p = torch.softmax(x, dim=-1)
    p[torch.arange(x.size(0)), targets.clamp(min=0)] -= 1.0
    return p * keep.unsqueeze(1) * (grad_out / keep.sum().clamp(min=1))
