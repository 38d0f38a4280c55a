"""CPU restatement of the optimizer step of ``train.py:204-209,240``: ``torch.optim.AdamW`` with torch's defaults
(betas (0.9, 0.999), eps 1e-8, weight decay 0.01, no amsgrad), written out as plain tensor arithmetic in the order
torch applies it.  Test infrastructure only.  The reference keeps the AdamW state in the parameter dtype; the
build under test keeps fp32 master weights and moments for bf16 parameters, which is what ``master_step`` states.

``lp_step`` states the reference's own layout -- parameter and moments in the parameter dtype -- with fp32 arithmetic
and one rounding per state, which is what torch's ``fused=True`` AdamW computes (its default for-each path rounds
after every operation instead).

Pinned by ``tests/test_oracle_layers.py`` against ``torch.optim.AdamW`` itself (a library routine) over several steps:
``adamw_step`` against the default implementation on fp32 parameters, ``lp_step`` against ``fused=True`` on bf16
parameters.
"""
from __future__ import annotations

import math

import torch


def adamw_step(p: torch.Tensor, g: torch.Tensor, m: torch.Tensor, v: torch.Tensor, step: int, lr: float,
               beta1: float = 0.9, beta2: float = 0.999, eps: float = 1e-8, weight_decay: float = 0.01):
    """One AdamW update of (p, m, v) by gradient g at 1-based `step`; returns the new (p, m, v), inputs untouched."""
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    p = p * (1.0 - lr * weight_decay)
    m = m + (g - m) * (1.0 - beta1)
    v = v * beta2 + g * g * (1.0 - beta2)
    denom = v.sqrt() / math.sqrt(bc2) + eps
    p = p - (lr / bc1) * (m / denom)
    return p, m, v


def master_step(master: torch.Tensor, grad_lp: torch.Tensor, m: torch.Tensor, v: torch.Tensor, step: int, lr: float,
                lp_dtype=torch.bfloat16, **kw):
    """AdamW on fp32 master weights from a low-precision gradient; also returns the low-precision copy of the
    new parameter (what the model computes with)."""
    p, m, v = adamw_step(master.float(), grad_lp.float(), m.float(), v.float(), step, lr, **kw)
    return p, m, v, p.to(lp_dtype)


def lp_step(p: torch.Tensor, g: torch.Tensor, m: torch.Tensor, v: torch.Tensor, step: int, lr: float, **kw):
    """AdamW on a low-precision parameter updated in place: fp32 arithmetic, then the parameter is rounded once to
    p.dtype and the moments once to their own dtype (p.dtype as the reference holds them, or fp32)."""
    p2, m2, v2 = adamw_step(p.float(), g.float(), m.float(), v.float(), step, lr, **kw)
    return p2.to(p.dtype), m2.to(m.dtype), v2.to(v.dtype)
