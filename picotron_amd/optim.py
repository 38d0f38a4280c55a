"""AdamW for the model's parameters, one fused HIP pass per parameter tensor.

The reference builds ``torch.optim.AdamW(model.parameters(), lr)`` (``train.py:204-209``; its ``fused`` switch is
dead code) on the bf16 model and so keeps the optimizer state in the parameter dtype.  Two layouts are offered:

``master_weights=True`` (default)  fp32 state: a master copy of every parameter plus both moments in three flat
    buffers; ``step()`` reads each bf16 gradient once and rewrites the bf16 parameter from the updated master weight
    in the same kernel (``pico_adamw``) -- no cast passes.  28 bytes of HBM traffic per parameter.
``master_weights=False``  the bf16 parameter is updated in place (``pico_adamw_lp``); fp32 arithmetic inside the
    kernel, one rounding per stored value.  ``state_dtype=torch.float32`` keeps both moments in fp32 ("bf16 parameters
    with fp32 AdamW state", 22 bytes per parameter); ``state_dtype=None`` keeps them in the parameter dtype, which is
    the reference's own layout (14 bytes per parameter)."""
from __future__ import annotations

from typing import Iterable

import torch

from . import ops


class FusedAdamW:
    def __init__(self, params: Iterable[torch.nn.Parameter], lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1e-2, overlap_with_backward: bool = False, master_weights: bool = True, state_dtype=None):
        self.params = [p for p in params if p.requires_grad]
        if not self.params:
            raise ValueError("FusedAdamW: no parameters")
        for p in self.params:
            if not p.is_cuda or p.dtype not in (torch.bfloat16, torch.float32) or not p.is_contiguous():
                raise RuntimeError("FusedAdamW: parameters must be contiguous bf16 / fp32 tensors on the GPU")
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.step_count = 0
        self._plans = {}
        dev = self.params[0].device
        # every tensor starts on a multiple of 8 elements so that all kernel accesses are 16-byte aligned
        self.offsets, total = [], 0
        for p in self.params:
            self.offsets.append(total)
            total += (p.numel() + 7) // 8 * 8
        self.master_weights = master_weights
        if master_weights:
            if state_dtype not in (None, torch.float32):
                raise RuntimeError("FusedAdamW: master weights come with fp32 moments")
            state_dtype = torch.float32
            self.master = torch.zeros(total, dtype=torch.float32, device=dev)
            for p, off in zip(self.params, self.offsets):
                self.master[off:off + p.numel()].copy_(p.detach().reshape(-1))
        else:
            if any(p.dtype != self.params[0].dtype for p in self.params):
                raise RuntimeError("FusedAdamW(master_weights=False): all parameters must share one dtype")
            if state_dtype is None:
                state_dtype = self.params[0].dtype
            if state_dtype not in (torch.float32, self.params[0].dtype):
                raise RuntimeError("FusedAdamW: state_dtype must be torch.float32 or the parameter dtype")
            self.master = None
        self.exp_avg = torch.zeros(total, dtype=state_dtype, device=dev)
        self.exp_avg_sq = torch.zeros(total, dtype=state_dtype, device=dev)
        # Optional: update each parameter on a second stream as soon as the backward pass has produced its gradient.
        # The update is a pure HBM stream and the rest of the backward is GEMM-bound, so the two can overlap (measured:
        # +1 % tokens/s on the SmolLM-1.7B-shaped step, so it is off by default); a weight is read only by its own
        # layer's backward node, which has finished when the hook fires.  zero_grad() opens a
        # step (it fixes the step number for the bias corrections), step() only joins the streams.
        self.overlap = overlap_with_backward
        self._open = False
        if self.overlap:
            self.side = torch.cuda.Stream(device=dev)
            for i, p in enumerate(self.params):
                p.register_post_accumulate_grad_hook(lambda p_, i_=i: self._on_grad(i_, p_))

    def _update(self, p, off, g, grad_scale):
        n = p.numel()
        m, v = self.exp_avg[off:off + n], self.exp_avg_sq[off:off + n]
        hyper = (self.step_count, self.lr, self.betas[0], self.betas[1], self.eps, self.weight_decay, grad_scale)
        if self.master_weights:
            ops.adamw_(p if p.dtype == torch.bfloat16 else None, self.master[off:off + n], g, m, v, *hyper)
            if p.dtype == torch.float32:
                p.copy_(self.master[off:off + n].view_as(p))
        elif p.dtype == torch.bfloat16:
            ops.adamw_lp_(p.view(-1), g, m, v, *hyper)
        else:
            ops.adamw_(None, p.view(-1), g, m, v, *hyper)

    @torch.no_grad()
    def _on_grad(self, i, p):
        if not self._open or p.grad is None:
            return
        cur = torch.cuda.current_stream()
        self.side.wait_stream(cur)
        off, g = self.offsets[i], p.grad
        with torch.cuda.stream(self.side):
            self._update(p, off, g, 1.0)
        g.record_stream(self.side)   # its memory must not be handed out again before the side stream has read it
        p.grad = None

    def zero_grad(self, set_to_none: bool = True):
        if self.overlap:
            self.step_count += 1
            self._open = True
        for p in self.params:
            if set_to_none:
                p.grad = None
            elif p.grad is not None:
                p.grad.zero_()

    @torch.no_grad()
    def step(self, grad_scale: float = 1.0):
        if self.overlap:
            if grad_scale != 1.0:
                raise RuntimeError("FusedAdamW: grad_scale is not available with overlap_with_backward")
            torch.cuda.current_stream().wait_stream(self.side)
            self._open = False
            return
        self.step_count += 1
        live = tuple(i for i, p in enumerate(self.params) if p.grad is not None)
        if not live:
            return
        hyper = (self.step_count, self.lr, self.betas[0], self.betas[1], self.eps, self.weight_decay, grad_scale)
        # one launch table per gradient dtype; the tables (everything but the gradients' addresses) are built once per
        # set of live parameters and reused, so the host side of a step stays far below the kernel's own time
        by_dtype = {}
        for i in live:
            by_dtype.setdefault(self.params[i].grad.dtype, []).append(i)
        for gdt, idx in by_dtype.items():
            key = (gdt, tuple(idx))
            plan = self._plans.get(key)
            if plan is None or any(self.params[i].data_ptr() != ptr for i, ptr in zip(idx, plan.param_ptrs)):
                plan = self._plans[key] = self._make_plan(idx)
            plan.step([self.params[i].grad for i in idx], *hyper)
            if self.master_weights:
                for i in idx:
                    p = self.params[i]
                    if p.dtype == torch.float32:
                        off = self.offsets[i]
                        p.copy_(self.master[off:off + p.numel()].view_as(p))

    def _make_plan(self, idx):
        ps = [self.params[i] for i in idx]
        ms = [self.exp_avg[self.offsets[i]:self.offsets[i] + self.params[i].numel()] for i in idx]
        vs = [self.exp_avg_sq[self.offsets[i]:self.offsets[i] + self.params[i].numel()] for i in idx]
        if self.master_weights:
            ws = [self.master[self.offsets[i]:self.offsets[i] + self.params[i].numel()] for i in idx]
            plan = ops.AdamWMultiPlan(ws, ms, vs, [p.detach().view(-1) if p.dtype == torch.bfloat16 else None for p in ps])
        else:
            plan = ops.AdamWMultiPlan([p.detach().view(-1) for p in ps], ms, vs)
        plan.param_ptrs = [p.data_ptr() for p in ps]   # a parameter that was moved or cast since invalidates the plan
        return plan
