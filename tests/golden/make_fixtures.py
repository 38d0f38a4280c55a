"""Writes tests/golden/vectors.npz: inputs and expected outputs for every kernel of the path, computed in fp64 by
library routines of torch alone (softmax / logsumexp / autograd, F.rms_norm, F.silu, F.cross_entropy,
torch.optim.AdamW) -- neither the oracle in oracle/ nor the reference is imported.  The inputs are rounded to bf16
first, so the same numbers can be fed to the bf16 kernels without a second rounding; everything is stored as fp32.

    python tests/golden/make_fixtures.py

The committed file was made with this script; rerunning it reproduces it bit for bit on the same torch build."""
import math
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_values(*shape, gen, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(torch.bfloat16).to(torch.float64)


def attention_case(gen, B, Hq, Hkv, Sq, Sk, D, causal, q_offset):
    """softmax(q k^T * scale + mask) v with the causal diagonal shifted by q_offset (query i sits at position
    q_offset + i: what a context-parallel rank sees), GQA by repeating kv heads, gradients by autograd."""
    scale = 1.0 / math.sqrt(D)
    q = bf16_values(B, Hq, Sq, D, gen=gen, scale=scale).requires_grad_()
    k = bf16_values(B, Hkv, Sk, D, gen=gen).requires_grad_()
    v = bf16_values(B, Hkv, Sk, D, gen=gen).requires_grad_()
    do = bf16_values(B, Hq, Sq, D, gen=gen)
    rep = Hq // Hkv
    s = (q @ k.repeat_interleave(rep, 1).transpose(-1, -2)) * scale
    if causal:
        qi = torch.arange(Sq)[:, None] + q_offset
        kj = torch.arange(Sk)[None, :]
        s = s.masked_fill(kj > qi, float("-inf"))
    out = torch.softmax(s, -1) @ v.repeat_interleave(rep, 1)
    lse = torch.logsumexp(s, -1)
    dq, dk, dv = torch.autograd.grad(out, (q, k, v), do)
    return dict(q=q.detach(), k=k.detach(), v=v.detach(), do=do, out=out.detach(), lse=lse.detach(), dq=dq, dk=dk, dv=dv,
                meta=torch.tensor([B, Hq, Hkv, Sq, Sk, D, int(causal), q_offset], dtype=torch.float64))


def main():
    g = torch.Generator().manual_seed(20240611)
    vec = {}
    for name, args in (("attn_causal_offset", (1, 4, 2, 40, 72, 64, True, 32)), ("attn_dense_ragged", (1, 2, 2, 33, 50, 128, False, 0)),
                       ("attn_causal_square", (1, 2, 1, 64, 64, 64, True, 0))):
        for key, t in attention_case(g, *args).items():
            vec[f"{name}.{key}"] = t
    # RMSNorm (fp32 maths, one rounding: the TritonRMSNorm flavour) and its gradients
    x = bf16_values(5, 576, gen=g).requires_grad_()
    w = (1 + 0.1 * torch.randn(576, generator=g)).to(torch.bfloat16).to(torch.float64).requires_grad_()
    dy = bf16_values(5, 576, gen=g)
    y = F.rms_norm(x, (576,), w, 1e-5)
    dx, dw = torch.autograd.grad(y, (x, w), dy)
    vec.update({"rmsnorm.x": x.detach(), "rmsnorm.w": w.detach(), "rmsnorm.dy": dy, "rmsnorm.y": y.detach(), "rmsnorm.dx": dx, "rmsnorm.dw": dw})
    # RoPE, non-interleaved halves, rows 3.. of the tables (a chunk that starts at position 3), base 10000
    D, S, off = 64, 7, 3
    xr = bf16_values(1, 2, S, D, gen=g)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    ang = (torch.arange(S, dtype=torch.float64) + off)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang), torch.sin(ang)
    x1, x2 = xr[..., : D // 2], xr[..., D // 2:]
    vec.update({"rope.x": xr, "rope.offset": torch.tensor([off], dtype=torch.float64),
                "rope.y": torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], -1)})
    # SwiGLU
    gate, up = bf16_values(6, 96, gen=g).requires_grad_(), bf16_values(6, 96, gen=g).requires_grad_()
    dyo = bf16_values(6, 96, gen=g)
    yo = F.silu(gate) * up
    dg, du = torch.autograd.grad(yo, (gate, up), dyo)
    vec.update({"swiglu.gate": gate.detach(), "swiglu.up": up.detach(), "swiglu.dy": dyo, "swiglu.y": yo.detach(), "swiglu.dgate": dg, "swiglu.dup": du})
    # cross-entropy, mean over the rows that count
    logits = bf16_values(9, 200, gen=g, scale=3.0).requires_grad_()
    tgt = torch.randint(0, 200, (9,), generator=g)
    tgt[4] = -100
    loss = F.cross_entropy(logits, tgt)
    (dl,) = torch.autograd.grad(loss, logits)
    vec.update({"ce.logits": logits.detach(), "ce.targets": tgt.to(torch.float64), "ce.loss": loss.detach().reshape(1), "ce.dlogits": dl,
                "ce.lse": torch.logsumexp(logits.detach(), -1)})
    # three AdamW steps (torch defaults but lr, no amsgrad)
    p = torch.nn.Parameter(bf16_values(300, gen=g))
    opt = torch.optim.AdamW([p], lr=1e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    vec["adamw.p0"] = p.detach().clone()
    for step in range(3):
        p.grad = bf16_values(300, gen=g, scale=0.1 * (step + 1))
        vec[f"adamw.g{step}"] = p.grad.clone()
        opt.step()
        vec[f"adamw.p{step + 1}"] = p.detach().clone()
    vec["adamw.m3"], vec["adamw.v3"] = opt.state[p]["exp_avg"].clone(), opt.state[p]["exp_avg_sq"].clone()
    # stored as fp32: exact for the bf16-valued inputs, and 2^-24 relative on the expected values, far below any tolerance
    np.savez_compressed(os.path.join(HERE, "vectors.npz"), **{k: v.to(torch.float32).numpy() for k, v in vec.items()})
    print("wrote", len(vec), "arrays")


if __name__ == "__main__":
    main()
