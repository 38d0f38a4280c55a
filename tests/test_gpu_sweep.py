"""A seeded sweep over attention shapes (ragged lengths, shifted diagonals, GQA, both head dims, all launch-size classes):
forward and backward through the C ABI against an fp32 torch reference computed on the GPU."""
import math
import random

import pytest
import torch

pytestmark = pytest.mark.gpu


def reference(q, k, v, scale, q_offset, causal, do):
    q, k, v = (t.float().detach().requires_grad_() for t in (q, k, v))
    rep = q.size(1) // k.size(1)
    s = (q @ k.repeat_interleave(rep, 1).transpose(-1, -2)) * scale
    if causal:
        qi = torch.arange(q.size(2), device=q.device)[:, None] + q_offset
        kj = torch.arange(k.size(2), device=q.device)[None, :]
        s = s.masked_fill(kj > qi, float("-inf"))
    lse = torch.logsumexp(s, -1)
    p = torch.exp(s - lse.masked_fill(lse == float("-inf"), 0.0)[..., None])
    p = torch.where(torch.isfinite(s), p, torch.zeros_like(p))      # rows that see no key: all zeros
    out = p @ v.repeat_interleave(rep, 1)
    gq, gk, gv = torch.autograd.grad(out, (q, k, v), do.float())
    return out.detach(), lse.detach(), gq, gk, gv


def rel_l2(a, b):
    a, b = a.double(), b.double()
    if (a - b).abs().max().item() <= 1e-4:      # both (near) zero, e.g. one visible key: dS = 0
        return 0.0
    return ((a - b).norm() / b.norm().clamp_min(1e-20)).item()


def cases(count, seed):
    rng = random.Random(seed)
    for case in range(count):
        D = rng.choice([64, 64, 128])
        Hkv = rng.choice([1, 2, 4, 8])
        Hq = Hkv * rng.choice([1, 1, 2, 4])
        B = rng.choice([1, 1, 2, 3])
        Sq = rng.choice([1, 7, 31, 32, 33, 63, 64, 65, 100, 128, 129, 191, 256, 300, 511, 777, 1024])
        causal = rng.random() < 0.7
        if causal and rng.random() < 0.5:
            Sk, q_offset = Sq, 0
        else:
            Sk = rng.choice([1, 17, 64, 65, 127, 128, 129, 200, 256, 383, 512, 640, 1000, 1537])
            q_offset = rng.choice([0, 0, 5, 64, 100, 128, max(Sk - Sq, 0)]) if causal else 0
        if rng.random() < 0.15:                 # enough heads for the 8-wave / 4-wave launch classes
            B, Hq, Hkv = 2, 32, 32 // rng.choice([1, 4])
        yield case, B, Hq, Hkv, Sq, Sk, D, causal, q_offset


def test_seeded_shape_sweep(device):
    from picotron_amd import ops
    failures = []
    for case, B, Hq, Hkv, Sq, Sk, D, causal, q_offset in cases(80, seed=2024):
        g = torch.Generator().manual_seed(case)
        q = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16).to(device)
        k = torch.randn(B, Hkv, Sk, D, generator=g).to(torch.bfloat16).to(device)
        v = torch.randn(B, Hkv, Sk, D, generator=g).to(torch.bfloat16).to(device)
        do = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16).to(device)
        scale = 1 / math.sqrt(D)
        out, lse = ops.attn_fwd(q, k, v, scale, causal, q_offset)
        dq, dk, dv = ops.attn_bwd(do, q, k, v, lse, None, scale, causal, q_offset, dq_dtype=torch.float32,
                                  dkv_dtype=torch.float32, out=out)
        # the reference runs on whole GQA groups: the first 8 query heads (or all) and the kv heads they read
        nq = min(Hq, 8)
        nkv = max(1, nq // (Hq // Hkv))
        nq = nkv * (Hq // Hkv)
        r_o, r_l, r_dq, r_dk, r_dv = reference(q[:, :nq], k[:, :nkv], v[:, :nkv], scale, q_offset, causal, do[:, :nq])
        fin = torch.isfinite(r_l)
        errs = {
            "out": (out[:, :nq].float() - r_o).abs().max().item() <= 2e-2,
            "lse": (not fin.any()) or (lse[:, :nq][fin] - r_l[fin]).abs().max().item() <= 1e-3,
            "lse -inf rows": (fin.all()) or bool((lse[:, :nq][~fin] == float("-inf")).all()),
            "dq": rel_l2(dq[:, :nq], r_dq) <= 1e-2,
            "dk": rel_l2(dk[:, :nkv], r_dk) <= 1e-2,
            "dv": rel_l2(dv[:, :nkv], r_dv) <= 1e-2,
        }
        bad = [n for n, ok in errs.items() if not ok]
        if bad:
            failures.append((case, B, Hq, Hkv, Sq, Sk, D, causal, q_offset, bad))
    assert not failures, failures


def test_seeded_sweep_of_rope_inside_attention(device):
    """pico_attn_fwd_rope / pico_attn_bwd_rope over 40 seeded shapes (every launch-size class, GQA, ragged lengths,
    position offsets, both table dtypes) against the same kernels fed by separate RoPE launches: identical forward
    (the rotated q is bit-equal), gradients equal up to the one rounding the fused path does not do twice."""
    from picotron_amd import ops
    from oracle import layers as OL
    failures = []
    for case, B, Hq, Hkv, Sq, Sk, D, causal, q_offset in cases(40, seed=77):
        rng = random.Random(case)
        pos0 = rng.choice([0, 0, 3, 129, 1000])
        tdt = rng.choice([torch.bfloat16, torch.float32])
        g = torch.Generator().manual_seed(500 + case)
        q = torch.randn(B, Sq, Hq, D, generator=g).to(torch.bfloat16).to(device).transpose(1, 2)
        k = torch.randn(B, Sk, Hkv, D, generator=g).to(torch.bfloat16).to(device).transpose(1, 2)
        v = torch.randn(B, Sk, Hkv, D, generator=g).to(torch.bfloat16).to(device).transpose(1, 2)
        do = torch.randn(B, Sq, Hq, D, generator=g).to(torch.bfloat16).to(device).transpose(1, 2)
        scale = 1 / math.sqrt(D)
        cos, sin = OL.get_cos_sin(pos0 + q_offset + max(Sq, Sk) + 1, D, 10000.0, tdt)
        cos, sin = cos.to(device), sin.to(device)
        qp, kp = pos0 + q_offset, pos0
        k_rot = ops.rope(k, cos, sin, pos_offset=kp)
        q_rot_ref = ops.rope(q, cos, sin, pos_offset=qp)
        o0, l0 = ops.attn_fwd(q_rot_ref, k_rot, v, scale, causal, q_offset, bshd_out=True)
        o1, l1, q_rot = ops.attn_fwd_rope(q, k_rot, v, cos, sin, scale, causal, q_offset, q_pos_offset=qp)
        bad = []
        if not (torch.equal(q_rot, q_rot_ref) and torch.equal(o0, o1) and torch.equal(l0, l1)):
            bad.append("forward")

        def grads():
            return (torch.empty(B, Sq, Hq, D, dtype=torch.bfloat16, device=device).transpose(1, 2),
                    torch.empty(B, Sk, Hkv, D, dtype=torch.bfloat16, device=device).transpose(1, 2),
                    torch.empty(B, Sk, Hkv, D, dtype=torch.bfloat16, device=device).transpose(1, 2))
        dq0, dk0, dv0 = grads()
        ops.attn_bwd(do, q_rot, k_rot, v, l0, None, scale, causal, q_offset, dq0, dk0, dv0, out=o0)
        dq0 = ops.rope(dq0, cos, sin, pos_offset=qp, inverse=True)
        dk0 = ops.rope(dk0, cos, sin, pos_offset=kp, inverse=True)
        dq1, dk1, dv1 = grads()
        ops.attn_bwd_rope(do, q_rot, k_rot, v, o1, l1, cos, sin, scale, causal, dq1, dk1, dv1, q_offset,
                          q_pos_offset=qp, k_pos_offset=kp)
        if not torch.equal(dv0, dv1):
            bad.append("dv")
        if rel_l2(dq1, dq0) > 6e-3:
            bad.append("dq")
        if rel_l2(dk1, dk0) > 6e-3:
            bad.append("dk")
        if bad:
            failures.append((case, B, Hq, Hkv, Sq, Sk, D, causal, q_offset, pos0, str(tdt), bad))
    assert not failures, failures


def test_seeded_sweep_of_the_bandwidth_kernels(device):
    """RMSNorm (both rounding orders, with and without the fused residual), SwiGLU and cross-entropy, forward and
    backward, at 40 seeded sizes against torch in fp32 on the GPU."""
    import torch.nn.functional as F
    from picotron_amd import ops
    rng = random.Random(7)
    failures = []
    for case in range(40):
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float32])
        tol = 4e-2 if dtype == torch.bfloat16 else 2e-5
        rows = rng.choice([1, 3, 17, 64, 255, 1000, 4096])
        hidden = 8 * rng.choice([1, 9, 72, 96, 128, 256, 333, 512, 1024])
        g = torch.Generator().manual_seed(1000 + case)
        x = torch.randn(rows, hidden, generator=g).to(dtype).to(device)
        res = torch.randn(rows, hidden, generator=g).to(dtype).to(device)
        w = (torch.rand(hidden, generator=g) + 0.5).to(dtype).to(device)
        dy = torch.randn(rows, hidden, generator=g).to(dtype).to(device)
        eps = 1e-5
        bad = []
        # RMSNorm
        for cts in (False, True):
            y, rstd, _ = ops.rmsnorm_fwd(x, w, eps, cts)
            xf = x.float().requires_grad_()
            wf = w.float().requires_grad_()
            normed = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
            want = (normed.to(dtype).float() * wf) if cts else normed * wf
            if (y.float() - want).abs().max().item() > tol * max(1.0, want.abs().max().item()):
                bad.append(f"rmsnorm_fwd cts={cts}")
        y, rstd, h = ops.rmsnorm_fwd(x, w, eps, False, residual=res, want_residual_out=True)
        hf = (x.float() + res.float()).to(dtype).float().requires_grad_()
        wf = w.float().requires_grad_()
        want = hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + eps) * wf
        gx, gw = torch.autograd.grad(want, (hf, wf), dy.float())
        dx, dw = ops.rmsnorm_bwd(dy, h, w, rstd, dresidual=res)
        if (h.float() - hf).abs().max().item() > 0 or rel_l2(y.float(), want.detach()) > 1e-2:
            bad.append("rmsnorm_fwd residual")
        if rel_l2(dx.float(), gx + res.float()) > 1e-2 or rel_l2(dw.float(), gw) > 1e-2:
            bad.append("rmsnorm_bwd")
        # SwiGLU
        gf, uf = x.float().requires_grad_(), res.float().requires_grad_()
        want = F.silu(gf) * uf
        ggate, gup = torch.autograd.grad(want, (gf, uf), dy.float())
        dgate, dup = ops.swiglu_bwd(dy, x, res)
        if rel_l2(ops.swiglu_fwd(x, res).float(), want.detach()) > 1e-2 or rel_l2(dgate.float(), ggate) > 1e-2 or rel_l2(dup.float(), gup) > 1e-2:
            bad.append("swiglu")
        # cross-entropy over `hidden` classes
        tgt = torch.randint(0, hidden, (rows,), generator=g).to(device)
        if rows > 2:
            tgt[1] = -100
        lf = x.float().requires_grad_()
        want_loss = F.cross_entropy(lf, tgt, ignore_index=-100, reduction="none")
        loss_rows, lse = ops.cross_entropy_fwd(x, tgt)
        count = max(int((tgt != -100).sum().item()), 1)
        (gl,) = torch.autograd.grad(want_loss.sum() / count, lf)
        dl = ops.cross_entropy_bwd(x, tgt, lse, torch.full((1,), 1.0 / count, device=device))
        if (loss_rows - want_loss.detach()).abs().max().item() > 1e-3 or rel_l2(dl.float(), gl) > 1e-2:
            bad.append("cross_entropy")
        if bad:
            failures.append((case, str(dtype), rows, hidden, bad))
    assert not failures, failures
