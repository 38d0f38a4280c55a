"""Pins oracle/layers.py: cos/sin tables, RoPE, RMSNorm, SwiGLU -- against transformers' local Llama
implementation, torch library routines, fp64 closed forms, autograd and rotation invariants."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import layers


def rnd(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=dtype)


# ------------------------------------------------------------------ cos / sin tables
@pytest.mark.parametrize("S,D,base", [(64, 64, 10000.0), (128, 128, 10000.0), (33, 16, 500000.0)])
def test_cos_sin_closed_form(S, D, base):
    cos, sin = layers.get_cos_sin(S, D, base, dtype=torch.float32)
    assert cos.shape == (S, D) and sin.shape == (S, D)
    # halves are duplicates
    assert torch.equal(cos[:, :D // 2], cos[:, D // 2:]) and torch.equal(sin[:, :D // 2], sin[:, D // 2:])
    i = torch.arange(0, D, 2, dtype=torch.float64)
    ang = torch.arange(S, dtype=torch.float64).unsqueeze(1) * (1.0 / base ** (i / D))
    # fp32 angle of magnitude up to S carries ~S*6e-8 absolute error
    assert torch.allclose(cos[:, :D // 2].double(), torch.cos(ang), atol=S * 2e-7)
    assert torch.allclose(sin[:, :D // 2].double(), torch.sin(ang), atol=S * 2e-7)
    # position 0 is the identity rotation
    assert torch.equal(cos[0], torch.ones(D)) and torch.equal(sin[0], torch.zeros(D))


def test_cos_sin_default_dtype_is_bf16():
    cos32, sin32 = layers.get_cos_sin(16, 8, 10000.0, dtype=torch.float32)
    cos, sin = layers.get_cos_sin(16, 8, 10000.0)
    assert cos.dtype == torch.bfloat16
    assert torch.equal(cos, cos32.to(torch.bfloat16)) and torch.equal(sin, sin32.to(torch.bfloat16))


def test_cos_sin_vs_transformers_rotary():
    tr = pytest.importorskip("transformers")
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
    cfg = tr.LlamaConfig(hidden_size=256, num_attention_heads=4, max_position_embeddings=96, rope_theta=10000.0)
    try:
        rot = LlamaRotaryEmbedding(config=cfg)
    except Exception as e:  # API drift in the installed version
        pytest.skip(f"LlamaRotaryEmbedding not constructible: {e}")
    x = torch.zeros(1, 96, 256)
    cos_t, sin_t = rot(x, torch.arange(96).unsqueeze(0))
    cos, sin = layers.get_cos_sin(96, 64, 10000.0, dtype=torch.float32)
    assert torch.allclose(cos, cos_t[0].float(), atol=1e-5) and torch.allclose(sin, sin_t[0].float(), atol=1e-5)


# ------------------------------------------------------------------ RoPE
def test_rope_vs_transformers():
    pytest.importorskip("transformers")
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb as hf_rope
    x = rnd(2, 3, 10, 8, seed=1, dtype=torch.float32)
    cos, sin = layers.get_cos_sin(10, 8, 10000.0, dtype=torch.float32)
    want, _ = hf_rope(x, x, cos.unsqueeze(0), sin.unsqueeze(0))
    assert torch.allclose(layers.apply_rotary_pos_emb(x, cos, sin), want, atol=1e-6)


def test_rope_explicit_pairs_and_invariants():
    B, H, S, D = 1, 2, 7, 6
    x = rnd(B, H, S, D, seed=2)
    cos, sin = layers.get_cos_sin(S, D, 100.0, dtype=torch.float64)
    y = layers.apply_rotary_pos_emb(x, cos, sin)
    half = D // 2
    for s in range(S):
        for i in range(half):
            th = s * (1.0 / 100.0 ** (2 * i / D))
            a, b = x[0, 1, s, i], x[0, 1, s, i + half]
            assert math.isclose(y[0, 1, s, i].item(), a * math.cos(th) - b * math.sin(th), abs_tol=1e-6)
            assert math.isclose(y[0, 1, s, i + half].item(), b * math.cos(th) + a * math.sin(th), abs_tol=1e-6)
    # pairwise norm preserved (up to the fp32 angle), position 0 untouched
    n_in = x[..., :half] ** 2 + x[..., half:] ** 2
    n_out = y[..., :half] ** 2 + y[..., half:] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-5)
    assert torch.allclose(y[:, :, 0], x[:, :, 0])


def test_rope_backward_closed_form_vs_autograd():
    x = rnd(2, 2, 9, 8, seed=3).requires_grad_()
    dy = rnd(2, 2, 9, 8, seed=4)
    cos, sin = layers.get_cos_sin(9, 8, 10000.0, dtype=torch.float64)
    (gx,) = torch.autograd.grad(layers.apply_rotary_pos_emb(x, cos, sin), x, dy)
    assert torch.allclose(layers.apply_rotary_pos_emb_backward(dy, cos, sin), gx, atol=1e-12)
    # the adjoint is the inverse rotation
    y = layers.apply_rotary_pos_emb(x.detach(), cos, sin)
    assert torch.allclose(layers.apply_rotary_pos_emb_backward(y, cos, sin), x.detach(), atol=1e-5)


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_vs_transformers_llama(dtype):
    pytest.importorskip("transformers")
    from transformers.models.llama.modeling_llama import LlamaRMSNorm
    x = rnd(3, 5, 64, seed=5, dtype=torch.float32).to(dtype)
    w = (1 + 0.1 * rnd(64, seed=6, dtype=torch.float32)).to(dtype)
    m = LlamaRMSNorm(64, eps=1e-5)
    with torch.no_grad():
        m.weight.copy_(w)
        want = m.to(dtype)(x)
    got = layers.rmsnorm(x, w, 1e-5, cast_then_scale=True)
    assert got.dtype == want.dtype
    assert torch.equal(got, want)


def test_rmsnorm_vs_functional_rms_norm():
    x = rnd(4, 7, 32, seed=7, dtype=torch.float32)
    w = 1 + 0.1 * rnd(32, seed=8, dtype=torch.float32)
    want = F.rms_norm(x, (32,), w, 1e-5)
    assert torch.allclose(layers.rmsnorm(x, w, 1e-5, True), want, atol=1e-6)
    assert torch.allclose(layers.rmsnorm(x, w, 1e-5, False), want, atol=1e-6)


def test_rmsnorm_backward_closed_form_vs_autograd():
    x = rnd(3, 4, 16, seed=9).requires_grad_()
    w = (1 + 0.1 * rnd(16, seed=10)).requires_grad_()
    dy = rnd(3, 4, 16, seed=11)
    gx, gw = torch.autograd.grad(layers.rmsnorm(x, w, 1e-5), (x, w), dy)
    dx, dw = layers.rmsnorm_backward(dy, x.detach(), w.detach(), 1e-5)
    assert torch.allclose(dx, gx, atol=1e-12) and torch.allclose(dw, gw, atol=1e-12)
    assert torch.autograd.gradcheck(lambda a, b: layers.rmsnorm(a, b, 1e-5), (x, w))


# ------------------------------------------------------------------ SwiGLU
def test_swiglu_forward_and_backward():
    g, u = rnd(5, 12, seed=12).requires_grad_(), rnd(5, 12, seed=13).requires_grad_()
    dy = rnd(5, 12, seed=14)
    y = layers.swiglu(g, u)
    assert torch.allclose(y, g * torch.sigmoid(g) * u, atol=1e-14)
    gg, gu = torch.autograd.grad(y, (g, u), dy)
    dg, du = layers.swiglu_backward(dy, g.detach(), u.detach())
    assert torch.allclose(dg, gg, atol=1e-12) and torch.allclose(du, gu, atol=1e-12)
    # spot values: silu(0) = 0, d/dg silu at 0 = 1/2
    z = torch.zeros(1, dtype=torch.float64)
    dg0, du0 = layers.swiglu_backward(torch.ones(1, dtype=torch.float64), z, torch.full((1,), 3.0, dtype=torch.float64))
    assert dg0.item() == pytest.approx(1.5) and du0.item() == 0.0


def test_adamw_step_matches_torch_adamw():
    """oracle.optim.adamw_step against torch.optim.AdamW (the routine the reference calls, train.py:204-209) over
    five steps with changing gradients, in fp64 and fp32; a wrong bias correction, a coupled weight decay or a
    swapped beta shows up in the first step already."""
    from oracle import optim as OO
    for dtype, tol in ((torch.float64, 1e-12), (torch.float32, 2e-6)):
        g = torch.Generator().manual_seed(7)
        p0 = torch.randn(257, generator=g, dtype=torch.float64).to(dtype)
        ref = torch.nn.Parameter(p0.clone())
        opt = torch.optim.AdamW([ref], lr=3e-3, betas=(0.85, 0.97), eps=1e-7, weight_decay=0.05)
        p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
        for step in range(1, 6):
            grad = torch.randn(257, generator=g, dtype=torch.float64).to(dtype) * (0.1 * step)
            ref.grad = grad.clone()
            opt.step()
            p, m, v = OO.adamw_step(p, grad, m, v, step, 3e-3, 0.85, 0.97, 1e-7, 0.05)
            assert (p - ref.detach()).abs().max().item() <= tol * max(1.0, p.abs().max().item())
        st = opt.state[ref]
        assert (m - st["exp_avg"]).abs().max().item() <= tol and (v - st["exp_avg_sq"]).abs().max().item() <= tol


def test_adamw_lp_step_matches_torch_fused_adamw():
    """oracle.optim.lp_step (bf16 parameter and moments, fp32 arithmetic, one rounding per state) against
    torch.optim.AdamW(fused=True) on a bf16 parameter: after five steps every state is within one bf16 ulp and
    almost all are identical (the two may order a multiplication differently inside fp32)."""
    from oracle import optim as OO
    g = torch.Generator().manual_seed(11)
    p0 = torch.randn(4099, generator=g).bfloat16()
    ref = torch.nn.Parameter(p0.clone())
    try:
        opt = torch.optim.AdamW([ref], lr=3e-3, betas=(0.85, 0.97), eps=1e-7, weight_decay=0.05, fused=True)
    except RuntimeError as e:   # a torch build without the fused CPU kernel
        pytest.skip(f"torch has no fused AdamW on the CPU: {e}")
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    for step in range(1, 6):
        grad = (torch.randn(4099, generator=g) * (0.1 * step)).bfloat16()
        ref.grad = grad.clone()
        opt.step()
        p, m, v = OO.lp_step(p, grad, m, v, step, 3e-3, beta1=0.85, beta2=0.97, eps=1e-7, weight_decay=0.05)
    st = opt.state[ref]
    for got, want in ((p, ref.detach()), (m, st["exp_avg"]), (v, st["exp_avg_sq"])):
        assert got.dtype == want.dtype == torch.bfloat16
        diff = (got.float() - want.float()).abs()
        assert (diff <= want.float().abs() * 2.0 ** -7 + want.float().abs().mean() * 2.0 ** -7).all()
        assert (diff == 0).float().mean().item() >= 0.98


def test_cross_entropy_matches_torch():
    """oracle.layers.cross_entropy / _backward against F.cross_entropy (the routine train.py:49 calls) and autograd,
    with ignored rows."""
    import torch.nn.functional as F
    from oracle import layers as OL
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(37, 101, generator=g, dtype=torch.float64) * 3).requires_grad_()
    t = torch.randint(0, 101, (37,), generator=g)
    t[3] = -100
    t[20] = -100
    want = F.cross_entropy(x, t, reduction="mean")
    got, lse = OL.cross_entropy(x.detach(), t)
    assert abs(got.item() - want.item()) <= 1e-6
    assert (lse - torch.logsumexp(x.detach(), -1)).abs().max().item() <= 1e-6
    (gx,) = torch.autograd.grad(want * 0.7, x)
    assert (OL.cross_entropy_backward(x.detach(), t, 0.7) - gx).abs().max().item() <= 1e-6
