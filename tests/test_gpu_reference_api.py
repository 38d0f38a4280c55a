"""The mirrored reference functions called the way the reference's own code calls them, one by one, against the oracle:
``ring_attention_forward`` / ``update_out_and_lse`` / ``ring_attention_backward`` strung together by hand into the ring
of ``RingAttentionFunc`` (``context_parallel.py:22-110``), and ``apply_rotary_pos_emb`` / ``get_cos_sin`` /
``LlamaRMSNorm`` / ``TritonRMSNorm`` / ``MLP`` with the argument lists of ``model.py``."""
import math
import os

import pytest
import torch

from oracle import layers as OL
from oracle import ring as OR

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def maxabs(a, b):
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


@pytest.fixture()
def cp(device):
    import picotron_amd.process_group_manager as pgm
    pgm.setup_process_group_manager(1, 1, 1, 1)
    os.environ["CONTEXT_PARALLEL"] = "0"
    from picotron_amd.context_parallel import context_parallel
    return context_parallel


@pytest.mark.parametrize("world", [1, 2, 4])
def test_block_functions_compose_into_the_ring_by_hand(cp, device, world):
    """For every rank: blocks in the order the ring delivers them (own chunk first, then rank-1, ...), causal only on
    the first, merged with update_out_and_lse; then the backward block by block with the final out / lse, dq summed
    per rank and dk / dv summed per chunk -- everything through the three public functions."""
    B, H, S, D = 2, 3, 64 * world, 64
    Sc, scale = S // world, 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(11)
    q, k, v, do = (torch.randn(B, H, S, D, generator=g).to(torch.bfloat16) for _ in range(4))
    w_o, w_l = OR.all_ranks_forward(q.float(), k.float(), v.float(), world, scale, True)
    w_dq, w_dk, w_dv = OR.all_ranks_backward(do.float(), q.float(), k.float(), v.float(), w_o, w_l, world, scale, True)
    qd, kd, vd, dod = (t.to(device) for t in (q, k, v, do))
    chunk = lambda t, c: t[:, :, c * Sc:(c + 1) * Sc].contiguous()
    dk = torch.zeros(B, H, S, D, dtype=torch.float32, device=device)
    dv = torch.zeros_like(dk)
    for rank in range(world):
        q_r, do_r = chunk(qd, rank), chunk(dod, rank)
        out = lse = None
        for step in range(rank + 1):
            held = rank - step
            block_out, block_lse = cp.ring_attention_forward(q_r, chunk(kd, held), chunk(vd, held), scale, step == 0)
            assert block_out.shape == (B, H, Sc, D) and block_out.dtype == q_r.dtype and block_lse.shape == (B, H, Sc)
            out, lse = cp.update_out_and_lse(out, lse, block_out, block_lse)
            assert out.dtype == torch.float32 and lse.shape == (B, H, Sc, 1)
        out = out.to(q_r.dtype)
        lse = lse.squeeze(dim=-1)
        rows = slice(rank * Sc, (rank + 1) * Sc)
        assert maxabs(out, w_o[:, :, rows]) <= 2e-2 and maxabs(lse, w_l[:, :, rows]) <= 1e-3
        dq = None
        for step in range(rank + 1):
            held = rank - step
            b_dq, b_dk, b_dv = cp.ring_attention_backward(do_r, q_r, chunk(kd, held), chunk(vd, held), out, lse, scale, step == 0)
            dq = b_dq.to(torch.float32) if dq is None else dq + b_dq
            dk[:, :, held * Sc:(held + 1) * Sc] += b_dk
            dv[:, :, held * Sc:(held + 1) * Sc] += b_dv
        assert rel_l2(dq, w_dq[:, :, rows]) <= 1e-2
    assert rel_l2(dk, w_dk) <= 1e-2 and rel_l2(dv, w_dv) <= 1e-2


def test_first_update_with_a_slice_is_an_error(cp, device):
    o = torch.zeros(1, 1, 4, 64, device=device)
    l = torch.zeros(1, 1, 4, device=device)
    with pytest.raises(RuntimeError, match="first update_out_and_lse should not pass slice_ args"):
        cp.update_out_and_lse(None, None, o, l, slice_=(slice(None),))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rotary_functions_with_the_reference_argument_lists(device, dtype, monkeypatch):
    from picotron_amd import model as M
    monkeypatch.setenv("DTYPE", "bfloat16" if dtype == torch.bfloat16 else "float32")
    monkeypatch.setenv("LOCAL_RANK", "0")
    S, D = 96, 64
    cos, sin = M.get_cos_sin(S, head_dim=D, base=10000.0)
    w_cos, w_sin = OL.get_cos_sin(S, D, 10000.0, dtype=dtype)
    assert cos.shape == (S, D) and cos.dtype == dtype and cos.is_cuda
    # the angles are computed on the device in fp32: the device's cos / sin may differ from the host's in the last bit
    assert maxabs(cos, w_cos) <= (8e-3 if dtype == torch.bfloat16 else 2e-6) and maxabs(sin, w_sin) <= (8e-3 if dtype == torch.bfloat16 else 2e-6)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 5, S, D, generator=g).to(dtype)
    y = M.apply_rotary_pos_emb(x.to(device), cos, sin)
    want = OL.apply_rotary_pos_emb(x.float(), cos.float().cpu(), sin.float().cpu())
    assert y.dtype == dtype and maxabs(y, want) <= (3e-2 if dtype == torch.bfloat16 else 1e-5)
    # the layout Attention.forward hands over: [B,H,S,D] as a transposed view of [B,S,H,D]
    xt = x.transpose(1, 2).contiguous().to(device).transpose(1, 2)
    assert torch.equal(M.apply_rotary_pos_emb(xt, cos, sin), y)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_norm_modules_with_the_reference_argument_lists(device, dtype):
    from picotron_amd import model as M
    h, eps = 576, 1e-5
    g = torch.Generator().manual_seed(6)
    x = torch.randn(2, 33, h, generator=g).to(dtype)
    res = torch.randn(2, 33, h, generator=g).to(dtype)
    w = (torch.rand(h, generator=g) + 0.5).to(dtype)
    tol = 4e-2 if dtype == torch.bfloat16 else 1e-5

    llama = M.LlamaRMSNorm(h, eps=eps).to(device=device, dtype=dtype)
    triton = M.TritonRMSNorm(h, eps=eps, device=device, dtype=dtype)
    assert torch.equal(llama.weight, torch.ones_like(llama.weight)) and torch.equal(triton.weight, torch.ones_like(triton.weight))
    with torch.no_grad():
        llama.weight.copy_(w)
        triton.weight.copy_(w)
    y = llama(x.to(device))
    assert y.dtype == dtype and maxabs(y, OL.rmsnorm(x, w, eps, cast_then_scale=True).float()) <= tol
    y = triton(x.to(device), residual=None, dropout_p=0.0, prenorm=False, residual_in_fp32=False, return_dropout_mask=False)
    assert y.dtype == dtype and maxabs(y, OL.rmsnorm(x.float(), w.float(), eps, cast_then_scale=False)) <= tol
    # residual= / prenorm= as flash-attn's layer_norm_fn defines them: the sum is normalised and returned as well
    y, hsum = triton(x.to(device), residual=res.to(device), prenorm=True)
    want_sum = (x.float() + res.float()).to(dtype)
    assert maxabs(hsum, want_sum.float()) <= (4e-2 if dtype == torch.bfloat16 else 1e-6)
    assert maxabs(y, OL.rmsnorm(hsum.float().cpu(), w.float(), eps, cast_then_scale=False)) <= tol
    # dropout_p / residual_in_fp32 / return_dropout_mask, the rest of layer_norm_fn's argument list: the returned keep
    # mask fixes the expected value (h = x * mask / (1 - p) + residual, kept in fp32 when asked; y = rmsnorm(h) * w)
    torch.manual_seed(11)
    y, hsum, mask, mask1 = triton(x.to(device), residual=res.to(device), dropout_p=0.25, prenorm=True, residual_in_fp32=True,
                                  return_dropout_mask=True)
    assert mask1 is None and mask.dtype == torch.bool and 0.6 < mask.float().mean().item() < 0.9
    want_h = x.float() * mask.cpu() / 0.75 + res.float()
    assert hsum.dtype == torch.float32 and maxabs(hsum, want_h) <= 1e-5
    assert y.dtype == dtype and maxabs(y, OL.rmsnorm(want_h, w.float(), eps, cast_then_scale=False)) <= tol
    y2, mask2, _ = triton(x.to(device), dropout_p=0.0, return_dropout_mask=True)
    assert bool(mask2.all()) and maxabs(y2, OL.rmsnorm(x.float(), w.float(), eps, cast_then_scale=False)) <= tol
    # and gradients flow through the composed path
    xg = x.to(device).requires_grad_()
    y3, h3 = triton(xg, residual=res.to(device), prenorm=True, residual_in_fp32=True)
    (y3.float().sum() + h3.sum()).backward()
    assert xg.grad is not None and triton.weight.grad is not None and torch.isfinite(xg.grad.float()).all()


def test_mlp_module_matches_the_oracle_formula(device):
    from types import SimpleNamespace
    from picotron_amd import model as M
    cfg = SimpleNamespace(hidden_size=128, intermediate_size=384)
    torch.manual_seed(7)
    mlp = M.MLP(cfg).to(device=device, dtype=torch.bfloat16)
    x = torch.randn(2, 17, 128).to(torch.bfloat16)
    xd = x.to(device).requires_grad_()
    y = mlp(xd)
    wg, wu, wd = (getattr(mlp, n).weight.detach().float().cpu() for n in ("gate_proj", "up_proj", "down_proj"))
    xf = x.float().requires_grad_()
    want = OL.swiglu(xf @ wg.t(), xf @ wu.t()) @ wd.t()
    assert rel_l2(y, want.detach()) <= 1e-2
    gy = torch.randn(2, 17, 128, generator=torch.Generator().manual_seed(8)).to(torch.bfloat16)
    y.backward(gy.to(device))
    want.backward(gy.float())
    assert rel_l2(xd.grad, xf.grad) <= 2e-2
