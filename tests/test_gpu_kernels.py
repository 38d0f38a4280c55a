"""GPU parity: every C-ABI kernel against the CPU oracle on the same seeded inputs.

Tolerances (from the acceptance criteria of the path): bf16 forward outputs max-abs <= 2e-2,
lse <= 1e-3, gradients relative L2 <= 1e-2, all against an fp32 oracle; fp32 kernels much tighter.
"""
import math

import pytest
import torch

from oracle import layers as OL
from oracle import ring as OR

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def maxabs(a, b):
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


@pytest.fixture(scope="module")
def ops(device):
    from picotron_amd import ops as _ops
    return _ops


# ------------------------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("rows,hidden", [(7, 576), (64, 2048), (33, 4096), (5, 8192), (3, 64), (0, 128), (6, 16384), (9, 12288)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("cts", [True, False])
def test_rmsnorm_fwd(ops, device, rows, hidden, dtype, cts):
    x = rnd(rows, hidden, seed=1, dtype=dtype)
    w = (1 + 0.1 * rnd(hidden, seed=2)).to(dtype)
    y, rstd, _ = ops.rmsnorm_fwd(x.to(device), w.to(device), 1e-5, cts)
    want = OL.rmsnorm(x, w, 1e-5, cast_then_scale=cts)
    assert y.dtype == dtype and y.shape == x.shape
    if rows == 0:
        return
    if dtype == torch.float32:
        assert maxabs(y, want) <= 2e-5
    else:
        # same bf16 roundings as the oracle except where the fp32 reduction order flips a rounding
        assert maxabs(y, want) <= 2e-2
        assert (y.cpu() != want).float().mean().item() < 0.02
    want_rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    assert torch.allclose(rstd.cpu(), want_rstd, rtol=1e-5, atol=1e-6)


def test_rmsnorm_fwd_residual(ops, device):
    x, r = rnd(9, 1024, seed=3, dtype=torch.bfloat16), rnd(9, 1024, seed=4, dtype=torch.bfloat16)
    w = (1 + 0.1 * rnd(1024, seed=5)).to(torch.bfloat16)
    y, _, res = ops.rmsnorm_fwd(x.to(device), w.to(device), 1e-5, False, residual=r.to(device), want_residual_out=True)
    h = x.float() + r.float()
    assert maxabs(res, h.to(torch.bfloat16)) == 0.0
    assert maxabs(y, OL.rmsnorm(h, w.float(), 1e-5, cast_then_scale=False)) <= 2e-2


@pytest.mark.parametrize("rows,hidden", [(7, 576), (300, 2048), (1030, 1024), (33, 4096), (5, 8192), (0, 64), (6, 16384), (9, 12288)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_bwd(ops, device, rows, hidden, dtype):
    x, dy = rnd(rows, hidden, seed=6, dtype=dtype), rnd(rows, hidden, seed=7, dtype=dtype)
    w = (1 + 0.1 * rnd(hidden, seed=8)).to(dtype)
    rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    dx, dw = ops.rmsnorm_bwd(dy.to(device), x.to(device), w.to(device), rstd.to(device))
    want_dx, want_dw = OL.rmsnorm_backward(dy, x, w, 1e-5)
    assert dw.dtype == torch.float32 and dw.shape == (hidden,)
    if rows == 0:
        assert dw.abs().max().item() == 0.0
        return
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert rel_l2(dx, want_dx) <= tol
    assert rel_l2(dw, want_dw) <= 1e-5


@pytest.mark.parametrize("rows,hidden", [(7, 576), (300, 2048), (33, 8192), (1030, 1024)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_bwd_adds_residual_gradient_and_rounds_dweight(ops, device, rows, hidden, dtype):
    """dresidual is added to dx inside the kernel (fp32 sum, one rounding) and dweight comes back in the requested
    dtype: against the oracle's dx + dresidual, and bit-identical in dweight (after rounding) to the call without."""
    x, dy, dr = (rnd(rows, hidden, seed=s_, dtype=dtype) for s_ in (6, 7, 12))
    w = (1 + 0.1 * rnd(hidden, seed=8)).to(dtype)
    rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    dev = lambda t: t.to(device)
    dx0, dw0 = ops.rmsnorm_bwd(dev(dy), dev(x), dev(w), dev(rstd))
    dx, dw = ops.rmsnorm_bwd(dev(dy), dev(x), dev(w), dev(rstd), dresidual=dev(dr), dw_dtype=dtype)
    want_dx, _ = OL.rmsnorm_backward(dy, x, w, 1e-5)
    assert rel_l2(dx, want_dx.float() + dr.float()) <= (1e-5 if dtype == torch.float32 else 4e-3)
    assert dw.dtype == dtype and torch.equal(dw.cpu(), dw0.cpu().to(dtype))
    # the sum is taken before rounding: never further from the exact sum than rounding it once
    exact = dx0.double().cpu() * 0 + (want_dx.double() + dr.double())
    if dtype == torch.bfloat16:
        assert ((dx.double().cpu() - exact).abs() <= exact.abs() * 2.0 ** -8 + want_dx.double().abs() * 2.0 ** -7 + 1e-6).all()


def test_rmsnorm_bwd_is_bit_reproducible_at_every_row_length_class(ops, device):
    """dweight is summed without atomics: two runs give the same bits, for the row-per-wave kernels, for the rows a
    256-thread group owns (two groups per block meet in LDS, in group order) and for the longest rows."""
    for rows, hidden, dtype in ((1000, 2048, torch.bfloat16), (1000, 4096, torch.bfloat16), (700, 8192, torch.bfloat16),
                                (300, 16384, torch.bfloat16), (500, 8192, torch.float32), (900, 1000, torch.float32)):
        x = rnd(rows, hidden, seed=70, dtype=dtype).to(device)
        dy = rnd(rows, hidden, seed=71, dtype=dtype).to(device)
        w = (1 + 0.1 * rnd(hidden, seed=72)).to(dtype).to(device)
        _, rstd, _ = ops.rmsnorm_fwd(x, w, 1e-5, False)
        a = ops.rmsnorm_bwd(dy, x, w, rstd)
        for _ in range(3):
            b = ops.rmsnorm_bwd(dy, x, w, rstd)
            assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]), (rows, hidden, dtype)


# ------------------------------------------------------------------------------------ RoPE
@pytest.mark.parametrize("B,H,S,D", [(2, 3, 17, 64), (1, 4, 33, 128), (1, 2, 5, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
@pytest.mark.parametrize("table_dtype", [torch.bfloat16, torch.float32])
def test_rope_fwd_bwd(ops, device, B, H, S, D, dtype, layout, table_dtype):
    off = 11
    cos, sin = OL.get_cos_sin(off + S, D, 10000.0, dtype=table_dtype)
    if layout == "bhsd":
        x = rnd(B, H, S, D, seed=9, dtype=dtype)
    else:
        x = rnd(B, S, H, D, seed=9, dtype=dtype).transpose(1, 2)
    xd = x.to(device)
    if layout == "bshd":
        xd = x.transpose(1, 2).contiguous().to(device).transpose(1, 2)
    y = ops.rope(xd, cos.to(device), sin.to(device), pos_offset=off)
    want = OL.apply_rotary_pos_emb(x.float(), cos[off:].float(), sin[off:].float())
    assert y.shape == x.shape and y.stride() == xd.stride()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert maxabs(y, want) <= tol
    back = ops.rope(xd, cos.to(device), sin.to(device), pos_offset=off, inverse=True)
    assert maxabs(back, OL.apply_rotary_pos_emb_backward(x.float(), cos[off:].float(), sin[off:].float())) <= tol


def test_rope_positions_are_exact(ops, device):
    """pos_offset selects table rows exactly: rotating with offset r*Sc equals slicing the tables first."""
    S, D, W = 32, 64, 4
    cos, sin = OL.get_cos_sin(S, D, 10000.0)
    x = rnd(1, 2, S // W, D, seed=10, dtype=torch.bfloat16).to(device)
    for r in range(W):
        c_r, s_r = OR.rope_slice(cos, sin, r, W)
        a = ops.rope(x, cos.to(device), sin.to(device), pos_offset=r * (S // W))
        b = ops.rope(x, c_r.contiguous().to(device), s_r.contiguous().to(device), pos_offset=0)
        assert torch.equal(a, b)


# ------------------------------------------------------------------------------------ SwiGLU
@pytest.mark.parametrize("shape", [(3, 5, 1536), (64, 8192), (1, 8), (0, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_swiglu(ops, device, shape, dtype):
    g, u, dy = (rnd(*shape, seed=s, dtype=dtype) for s in (11, 12, 13))
    y = ops.swiglu_fwd(g.to(device), u.to(device))
    dg, du = ops.swiglu_bwd(dy.to(device), g.to(device), u.to(device))
    if g.numel() == 0:
        assert y.shape == g.shape
        return
    want = OL.swiglu(g.float(), u.float())
    wdg, wdu = OL.swiglu_backward(dy.float(), g.float(), u.float())
    if dtype == torch.float32:
        assert maxabs(y, want) <= 1e-5 and rel_l2(dg, wdg) <= 1e-5 and rel_l2(du, wdu) <= 1e-5
    else:
        assert rel_l2(y, want) <= 5e-3 and rel_l2(dg, wdg) <= 5e-3 and rel_l2(du, wdu) <= 5e-3


def test_swiglu_strided_halves(ops, device):
    """gate and up as the two halves of one [T, 2I] GEMM output (row pitch 2I)."""
    gu = rnd(10, 256, seed=14, dtype=torch.bfloat16).to(device)
    y = ops.swiglu_fwd(gu[:, :128], gu[:, 128:])
    want = OL.swiglu(gu[:, :128].float().cpu(), gu[:, 128:].float().cpu())
    assert rel_l2(y, want) <= 5e-3


# ------------------------------------------------------------------------------------ lse merge
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("bdtype", [torch.bfloat16, torch.float32])
def test_lse_merge(ops, device, D, bdtype):
    rows = (2, 3, 37)
    out, bo = rnd(*rows, D, seed=15), rnd(*rows, D, seed=16).to(bdtype)
    lse, bl = rnd(*rows, seed=17) * 3, rnd(*rows, seed=18) * 3
    bl[0, 0, :5] = float("-inf")           # a block that saw nothing leaves the row untouched
    lse[1, 1, :3] = float("-inf")          # a running state that saw nothing adopts the block
    o_d, l_d = out.to(device).clone(), lse.to(device).clone()
    ops.lse_merge_(o_d, l_d, bo.to(device), bl.to(device))
    w_o, w_l = OR.merge(out.clone(), lse.unsqueeze(-1).clone(), bo.float(), bl)
    w_l = w_l.squeeze(-1)
    assert torch.equal(o_d.cpu()[0, 0, :5], out[0, 0, :5]) and torch.equal(l_d.cpu()[0, 0, :5], lse[0, 0, :5])
    assert maxabs(o_d.cpu()[1, 1, :3], bo.float()[1, 1, :3]) <= 1e-6
    fin = torch.isfinite(w_l)
    assert maxabs(l_d.cpu()[fin], w_l[fin]) <= 1e-5
    ok = torch.isfinite(w_o).all(-1)
    assert maxabs(o_d.cpu()[ok], w_o[ok]) <= 1e-5


# ------------------------------------------------------------------------------------ attention forward
def attn_inputs(B, Hq, Hkv, Sq, Sk, D, seed):
    q = rnd(B, Hq, Sq, D, seed=seed, scale=1.0).to(torch.bfloat16)
    k = rnd(B, Hkv, Sk, D, seed=seed + 1).to(torch.bfloat16)
    v = rnd(B, Hkv, Sk, D, seed=seed + 2).to(torch.bfloat16)
    return q, k, v


def expand_kv(t, Hq):
    return t.repeat_interleave(Hq // t.size(1), dim=1)


FWD_CASES = [
    # B, Hq, Hkv, Sq, Sk, D, causal, q_offset
    (1, 2, 2, 128, 128, 64, True, 0),
    (2, 4, 4, 256, 256, 64, True, 0),
    (1, 2, 2, 256, 256, 64, False, 0),
    (1, 2, 2, 128, 512, 64, True, 384),     # all ring steps of rank 3 of 4 in one launch
    (1, 4, 2, 192, 192, 64, True, 0),       # GQA
    (1, 2, 2, 100, 100, 64, True, 0),       # ragged
    (1, 2, 1, 77, 203, 64, False, 0),       # ragged, rectangular, GQA
    (1, 2, 2, 256, 256, 128, True, 0),
    (1, 8, 2, 128, 384, 128, True, 256),
    (1, 1, 1, 61, 130, 128, False, 0),
    (1, 1, 1, 1, 1, 64, True, 0),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,q_offset", FWD_CASES)
def test_attn_fwd(ops, device, B, Hq, Hkv, Sq, Sk, D, causal, q_offset):
    q, k, v = attn_inputs(B, Hq, Hkv, Sq, Sk, D, seed=20)
    scale = 1 / math.sqrt(D)
    out, lse = ops.attn_fwd(q.to(device), k.to(device), v.to(device), scale, causal, q_offset)
    want_o, want_lse = OR.full_attention_closed_form(q.float(), expand_kv(k, Hq).float(), expand_kv(v, Hq).float(),
                                                     scale, causal, q_offset)
    assert out.dtype == torch.bfloat16 and lse.dtype == torch.float32
    assert maxabs(out, want_o) <= 2e-2
    assert maxabs(lse, want_lse) <= 1e-3


def test_attn_fwd_block_equals_oracle_block(ops, device):
    """The per-block entry (q_offset 0, Sq == Sk) is ring_attention_forward: diag masked, off-diag dense."""
    q, k, v = attn_inputs(2, 3, 3, 160, 160, 64, seed=30)
    for causal in (True, False):
        out, lse = ops.attn_fwd(q.to(device), k.to(device), v.to(device), 0.125, causal)
        w_o, w_l = OR.block_forward(q.float(), k.float(), v.float(), 0.125, causal)
        assert maxabs(out, w_o) <= 2e-2 and maxabs(lse, w_l) <= 1e-3


def test_attn_fwd_strided_q_and_bshd_out(ops, device):
    """q as a transposed view of a [B,S,H,D] buffer (what Attention produces); out written BSHD."""
    B, H, S, D = 2, 4, 128, 64
    q_bshd = rnd(B, S, H, D, seed=31).to(torch.bfloat16)
    _, k, v = attn_inputs(B, H, H, S, S, D, seed=32)
    qd = q_bshd.to(device).transpose(1, 2)
    assert not qd.is_contiguous()
    out, lse = ops.attn_fwd(qd, k.to(device), v.to(device), 0.125, True, bshd_out=True)
    assert out.transpose(1, 2).is_contiguous()
    w_o, w_l = OR.block_forward(q_bshd.transpose(1, 2).float(), k.float(), v.float(), 0.125, True)
    assert maxabs(out, w_o) <= 2e-2 and maxabs(lse, w_l) <= 1e-3


@pytest.mark.parametrize("D", [64, 128])
def test_attn_fwd_fused_merge_equals_ring(ops, device, D):
    """Rank r's ring via per-chunk launches with the fused merge == the oracle's rank_forward."""
    W, Sc, B, H = 4, 96, 1, 2
    q, k, v = attn_inputs(B, H, H, W * Sc, W * Sc, D, seed=40)
    scale = 1 / math.sqrt(D)
    ks, vs = k.chunk(W, 2), v.chunk(W, 2)
    for r in (0, 2, 3):
        q_r = q[:, :, r * Sc:(r + 1) * Sc].contiguous()
        out = torch.zeros(B, H, Sc, D, dtype=torch.float32, device=device)
        lse = torch.full((B, H, Sc), float("-inf"), dtype=torch.float32, device=device)
        for _, held, run, blk_causal in OR.schedule(W, r, True):
            if run:
                ops.attn_fwd(q_r.to(device), ks[held].contiguous().to(device), vs[held].contiguous().to(device), scale,
                             blk_causal, 0, out=out, lse=lse, merge=True)
        w_o, w_l = OR.rank_forward(q_r.float(), [t.float() for t in ks], [t.float() for t in vs], r, scale, True)
        assert maxabs(out, w_o) <= 2e-2 and maxabs(lse, w_l) <= 1e-3


# ------------------------------------------------------------------------------------ attention backward
BWD_CASES = [
    (1, 2, 2, 128, 128, 64, True, 0),
    (2, 2, 2, 256, 256, 64, True, 0),
    (1, 2, 2, 128, 256, 64, False, 0),
    (1, 2, 2, 128, 512, 64, True, 384),
    (1, 4, 2, 192, 192, 64, True, 0),
    (1, 2, 1, 77, 203, 64, False, 0),
    (1, 2, 2, 100, 100, 64, True, 0),
    (1, 2, 2, 256, 256, 128, True, 0),
    (1, 4, 2, 128, 384, 128, True, 256),
    (1, 1, 1, 61, 130, 128, False, 0),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,q_offset", BWD_CASES)
def test_attn_bwd(ops, device, B, Hq, Hkv, Sq, Sk, D, causal, q_offset):
    q, k, v = attn_inputs(B, Hq, Hkv, Sq, Sk, D, seed=50)
    do = rnd(B, Hq, Sq, D, seed=53).to(torch.bfloat16)
    scale = 1 / math.sqrt(D)
    qd, kd, vd, dod = (t.to(device) for t in (q, k, v, do))
    out, lse = ops.attn_fwd(qd, kd, vd, scale, causal, q_offset)
    delta = ops.attn_bwd_preprocess(dod, out)
    dq_acc, dk, dv = ops.attn_bwd(dod, qd, kd, vd, lse, delta, scale, causal, q_offset)
    # oracle: autograd through the fp32 closed form on the same bf16-rounded inputs
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    w_o, _ = OR.full_attention_closed_form(qf, expand_kv(kf, Hq), expand_kv(vf, Hq), scale, causal, q_offset)
    gq, gk, gv = torch.autograd.grad(w_o, (qf, kf, vf), do.float())
    assert maxabs(delta, (do.float() * w_o.detach()).sum(-1)) <= 5e-2
    assert rel_l2(dq_acc, gq) <= 1e-2
    assert rel_l2(dk, gk) <= 1e-2
    assert rel_l2(dv, gv) <= 1e-2


def test_attn_bwd_block_with_final_lse_and_accumulate(ops, device):
    """Ring backward of one rank: per-block launches that use the FINAL merged (out, lse), fp32 accumulation
    of dq across blocks and of dk/dv into existing buffers -- against the oracle's rank_backward."""
    W, Sc, B, H, D, r = 4, 64, 1, 2, 64, 2
    q, k, v = attn_inputs(B, H, H, W * Sc, W * Sc, D, seed=60)
    do = rnd(B, H, Sc, D, seed=63).to(torch.bfloat16)
    ks, vs = [t.contiguous() for t in k.chunk(W, 2)], [t.contiguous() for t in v.chunk(W, 2)]
    q_r = q[:, :, r * Sc:(r + 1) * Sc].contiguous()
    w_o, w_l = OR.rank_forward(q_r.float(), [t.float() for t in ks], [t.float() for t in vs], r, 0.125, True)
    w_dq, contrib = OR.rank_backward(do.float(), q_r.float(), [t.float() for t in ks], [t.float() for t in vs],
                                     w_o, w_l, r, 0.125, True)
    out_d, lse_d = w_o.to(torch.bfloat16).to(device), w_l.to(device)
    dq_acc = torch.empty(B, H, Sc, D, dtype=torch.float32, device=device)
    delta = ops.attn_bwd_preprocess(do.to(device), out_d, dq_acc)    # also zeroes dq_acc
    for _, held, run, blk_causal in OR.schedule(W, r, True):
        if not run:
            continue
        dk = torch.ones(B, H, Sc, D, dtype=torch.float32, device=device)   # pre-existing travelling accumulators
        dv = torch.full((B, H, Sc, D), 2.0, dtype=torch.float32, device=device)
        ops.attn_bwd(do.to(device), q_r.to(device), ks[held].to(device), vs[held].to(device), lse_d, delta, 0.125,
                     blk_causal, 0, dq_acc, dk, dv, dq_accumulate=True, dkv_accumulate=True)
        assert rel_l2(dk - 1.0, contrib[held][0]) <= 1e-2
        assert rel_l2(dv - 2.0, contrib[held][1]) <= 1e-2
    assert rel_l2(dq_acc, w_dq) <= 1e-2


def test_attn_bwd_bf16_strided_outputs_and_determinism(ops, device):
    """dq written as bf16 in q's [B,S,H,D] memory; two runs are bit-identical (no atomics in the backward)."""
    B, H, S, D = 2, 4, 192, 64
    q_bshd = rnd(B, S, H, D, seed=80).to(torch.bfloat16).to(device)
    qd = q_bshd.transpose(1, 2)
    _, k, v = attn_inputs(B, H, H, S, S, D, seed=81)
    do = rnd(B, H, S, D, seed=84).to(torch.bfloat16).to(device)
    kd, vd = k.to(device), v.to(device)
    out, lse = ops.attn_fwd(qd, kd, vd, 0.125, True)
    delta = ops.attn_bwd_preprocess(do, out)
    a = ops.attn_bwd(do, qd, kd, vd, lse, delta, 0.125, True, 0, dq_dtype=torch.bfloat16, dq_like=qd, dkv_dtype=torch.bfloat16)
    b = ops.attn_bwd(do, qd, kd, vd, lse, delta, 0.125, True, 0, dq_dtype=torch.bfloat16, dq_like=qd, dkv_dtype=torch.bfloat16)
    assert a[0].stride() == qd.stride() and a[0].dtype == torch.bfloat16
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    f = ops.attn_bwd(do, qd, kd, vd, lse, delta, 0.125, True, 0)
    for x, y in zip(a, f):
        assert rel_l2(x, y) <= 5e-3


def test_attn_bwd_side_stream_matches_one_stream(ops, device):
    """The dQ kernel on a second stream changes scheduling only: bit-identical gradients."""
    B, H, S, D = 2, 4, 320, 64
    q, k, v = (t.to(device) for t in attn_inputs(B, H, H, S, S, D, seed=86))
    do = rnd(B, H, S, D, seed=87).to(torch.bfloat16).to(device)
    out, lse = ops.attn_fwd(q, k, v, 0.125, True)
    delta = ops.attn_bwd_preprocess(do, out)
    one = ops.attn_bwd(do, q, k, v, lse, delta, 0.125, True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16)
    side = torch.cuda.Stream()
    for _ in range(3):
        two = ops.attn_bwd(do, q, k, v, lse, delta, 0.125, True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16,
                           side_stream=side)
        torch.cuda.synchronize()
        for x, y in zip(one, two):
            assert torch.equal(x, y)


def test_attn_bwd_paired_key_tiles_match_unpaired(ops, device):
    """A big causal launch lets each dK/dV workgroup take key tiles t and n-1-t; a launch of half the batch is too
    small for that and takes one tile per workgroup.  Same arithmetic per head, so the results are bit-identical --
    with an odd number of key tiles (the middle one has no partner) and a ragged last tile."""
    B, H, S, D = 8, 16, 1100, 64
    q, k, v = (t.to(device) for t in attn_inputs(B, H, H, S, S, D, seed=90))
    do = rnd(B, H, S, D, seed=91).to(torch.bfloat16).to(device)
    out, lse = ops.attn_fwd(q, k, v, 0.125, True)
    delta = ops.attn_bwd_preprocess(do, out)
    whole = ops.attn_bwd(do, q, k, v, lse, delta, 0.125, True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16)
    for half in (slice(0, 4), slice(4, 8)):
        part = ops.attn_bwd(do[half], q[half], k[half], v[half], lse[half].contiguous(), delta[half].contiguous(), 0.125,
                            True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16)
        for x, y in zip(whole, part):
            assert torch.equal(x[half], y)
    # and against the oracle on one head of it
    qf, kf, vf = (t[:1, :1].float().cpu().requires_grad_() for t in (q, k, v))
    w_o, _ = OR.full_attention_closed_form(qf, kf, vf, 0.125, True, 0)
    gq, gk, gv = torch.autograd.grad(w_o, (qf, kf, vf), do[:1, :1].float().cpu())
    assert rel_l2(whole[1][:1, :1], gk) <= 1e-2 and rel_l2(whole[2][:1, :1], gv) <= 1e-2 and rel_l2(whole[0][:1, :1], gq) <= 1e-2


def test_attn_bwd_head_dim_128_wave_pairs(ops, device):
    """head_dim 128: two waves share a 32-key block of the dK/dV kernel, take one 32-query sub-block each and add their
    partial dK / dV through LDS at the end of a key tile.  Two runs are bit-identical; a launch big enough for paired key
    tiles (t and n-1-t in one workgroup; odd tile count, ragged last tile) equals the launches of half the batch, which
    take one tile per workgroup; fp32 outputs with accumulate add to what is there; one head against the oracle."""
    B, H, S, D = 4, 16, 1100, 128
    scale = 1 / math.sqrt(D)
    q, k, v = (t.to(device) for t in attn_inputs(B, H, H, S, S, D, seed=95))
    do = rnd(B, H, S, D, seed=96).to(torch.bfloat16).to(device)
    out, lse = ops.attn_fwd(q, k, v, scale, True)
    delta = ops.attn_bwd_preprocess(do, out)
    whole = ops.attn_bwd(do, q, k, v, lse, delta, scale, True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16)
    again = ops.attn_bwd(do, q, k, v, lse, delta, scale, True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16)
    for x, y in zip(whole, again):
        assert torch.equal(x, y)
    for half in (slice(0, 2), slice(2, 4)):
        part = ops.attn_bwd(do[half], q[half], k[half], v[half], lse[half].contiguous(), delta[half].contiguous(), scale,
                            True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16)
        for x, y in zip(whole, part):
            assert torch.equal(x[half], y)
    # fp32 dk / dv added to what the buffers hold
    dk = torch.full((B, H, S, D), 2.0, dtype=torch.float32, device=device)
    dv = torch.full((B, H, S, D), -1.0, dtype=torch.float32, device=device)
    ops.attn_bwd(do, q, k, v, lse, delta, scale, True, 0, None, dk, dv, want_dq=False, dkv_accumulate=True)
    plain = ops.attn_bwd(do, q, k, v, lse, delta, scale, True, 0, want_dq=False)
    assert (dk - 2.0 - plain[1]).abs().max().item() <= 1e-5 * plain[1].abs().max().item() + 1e-6
    assert (dv + 1.0 - plain[2]).abs().max().item() <= 1e-5 * plain[2].abs().max().item() + 1e-6
    qf, kf, vf = (t[:1, :1].float().cpu().requires_grad_() for t in (q, k, v))
    w_o, _ = OR.full_attention_closed_form(qf, kf, vf, scale, True, 0)
    gq, gk, gv = torch.autograd.grad(w_o, (qf, kf, vf), do[:1, :1].float().cpu())
    assert rel_l2(whole[1][:1, :1], gk) <= 1e-2 and rel_l2(whole[2][:1, :1], gv) <= 1e-2 and rel_l2(whole[0][:1, :1], gq) <= 1e-2


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,q_offset", [
    (2, 4, 4, 300, 300, 64, True, 0), (1, 4, 2, 128, 384, 128, True, 256), (1, 2, 1, 77, 203, 64, False, 0)])
def test_attn_bwd_with_delta_computed_inside(ops, device, B, Hq, Hkv, Sq, Sk, D, causal, q_offset):
    """attn_bwd(out=...) computes delta = sum_d dO * O itself (in the dQ kernel's prologue for a bf16 out, through the
    pre-pass for an fp32 out or when dq is not wanted): same gradients as preprocess + attn_bwd, and delta is handed back."""
    q, k, v = (t.to(device) for t in attn_inputs(B, Hq, Hkv, Sq, Sk, D, seed=92))
    do = rnd(B, Hq, Sq, D, seed=93).to(torch.bfloat16).to(device)
    scale = 1 / math.sqrt(D)
    out, lse = ops.attn_fwd(q, k, v, scale, causal, q_offset)
    delta = ops.attn_bwd_preprocess(do, out)
    ref = ops.attn_bwd(do, q, k, v, lse, delta, scale, causal, q_offset)
    want = (do.float() * out.float()).sum(-1)
    for out_arg in (out, out.float()):
        d2 = torch.full_like(delta, float("nan"))
        got = ops.attn_bwd(do, q, k, v, lse, d2, scale, causal, q_offset, out=out_arg)
        assert maxabs(d2, want) <= 1e-3 * max(1.0, want.abs().max().item())
        for x, y in zip(got, ref):
            assert rel_l2(x, y) <= 1e-4
    # dq not wanted: the pre-pass supplies delta for the dK/dV kernel
    _, dk, dv = ops.attn_bwd(do, q, k, v, lse, None, scale, causal, q_offset, out=out, want_dq=False)
    assert rel_l2(dk, ref[1]) <= 1e-4 and rel_l2(dv, ref[2]) <= 1e-4


def test_attn_rejects_unsupported_layouts(ops, device):
    """Error behaviour of the boundary: gradient rows that are not 16-byte aligned raise, nothing is launched."""
    B, H, S, D = 1, 2, 64, 64
    q, k, v = (t.to(device) for t in attn_inputs(B, H, H, S, S, D, seed=88))
    do = rnd(B, H, S, D, seed=89).to(torch.bfloat16).to(device)
    out, lse = ops.attn_fwd(q, k, v, 0.125, True)
    delta = ops.attn_bwd_preprocess(do, out)
    # dk / dv rows 68 elements apart: not a multiple of 8
    pad = torch.empty(B, H, S, D + 4, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError, match="strides"):
        ops.attn_bwd(do, q, k, v, lse, delta, 0.125, True, 0, None, pad[..., :D], pad.clone()[..., :D], want_dq=False)


def test_attn_empty_inputs(ops, device):
    """No queries or no keys: nothing faults; gradients of the side that exists are zero."""
    z = torch.zeros(1, 2, 0, 64, dtype=torch.bfloat16, device=device)
    x = rnd(1, 2, 40, 64, seed=85).to(torch.bfloat16).to(device)
    out, lse = ops.attn_fwd(z, x, x, 0.125, False)
    assert out.shape == (1, 2, 0, 64)
    out, lse = ops.attn_fwd(x, z, z, 0.125, False)
    assert out.abs().max().item() == 0.0 and torch.isinf(lse).all()
    delta = ops.attn_bwd_preprocess(x, out)
    dq, dk, dv = ops.attn_bwd(x, x, z, z, lse, delta, 0.125, False, 0)
    assert dq.abs().max().item() == 0.0 and dk.shape == (1, 2, 0, 64)


def test_convert_f32(ops, device):
    src = rnd(2, 3, 5, 64, seed=70).to(device)
    like = torch.empty(2, 5, 3, 64, dtype=torch.bfloat16, device=device).transpose(1, 2)
    dst = ops.convert_f32(src, torch.bfloat16, like=like)
    assert dst.stride() == like.stride() and torch.equal(dst, src.to(torch.bfloat16))
    assert torch.equal(ops.convert_f32(src, torch.float32), src)


def test_cpu_tensor_is_rejected(ops):
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.swiglu_fwd(torch.zeros(2, 8), torch.zeros(2, 8))


def test_bad_head_dim_reports_error(ops, device):
    q = torch.zeros(1, 1, 8, 32, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError, match="head_dim"):
        ops.attn_fwd(q, q, q, 1.0, True)


@pytest.mark.parametrize("n,grad_dtype", [(8 * 1024 + 3, torch.bfloat16), (4096, torch.float32), (5, torch.bfloat16)])
def test_adamw_kernel_against_oracle(ops, device, n, grad_dtype):
    """pico_adamw over four steps against oracle.optim.master_step: fp32 states to a few ulp, the bf16 parameter is the
    rounded master weight."""
    from oracle import optim as OO
    g = torch.Generator().manual_seed(11)
    master = torch.randn(n, generator=g)
    m, v = torch.zeros(n), torch.zeros(n)
    d_master, d_m, d_v = master.to(device), m.to(device), v.to(device)
    d_p = torch.empty(n, dtype=torch.bfloat16, device=device)
    for step in range(1, 5):
        grad = (torch.randn(n, generator=g) * 0.05 * step).to(grad_dtype)
        ops.adamw_(d_p, d_master, grad.to(device), d_m, d_v, step, 2e-3, 0.9, 0.95, 1e-8, 0.1)
        master, m, v, p_lp = OO.master_step(master, grad, m, v, step, 2e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
        assert maxabs(d_master, master) <= 2e-6 * max(1.0, master.abs().max().item())
        assert maxabs(d_m, m) <= 1e-6 and maxabs(d_v, v) <= 1e-6
        assert torch.equal(d_p.cpu(), d_master.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("n,grad_dtype", [(8 * 1024 + 3, torch.bfloat16), (4096, torch.float32), (5, torch.bfloat16)])
@pytest.mark.parametrize("moment_dtype", [torch.bfloat16, torch.float32])
def test_adamw_lp_kernel_against_oracle(ops, device, n, grad_dtype, moment_dtype):
    """pico_adamw_lp (bf16 parameter updated in place, bf16 or fp32 moments) over four steps against
    oracle.optim.lp_step fed the kernel's own previous state: both compute in fp32 and round once, so almost every
    element is identical and the rest are one rounding step apart (the compiler may contract a multiply-add that the
    oracle rounds twice); fp32 moments agree to a few ulp."""
    from oracle import optim as OO
    g = torch.Generator().manual_seed(13)
    p = torch.randn(n, generator=g).bfloat16()
    d_p, d_m, d_v = p.to(device), torch.zeros(n, dtype=moment_dtype, device=device), torch.zeros(n, dtype=moment_dtype, device=device)
    for step in range(1, 5):
        grad = (torch.randn(n, generator=g) * 0.05 * step).to(grad_dtype)
        want = OO.lp_step(d_p.cpu(), grad, d_m.cpu(), d_v.cpu(), step, 2e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
        ops.adamw_lp_(d_p, grad.to(device), d_m, d_v, step, 2e-3, 0.9, 0.95, 1e-8, 0.1)
        for got, w in zip((d_p, d_m, d_v), want):
            assert got.dtype == w.dtype
            diff = (got.cpu().float() - w.float()).abs()
            if w.dtype == torch.float32:
                assert (diff <= 1e-6 * w.abs().max().clamp_min(1e-3)).all()
                continue
            assert (diff <= w.float().abs() * 2.0 ** -7 + w.float().abs().mean() * 2.0 ** -14).all()
            assert (diff != 0).sum().item() <= max(1, 0.03 * n)


@pytest.mark.parametrize("state_dtype,moment_dtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                                      (torch.float32, torch.float32)])
def test_adamw_multi_equals_one_call_per_tensor(ops, device, state_dtype, moment_dtype):
    """pico_adamw_multi over 61 tensors (more than one launch's table holds; sizes 0, 1, odd and many blocks) leaves
    every state bit-identical to pico_adamw / pico_adamw_lp called once per tensor."""
    g = torch.Generator().manual_seed(17)
    sizes = [0, 1, 5, 2048, 2049, 40000] + [int(x) for x in torch.randint(1, 30000, (55,), generator=g)]
    lp = state_dtype == torch.bfloat16
    def fresh():
        gg = torch.Generator().manual_seed(18)
        mk = lambda n, dt=state_dtype, pos=False: (torch.rand(n, generator=gg) if pos else torch.randn(n, generator=gg)).to(dt).to(device)
        return ([mk(n) for n in sizes], [mk(n, moment_dtype) for n in sizes], [mk(n, moment_dtype, True) for n in sizes],
                [torch.randn(n, generator=gg).bfloat16().to(device) for n in sizes])
    w1, m1, v1, gr = fresh()
    w2, m2, v2, _ = fresh()
    lp1 = None if lp else [torch.empty(n, dtype=torch.bfloat16, device=device) if i % 3 else None for i, n in enumerate(sizes)]
    lp2 = None if lp else [torch.empty(n, dtype=torch.bfloat16, device=device) if i % 3 else None for i, n in enumerate(sizes)]
    hyper = (3, 2e-3, 0.9, 0.95, 1e-8, 0.1, 0.5)
    ops.adamw_multi_(w1, gr, m1, v1, *hyper, param_lps=lp1)
    for i in range(len(sizes)):
        if lp:
            ops.adamw_lp_(w2[i], gr[i], m2[i], v2[i], *hyper)
        else:
            ops.adamw_(lp2[i], w2[i], gr[i], m2[i], v2[i], *hyper)
    for i in range(len(sizes)):
        assert torch.equal(w1[i], w2[i]) and torch.equal(m1[i], m2[i]) and torch.equal(v1[i], v2[i]), sizes[i]
        if not lp and lp1[i] is not None:
            assert torch.equal(lp1[i], lp2[i])
    with pytest.raises(RuntimeError, match="one entry per tensor"):
        ops.adamw_multi_(w1, gr[:-1], m1, v1, *hyper)


def test_fused_adamw_with_fp32_moments_and_no_master_copy(device):
    """FusedAdamW(master_weights=False, state_dtype=fp32): bf16 parameters updated in place, fp32 moments.  The moments
    follow torch.optim.AdamW run on fp32 copies fed the same gradients (they do not depend on the weights) to fp32
    accuracy; the parameters follow it to bf16 rounding accumulated over the steps."""
    from picotron_amd.optim import FusedAdamW
    torch.manual_seed(9)
    ps = [torch.nn.Parameter(torch.randn(33, 20, device=device).to(torch.bfloat16)), torch.nn.Parameter(torch.randn(7, device=device).to(torch.bfloat16))]
    ref = [torch.nn.Parameter(p.detach().float().clone()) for p in ps]
    opt = FusedAdamW(ps, lr=1e-2, weight_decay=0.02, master_weights=False, state_dtype=torch.float32)
    ropt = torch.optim.AdamW(ref, lr=1e-2, weight_decay=0.02)
    assert opt.master is None and opt.exp_avg.dtype == torch.float32
    for _ in range(3):
        for p, r in zip(ps, ref):
            p.grad = torch.randn_like(p)
            r.grad = p.grad.float()
        opt.step()
        ropt.step()
    for p, r, off in zip(ps, ref, opt.offsets):
        n = p.numel()
        st = ropt.state[r]
        assert maxabs(opt.exp_avg[off:off + n].view_as(p), st["exp_avg"]) <= 1e-6
        assert maxabs(opt.exp_avg_sq[off:off + n].view_as(p), st["exp_avg_sq"]) <= 1e-6
        assert maxabs(p.detach().float(), r.detach()) <= 3 * 2 ** -8 * r.detach().abs().max().item()


def test_fused_adamw_without_master_weights_follows_torch_fused_adamw(device):
    """FusedAdamW(master_weights=False) keeps the reference's state layout (train.py:209: AdamW on the bf16
    parameters); torch.optim.AdamW(fused=True) on bf16 copies, fed the same gradients, computes the same way (fp32
    arithmetic, one rounding per state), so parameters and moments agree to a rounding step after three steps."""
    from picotron_amd.optim import FusedAdamW
    torch.manual_seed(5)
    ps = [torch.nn.Parameter(torch.randn(33, 20, device=device).to(torch.bfloat16)), torch.nn.Parameter(torch.randn(7, device=device).to(torch.bfloat16))]
    ref = [torch.nn.Parameter(p.detach().clone()) for p in ps]
    opt = FusedAdamW(ps, lr=1e-2, weight_decay=0.02, master_weights=False)
    ropt = torch.optim.AdamW(ref, lr=1e-2, weight_decay=0.02, fused=True)
    assert opt.master is None and opt.exp_avg.dtype == torch.bfloat16
    for _ in range(3):
        for p, r in zip(ps, ref):
            p.grad = torch.randn_like(p)
            r.grad = p.grad.clone()
        opt.step()
        ropt.step()
    for p, r, off in zip(ps, ref, opt.offsets):
        n = p.numel()
        st = ropt.state[r]
        for got, w in ((p.detach(), r.detach()), (opt.exp_avg[off:off + n].view_as(p), st["exp_avg"]),
                       (opt.exp_avg_sq[off:off + n].view_as(p), st["exp_avg_sq"])):
            diff = (got.float() - w.float()).abs()
            assert (diff <= w.float().abs() * 2.0 ** -7 + w.float().abs().mean() * 2.0 ** -7).all()
            assert (diff != 0).sum().item() <= max(1, 0.05 * n)


def test_fused_adamw_trains_like_torch_adamw_on_master_weights(device):
    """picotron_amd.optim.FusedAdamW on bf16 parameters follows torch.optim.AdamW run on fp32 copies fed the same
    bf16 gradients."""
    from picotron_amd.optim import FusedAdamW
    torch.manual_seed(3)
    ps = [torch.nn.Parameter(torch.randn(33, 20, device=device).to(torch.bfloat16)), torch.nn.Parameter(torch.randn(7, device=device).to(torch.bfloat16))]
    ref = [torch.nn.Parameter(p.detach().float().clone()) for p in ps]
    opt, ropt = FusedAdamW(ps, lr=1e-2, weight_decay=0.02), torch.optim.AdamW(ref, lr=1e-2, weight_decay=0.02)
    for _ in range(3):
        for p, r in zip(ps, ref):
            p.grad = torch.randn_like(p)
            r.grad = p.grad.float()
        opt.step()
        ropt.step()
    for p, r, off in zip(ps, ref, opt.offsets):
        mine = opt.master[off:off + p.numel()].view_as(r)
        assert maxabs(mine, r.detach()) <= 1e-5
        assert torch.equal(p.detach().cpu(), mine.to(torch.bfloat16).cpu())
        assert maxabs(p.detach().float(), r.detach()) <= 2 ** -8 * r.detach().abs().max().item()


@pytest.mark.parametrize("rows,vocab,dtype", [(64, 49152, torch.bfloat16), (33, 1000, torch.bfloat16), (17, 515, torch.float32)])
def test_cross_entropy_against_oracle(ops, device, rows, vocab, dtype):
    """pico_cross_entropy_fwd / _bwd through the autograd function against the oracle: loss and lse to fp32 accuracy on
    the same (rounded) logits, dlogits to the rounding of their dtype; ignored rows give no loss and no gradient."""
    from oracle import layers as OL
    from picotron_amd.functional import cross_entropy
    g = torch.Generator().manual_seed(21)
    x = (torch.randn(rows, vocab, generator=g) * 4).to(dtype)
    t = torch.randint(0, vocab, (rows,), generator=g)
    t[1] = -100
    pitch = (vocab + 7) // 8 * 8   # rows start 16-byte aligned; the kernel's tail path covers vocab % vector != 0
    xd = torch.zeros(rows, pitch, dtype=dtype, device=device)[:, :vocab].copy_(x.to(device)).requires_grad_()
    loss = cross_entropy(xd, t.to(device))
    (loss * 0.5).backward()
    want, want_lse = OL.cross_entropy(x, t)
    assert abs(loss.item() - want.item()) <= 2e-5 * max(1.0, abs(want.item()))
    _, lse = ops.cross_entropy_fwd(xd.detach(), t.to(device))
    assert maxabs(lse, want_lse) <= 2e-5 * want_lse.abs().max().item()
    gw = OL.cross_entropy_backward(x, t, 0.5)
    tol = 2 ** -8 if dtype == torch.bfloat16 else 1e-6
    assert maxabs(xd.grad, gw) <= tol * gw.abs().max().item() + 1e-9
    assert xd.grad[1].abs().max().item() == 0.0


def test_cross_entropy_target_out_of_range_is_skipped_not_read(ops, device):
    """A target outside [0, vocab) that is not ignore_index (a pad id, a -100 with another ignore_index) must never be
    used as an index: the row counts as ignored in both directions, and the mean is over the rows that count."""
    from oracle import layers as OL
    from picotron_amd.functional import cross_entropy
    g = torch.Generator().manual_seed(4)
    rows, vocab = 12, 515
    x = (torch.randn(rows, vocab, generator=g) * 3).to(torch.bfloat16)
    t = torch.randint(0, vocab, (rows,), generator=g)
    bad = {0: -5, 3: vocab, 7: vocab + (1 << 40), 9: -100}
    for r, val in bad.items():
        t[r] = val
    pitch = (vocab + 7) // 8 * 8
    xd = torch.zeros(rows, pitch, dtype=torch.bfloat16, device=device)[:, :vocab].copy_(x.to(device)).requires_grad_()
    loss = cross_entropy(xd, t.to(device), ignore_index=-1)      # -100 is NOT the ignore index here
    loss.backward()
    loss_rows, _ = ops.cross_entropy_fwd(xd.detach(), t.to(device), -1)
    keep = torch.tensor([r not in bad for r in range(rows)])
    want, _ = OL.cross_entropy(x[keep], t[keep])
    assert abs(loss.item() - want.item()) <= 2e-5 * max(1.0, abs(want.item()))
    for r in bad:
        assert loss_rows[r].item() == 0.0 and xd.grad[r].abs().max().item() == 0.0
    gw = OL.cross_entropy_backward(x[keep], t[keep], 1.0)
    assert maxabs(xd.grad[keep.to(device)], gw) <= 2 ** -8 * gw.abs().max().item() + 1e-9
    # and with the opt-in host check the same input is an error, as it is for F.cross_entropy (train.py:46-49)
    import os
    os.environ["PICO_CHECK_TARGETS"] = "1"
    try:
        with pytest.raises(RuntimeError, match="outside"):
            cross_entropy(xd, t.to(device), -1)
    finally:
        os.environ.pop("PICO_CHECK_TARGETS", None)


def test_fused_adamw_overlapped_with_backward_gives_the_same_update(device):
    """overlap_with_backward updates each parameter from a hook on a second stream; same numbers as step()."""
    from picotron_amd.optim import FusedAdamW
    results = []
    for overlap in (False, True):
        torch.manual_seed(5)
        lin1 = torch.nn.Linear(64, 48, bias=False).to(device).to(torch.bfloat16)
        lin2 = torch.nn.Linear(48, 8, bias=False).to(device).to(torch.bfloat16)
        params = list(lin1.parameters()) + list(lin2.parameters())
        opt = FusedAdamW(params, lr=1e-2, overlap_with_backward=overlap)
        x = torch.randn(16, 64, device=device).to(torch.bfloat16)
        for _ in range(3):
            opt.zero_grad()
            lin2(torch.tanh(lin1(x))).float().square().mean().backward()
            opt.step()
        torch.cuda.synchronize()
        results.append([p.detach().float().cpu() for p in params] + [opt.master.cpu()])
    for a, b in zip(*results):
        assert torch.equal(a, b)


def test_empty_inputs_are_no_ops(ops, device):
    """Zero batch, zero queries, zero rows, zero parameters: every entry returns without touching memory."""
    bf = torch.bfloat16
    q = torch.zeros(0, 2, 16, 64, dtype=bf, device=device)
    out, lse = ops.attn_fwd(q, q, q, 0.125, True)
    assert out.shape == (0, 2, 16, 64) and lse.shape == (0, 2, 16)
    q0 = torch.zeros(1, 2, 0, 64, dtype=bf, device=device)
    kv = torch.randn(1, 2, 16, 64, device=device).to(bf)
    out, lse = ops.attn_fwd(q0, kv, kv, 0.125, False)
    assert out.numel() == 0 and lse.numel() == 0
    dq, dk, dv = ops.attn_bwd(q0, q0, kv, kv, lse, lse.clone(), 0.125, False, 0, dq_dtype=bf, dkv_dtype=bf)
    assert dq.numel() == 0 and dk.abs().max().item() == 0.0 and dv.abs().max().item() == 0.0   # no query: zero gradients
    cos, sin = OL.get_cos_sin(8, 64, 10000.0)
    assert ops.rope(torch.zeros(1, 2, 0, 64, dtype=bf, device=device), cos.to(device), sin.to(device)).numel() == 0
    logits = torch.zeros(0, 64, dtype=bf, device=device)
    loss_rows, lse_rows = ops.cross_entropy_fwd(logits, torch.zeros(0, dtype=torch.int64, device=device))
    assert loss_rows.numel() == 0 and lse_rows.numel() == 0
    e = torch.zeros(0, dtype=bf, device=device)
    ops.adamw_lp_(e, e, e.clone(), e.clone(), 1, 1e-3)
    ops.adamw_multi_([e], [e], [e.clone()], [e.clone()], 1, 1e-3)
    torch.cuda.synchronize()


# ------------------------------------------------------------------------------------ RoPE inside attention
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,q_offset,pos0", [
    (2, 4, 4, 256, 256, 64, 0, 0),        # MHA, one chunk, positions from 0
    (1, 8, 2, 200, 200, 64, 0, 37),       # GQA, ragged length, positions from 37
    (1, 4, 2, 192, 192, 128, 0, 5),       # head_dim 128
    (1, 4, 4, 128, 384, 64, 256, 1024),   # a query chunk behind two earlier key chunks (offset diagonal)
    (2, 2, 1, 33, 97, 128, 64, 0),        # odd sizes
])
@pytest.mark.parametrize("table_dtype", [torch.bfloat16, torch.float32])
def test_attention_with_rope_inside_vs_oracle(ops, device, B, Hq, Hkv, Sq, Sk, D, q_offset, pos0, table_dtype):
    """pico_attn_fwd_rope / pico_attn_bwd_rope: q rotated in the forward's prologue, dq / dk un-rotated in the backward's
    epilogues, k rotated by pico_rope -- against the oracle's apply_rotary_pos_emb + attention differentiated by
    autograd in fp32.  Positions: key j sits at pos0 + j, query i at pos0 + q_offset + i."""
    from oracle import layers as OL
    from oracle import ring as OR
    g = torch.Generator().manual_seed(100 + Sq + D)
    q = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, Sk, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, Sk, D, generator=g).to(torch.bfloat16)
    do = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(D)
    cos, sin = OL.get_cos_sin(pos0 + Sk + 3, D, 10000.0, table_dtype)
    # oracle, fp32, on the same bf16 inputs and the same (possibly bf16-rounded) tables
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    cq, sq_ = cos[pos0 + q_offset:pos0 + q_offset + Sq].float(), sin[pos0 + q_offset:pos0 + q_offset + Sq].float()
    ck, sk_ = cos[pos0:pos0 + Sk].float(), sin[pos0:pos0 + Sk].float()
    q_r = OL.apply_rotary_pos_emb(qf, cq, sq_)
    k_r = OL.apply_rotary_pos_emb(kf, ck, sk_)
    # the reference hands bf16 tensors from the rotation to the attention (model.py:136-137): round the rotated
    # operands the same way, with the gradient passed straight through the rounding
    q_r = q_r + (q_r.detach().to(torch.bfloat16).float() - q_r.detach())
    k_r = k_r + (k_r.detach().to(torch.bfloat16).float() - k_r.detach())
    rep = Hq // Hkv
    w_o, w_l = OR.full_attention_closed_form(q_r, k_r.repeat_interleave(rep, 1), vf.repeat_interleave(rep, 1), scale, True, q_offset)
    gq, gk, gv = torch.autograd.grad(w_o, (qf, kf, vf), do.float())

    cd, sd = cos.to(device), sin.to(device)
    qd, kd, vd, dod = (t.to(device) for t in (q, k, v, do))
    k_rot = ops.rope(kd, cd, sd, pos_offset=pos0)
    out, lse, q_rot = ops.attn_fwd_rope(qd, k_rot, vd, cd, sd, scale, True, q_offset, q_pos_offset=pos0 + q_offset)
    assert maxabs(q_rot, q_r.detach()) <= 3e-2
    assert torch.allclose(q_rot.float(), ops.rope(qd, cd, sd, pos_offset=pos0 + q_offset).float(), rtol=2 ** -7, atol=1e-3)
    # lse to 2e-3 here, 1e-3 elsewhere: the kernel's rotated q may differ from the oracle's rounded rotation by one bf16
    # ulp in single elements (fp32 products summed in another order before the one rounding); one ulp of an element in
    # [2, 4) is 2^-6, times |k| ~ 1, times sm_scale = 1/8 moves one score -- and a row's lse by at most as much -- by
    # 2e-3.  The last assertion of this test holds the same kernel, given that rotated q, bit-equal to pico_attn_fwd,
    # which is held to 1e-3.
    assert maxabs(out, w_o.detach()) <= 2e-2 and maxabs(lse, w_l.detach()) <= 2e-3
    dq = torch.empty(B, Sq, Hq, D, dtype=torch.bfloat16, device=device).transpose(1, 2)
    dk = torch.empty(B, Sk, Hkv, D, dtype=torch.bfloat16, device=device).transpose(1, 2)
    dv = torch.empty_like(dk)
    ops.attn_bwd_rope(dod, q_rot, k_rot, vd, out, lse, cd, sd, scale, True, dq, dk, dv, q_offset,
                      q_pos_offset=pos0 + q_offset, k_pos_offset=pos0)
    assert rel_l2(dq, gq) <= 1e-2 and rel_l2(dk, gk) <= 1e-2 and rel_l2(dv, gv) <= 1e-2
    # and the same numbers as the separate-launch path, up to the rounding the fused path does not do twice
    o2, l2 = ops.attn_fwd(q_rot, k_rot, vd, scale, True, q_offset)
    assert torch.equal(o2, out) and torch.equal(l2, lse)
