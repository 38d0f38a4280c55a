"""GPU parity at the shapes BASELINE.json names (configs[1], [3], [4]) -- against the CPU oracle where it
finishes in seconds, and through size-independent properties plus an fp32 torch reference on a slice of the
heads where it does not."""
import math

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


@pytest.fixture(scope="module")
def ops(device):
    from picotron_amd import ops as _ops
    return _ops


def ref_attention_fp32(q, k, v, scale, q_offset, do=None):
    """fp32 torch reference on the GPU for a slice of heads: softmax(QK^T*s + offset-causal mask) V (+ autograd)."""
    q, k, v = (t.float().detach().requires_grad_(do is not None) for t in (q, k, v))
    rep = q.size(1) // k.size(1)
    s = (q @ k.repeat_interleave(rep, 1).transpose(-1, -2)) * scale
    qi = torch.arange(q.size(2), device=q.device)[:, None] + q_offset
    kj = torch.arange(k.size(2), device=q.device)[None, :]
    s = s.masked_fill(kj > qi, float("-inf"))
    out = torch.softmax(s, -1) @ v.repeat_interleave(rep, 1)
    lse = torch.logsumexp(s, -1)
    if do is None:
        return out, lse
    gq, gk, gv = torch.autograd.grad(out, (q, k, v), do.float())
    return out.detach(), lse.detach(), gq, gk, gv


def test_configs1_ring_all_ranks_full_shape_vs_cpu_oracle(ops, device):
    """configs[1] exactly: B4 H32 S1024 D64, cp 4, seed 0, q scaled by 1/sqrt(D); every rank's ring on the GPU
    (one fused launch per rank and, separately, one launch per ring step) against the CPU oracle's ring."""
    B, H, S, D, W = 4, 32, 1024, 64, 4
    Sc, scale = S // W, 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(0)
    q = (torch.randn(B, H, S, D, generator=g) * scale).to(torch.bfloat16)
    k, v, do = (torch.randn(B, H, S, D, generator=g).to(torch.bfloat16) for _ in range(3))
    w_o, w_l = OR.all_ranks_forward(q.float(), k.float(), v.float(), W, scale, True)
    w_dq, w_dk, w_dv = OR.all_ranks_backward(do.float(), q.float(), k.float(), v.float(), w_o, w_l, W, scale, True)
    qd, kd, vd, dod = (t.to(device) for t in (q, k, v, do))
    dk = torch.zeros(B, H, S, D, dtype=torch.float32, device=device)
    dv = torch.zeros_like(dk)
    for r in range(W):
        qs, ks = slice(r * Sc, (r + 1) * Sc), slice(0, (r + 1) * Sc)
        out, lse = ops.attn_fwd(qd[:, :, qs], kd[:, :, ks], vd[:, :, ks], scale, True, r * Sc)
        # the same rank as one launch per ring step with the fused merge
        o32 = torch.empty(B, H, Sc, D, dtype=torch.float32, device=device)
        l32 = torch.empty(B, H, Sc, dtype=torch.float32, device=device)
        for step, held, run, blk_causal in OR.schedule(W, r, True):
            if run:
                cs = slice(held * Sc, (held + 1) * Sc)
                ops.attn_fwd(qd[:, :, qs], kd[:, :, cs], vd[:, :, cs], scale, blk_causal, 0, out=o32, lse=l32, merge=step > 0)
        assert maxabs(out, w_o[:, :, qs]) <= 2e-2 and maxabs(lse, w_l[:, :, qs]) <= 1e-3
        assert maxabs(o32, w_o[:, :, qs]) <= 2e-2 and maxabs(l32, w_l[:, :, qs]) <= 1e-3
        delta = ops.attn_bwd_preprocess(dod[:, :, qs], out)
        dq, _, _ = ops.attn_bwd(dod[:, :, qs], qd[:, :, qs], kd[:, :, ks], vd[:, :, ks], lse, delta, scale, True, r * Sc,
                                None, dk[:, :, ks], dv[:, :, ks], dkv_accumulate=True)
        assert rel_l2(dq, w_dq[:, :, qs]) <= 1e-2
    assert rel_l2(dk, w_dk) <= 1e-2 and rel_l2(dv, w_dv) <= 1e-2


def test_configs3_llama2_7b_attention_shape(ops, device):
    """configs[3]'s attention: MHA, head_dim 128, S 4096, B 1 -- all 32 heads run; 4 of them are checked against
    the CPU oracle (forward and backward), the rest against those through head-permutation invariance."""
    H, S, D = 32, 4096, 128
    scale = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(1)
    q, k, v, do = (torch.randn(1, 4, S, D, generator=g).to(torch.bfloat16) for _ in range(4))
    # heads 0..3 are distinct, the other 28 repeat them: equal heads must give equal results
    idx = torch.arange(H) % 4
    qd, kd, vd, dod = (t[:, idx].contiguous().to(device) for t in (q, k, v, do))
    out, lse = ops.attn_fwd(qd, kd, vd, scale, True)
    delta = ops.attn_bwd_preprocess(dod, out)
    dq, dk, dv = ops.attn_bwd(dod, qd, kd, vd, lse, delta, scale, True, 0, dq_dtype=torch.bfloat16, dkv_dtype=torch.bfloat16)
    for t in (out, lse, dq, dk, dv):
        assert torch.equal(t[:, 4:8], t[:, 0:4]) and torch.equal(t[:, 28:32], t[:, 0:4])
    w_o, w_l = OR.block_forward(q.float(), k.float(), v.float(), scale, True)
    w_dq, w_dk, w_dv = OR.block_backward(do.float(), q.float(), k.float(), v.float(), w_o, w_l, scale, True)
    assert maxabs(out[:, :4], w_o) <= 2e-2 and maxabs(lse[:, :4], w_l) <= 1e-3
    assert rel_l2(dq[:, :4], w_dq) <= 1e-2 and rel_l2(dk[:, :4], w_dk) <= 1e-2 and rel_l2(dv[:, :4], w_dv) <= 1e-2


@pytest.mark.parametrize("Sq,Sk,q_offset,Hkv", [(2100, 2100, 0, 32), (1790, 2081, 291, 8), (2049, 4100, 2051, 8)])
def test_head_dim_128_large_launch_ragged_lengths(ops, device, Sq, Sk, q_offset, Hkv):
    """head_dim 128 with enough workgroups for the large-launch kernels (128-key staged tiles in the forward), at
    lengths that are multiples of neither the query tile nor the key tile, with the causal diagonal shifted and GQA:
    forward and backward against an fp32 torch reference on a slice of the heads (first and last kv head)."""
    Hq, D = 32, 128
    scale = 1 / math.sqrt(D)
    g = torch.Generator(device="cpu").manual_seed(5)
    q = (torch.randn(1, Hq, Sq, D, generator=g)).to(torch.bfloat16).to(device)
    k = torch.randn(1, Hkv, Sk, D, generator=g).to(torch.bfloat16).to(device)
    v = torch.randn(1, Hkv, Sk, D, generator=g).to(torch.bfloat16).to(device)
    do = torch.randn(1, Hq, Sq, D, generator=g).to(torch.bfloat16).to(device)
    out, lse = ops.attn_fwd(q, k, v, scale, True, q_offset)
    dq, dk, dv = ops.attn_bwd(do, q, k, v, lse, None, scale, True, q_offset, dq_dtype=torch.bfloat16,
                              dkv_dtype=torch.bfloat16, out=out)
    rep = Hq // Hkv
    for kvh in (0, Hkv - 1):
        qs = slice(kvh * rep, (kvh + 1) * rep)
        r_o, r_l, r_dq, r_dk, r_dv = ref_attention_fp32(q[:, qs], k[:, kvh:kvh + 1], v[:, kvh:kvh + 1], scale, q_offset, do[:, qs])
        assert maxabs(out[:, qs], r_o) <= 2e-2 and maxabs(lse[:, qs], r_l) <= 1e-3
        assert rel_l2(dq[:, qs], r_dq) <= 1e-2
        assert rel_l2(dk[:, kvh:kvh + 1], r_dk) <= 1e-2 and rel_l2(dv[:, kvh:kvh + 1], r_dv) <= 1e-2
    # keys that no query may see get exactly zero gradient
    last_visible = q_offset + Sq - 1
    if last_visible + 1 < Sk:
        assert dk[:, :, last_visible + 1:].abs().max().item() == 0.0 and dv[:, :, last_visible + 1:].abs().max().item() == 0.0


@pytest.mark.parametrize("B,Hkv,Sq,Sk,q_offset,causal", [
    (4, 32, 1024, 1024, 0, True),      # configs[1] with the four ranks in one launch: the 8-wave kernels
    (4, 8, 1000, 1000, 0, True),       # 8-wave kernels, ragged, GQA
    (4, 8, 777, 1203, 0, False),       # 8-wave kernels, dense, rectangular
    (2, 32, 1024, 1024, 0, True),      # half the batch: the 4-wave kernels without key split
    (2, 8, 1000, 1290, 290, True),     # 4-wave kernels, ragged, shifted diagonal, GQA
    (1, 8, 1000, 1290, 290, True),     # key-split kernels (four waves per workgroup) on the same lengths
    (1, 8, 500, 800, 300, True),       # key-split kernels, fewer workgroups still
    (4, 32, 256, 1024, 768, True),     # rank 3 of 4 at configs[1]: rectangular, key split with eight waves per workgroup
    (4, 32, 256, 256, 0, True),        # rank 0 of 4: key split, four waves (few keys, not rectangular)
    (1, 8, 1024, 700, 0, False),       # dense: key split, eight waves
    (8, 32, 256, 1024, 768, True),     # rectangular with 256 workgroups of 256 queries: the 8-wave kernels
    (8, 32, 700, 700, 0, True),        # several generations of short tiles: 8-wave forward, 4-wave dQ
])
def test_head_dim_64_every_launch_size_class(ops, device, B, Hkv, Sq, Sk, q_offset, causal):
    """head_dim 64 at 32 query heads: the library picks 8-wave, 4-wave or key-split workgroups (of eight or four waves) by
    the number of workgroups a launch has and the keys a query sees; each class is run here at full and at ragged lengths (forward and backward) and checked
    against an fp32 torch reference on the first batch entry's first and last GQA group and on the last batch entry."""
    Hq, D = 32, 64
    scale = 1 / math.sqrt(D)
    g = torch.Generator(device="cpu").manual_seed(9)
    q = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16).to(device)
    k = torch.randn(B, Hkv, Sk, D, generator=g).to(torch.bfloat16).to(device)
    v = torch.randn(B, Hkv, Sk, D, generator=g).to(torch.bfloat16).to(device)
    do = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16).to(device)
    out, lse = ops.attn_fwd(q, k, v, scale, causal, q_offset)
    dq, dk, dv = ops.attn_bwd(do, q, k, v, lse, None, scale, causal, q_offset, dq_dtype=torch.bfloat16,
                              dkv_dtype=torch.bfloat16, out=out)
    rep = Hq // Hkv
    off = q_offset if causal else Sk          # a diagonal past the last key = no mask
    for b, kvh in ((0, 0), (0, Hkv - 1), (B - 1, Hkv // 2)):
        bs, qs, ks = slice(b, b + 1), slice(kvh * rep, (kvh + 1) * rep), slice(kvh, kvh + 1)
        r_o, r_l, r_dq, r_dk, r_dv = ref_attention_fp32(q[bs, qs], k[bs, ks], v[bs, ks], scale, off, do[bs, qs])
        assert maxabs(out[bs, qs], r_o) <= 2e-2 and maxabs(lse[bs, qs], r_l) <= 1e-3
        assert rel_l2(dq[bs, qs], r_dq) <= 1e-2
        assert rel_l2(dk[bs, ks], r_dk) <= 1e-2 and rel_l2(dv[bs, ks], r_dv) <= 1e-2
    if causal and q_offset + Sq < Sk:
        assert dk[:, :, q_offset + Sq:].abs().max().item() == 0.0 and dv[:, :, q_offset + Sq:].abs().max().item() == 0.0


def test_configs4_long_context_rank7_of_8(ops, device):
    """configs[4]: rank 7 of cp 8 at total seq 32768 -- a 4096-token q chunk over 8 K/V chunks of 4096, GQA 32/8,
    head_dim 128, with RoPE at absolute positions.  Full size on the GPU; checks: RoPE offset == sliced tables (exact),
    per-chunk launches with the fused merge == one launch with q_offset, gradients of the two schedules agree, and one
    GQA group (4 query heads, 1 kv head) matches an fp32 torch reference."""
    W, Sc, Hq, Hkv, D, r = 8, 4096, 32, 8, 128, 7
    S = W * Sc
    scale = 1 / math.sqrt(D)
    g = torch.Generator(device="cpu").manual_seed(0)
    q = (torch.randn(1, Hq, Sc, D, generator=g) * scale).to(torch.bfloat16).to(device)
    k = torch.randn(1, Hkv, S, D, generator=g).to(torch.bfloat16).to(device)
    v = torch.randn(1, Hkv, S, D, generator=g).to(torch.bfloat16).to(device)
    do = torch.randn(1, Hq, Sc, D, generator=g).to(torch.bfloat16).to(device)

    # RoPE with absolute positions r*Sc + arange(Sc) on q, and chunk c's positions on each K chunk
    cos, sin = OL.get_cos_sin(S, D, 10000.0)
    cos_d, sin_d = cos.to(device), sin.to(device)
    pos = OR.position_ids(r, S, W, 1)
    assert pos[0, 0].item() == 28672 and pos[0, -1].item() == 32767
    q_rot = ops.rope(q, cos_d, sin_d, pos_offset=r * Sc)
    c_r, s_r = OR.rope_slice(cos, sin, r, W)
    assert torch.equal(q_rot, ops.rope(q, c_r.contiguous().to(device), s_r.contiguous().to(device)))
    k_rot = torch.empty_like(k)
    for c in range(W):
        cs = slice(c * Sc, (c + 1) * Sc)
        ops.rope(k[:, :, cs], cos_d, sin_d, pos_offset=c * Sc, out=k_rot[:, :, cs])
    assert torch.equal(k_rot, ops.rope(k, cos_d, sin_d))      # chunkwise offsets == one pass over the whole sequence
    want = OL.apply_rotary_pos_emb(q[:, :2].float().cpu(), c_r.float(), s_r.float())
    assert maxabs(q_rot[:, :2], want) <= 2e-2

    # forward: one launch with the diagonal shifted by r*Sc  vs  8 launches (diagonal chunk first) with fused merge
    out1, lse1 = ops.attn_fwd(q_rot, k_rot, v, scale, True, r * Sc)
    o32 = torch.empty(1, Hq, Sc, D, dtype=torch.float32, device=device)
    l32 = torch.empty(1, Hq, Sc, dtype=torch.float32, device=device)
    for step, held, run, blk_causal in OR.schedule(W, r, True):
        assert run
        cs = slice(held * Sc, (held + 1) * Sc)
        ops.attn_fwd(q_rot, k_rot[:, :, cs], v[:, :, cs], scale, blk_causal, 0, out=o32, lse=l32, merge=step > 0)
    assert maxabs(o32, out1) <= 1e-2 and maxabs(l32, lse1) <= 1e-4
    # backward: both schedules, fp32 accumulation across the ring steps
    delta = ops.attn_bwd_preprocess(do, out1)
    dq1, dk1, dv1 = ops.attn_bwd(do, q_rot, k_rot, v, lse1, delta, scale, True, r * Sc)
    dq2 = torch.empty_like(dq1)
    dk2, dv2 = torch.zeros_like(dk1), torch.zeros_like(dv1)
    for step, held, run, blk_causal in OR.schedule(W, r, True):
        cs = slice(held * Sc, (held + 1) * Sc)
        ops.attn_bwd(do, q_rot, k_rot[:, :, cs], v[:, :, cs], lse1, delta, scale, blk_causal, 0, dq2, dk2[:, :, cs],
                     dv2[:, :, cs], dq_accumulate=step > 0, dkv_accumulate=True)
    assert rel_l2(dq2, dq1) <= 1e-3 and rel_l2(dk2, dk1) <= 1e-3 and rel_l2(dv2, dv1) <= 1e-3
    # one GQA group against fp32 torch on the GPU
    qs = slice(4, 8)
    r_o, r_l, r_dq, r_dk, r_dv = ref_attention_fp32(q_rot[:, qs], k_rot[:, 1:2], v[:, 1:2], scale, r * Sc, do[:, qs])
    assert maxabs(out1[:, qs], r_o) <= 2e-2 and maxabs(lse1[:, qs], r_l) <= 1e-3
    assert rel_l2(dq1[:, qs], r_dq) <= 1e-2 and rel_l2(dk1[:, 1:2], r_dk) <= 1e-2 and rel_l2(dv1[:, 1:2], r_dv) <= 1e-2

    # the same step as ONE launch per direction over the eight chunks as separate tensors, RoPE inside the kernels:
    # q rotated in the forward's prologue at the rank's positions, dq / dk un-rotated in the backward's epilogues at
    # every chunk's own positions.  Forward: bit-equal to the one-tensor launch on the rotated q it leaves behind.
    ks = [k_rot[:, :, c * Sc:(c + 1) * Sc].contiguous() for c in range(W)]
    vs = [v[:, :, c * Sc:(c + 1) * Sc].contiguous() for c in range(W)]
    out3, lse3, q_rot3 = ops.attn_fwd_chunks(q, ks, vs, scale, True, r * Sc, rope=(cos_d, sin_d), q_pos_offset=r * Sc,
                                              want_q_rot=True)
    assert maxabs(q_rot3, q_rot) <= 2 ** -5      # one bf16 ulp of a rotated element (fp32 rotation, one rounding)
    o_chk, l_chk = ops.attn_fwd(q_rot3, k_rot, v, scale, True, r * Sc)
    assert torch.equal(out3, o_chk) and torch.equal(lse3, l_chk)
    assert maxabs(out3, out1) <= 2e-2 and maxabs(lse3, lse1) <= 2e-3
    dq3 = torch.empty_like(dq1)
    dks3 = [torch.empty(1, Hkv, Sc, D, dtype=torch.float32, device=device) for _ in range(W)]
    dvs3 = [torch.empty_like(t) for t in dks3]
    ops.attn_bwd_chunks(do, q_rot3, ks, vs, lse3, scale, True, r * Sc, dq3, dks3, dvs3, out=out3,
                        rope=(cos_d, sin_d), q_pos_offset=r * Sc, k_pos_offset=0)
    # reference for the un-rotated gradients: rotate the one-tensor launch's gradients back with the RoPE kernel
    dq_want = ops.rope(dq1, cos_d, sin_d, pos_offset=r * Sc, inverse=True)
    dk_want = ops.rope(dk1, cos_d, sin_d, inverse=True)
    assert rel_l2(dq3, dq_want) <= 1e-2
    assert rel_l2(torch.cat(dks3, 2), dk_want) <= 1e-2 and rel_l2(torch.cat(dvs3, 2), dv1) <= 1e-2


def test_elementwise_properties_at_full_sizes(ops, device):
    """Size-independent properties at the SmolLM-1.7B / Llama-2-7B step's sizes: RoPE is an isometry and its backward
    its inverse; RMSNorm output has unit RMS before the weight; SwiGLU backward is linear in dy."""
    bf = torch.bfloat16
    x = torch.randn(4, 1024, 32, 64, device=device).to(bf).transpose(1, 2)
    cos, sin = (t.to(device) for t in OL.get_cos_sin(1024, 64, 10000.0, dtype=torch.float32))
    y = ops.rope(x, cos, sin)
    n_in, n_out = x.float().pow(2).sum(-1), y.float().pow(2).sum(-1)
    assert ((n_out - n_in).abs() / n_in.clamp_min(1e-3)).max().item() <= 3e-2
    back = ops.rope(y, cos, sin, inverse=True)
    assert rel_l2(back, x) <= 1e-2
    h = torch.randn(4096, 4096, device=device).to(bf)
    yn, rstd, _ = ops.rmsnorm_fwd(h, torch.ones(4096, dtype=bf, device=device), 1e-5, False)
    assert (yn.float().pow(2).mean(-1).sqrt() - 1).abs().max().item() <= 1e-2
    assert torch.allclose(rstd, torch.rsqrt(h.float().pow(2).mean(-1) + 1e-5), rtol=1e-4)
    gt, up, d1, d2 = (torch.randn(1024, 11008, device=device).to(bf) for _ in range(4))
    a1, b1 = ops.swiglu_bwd(d1, gt, up)
    a2, b2 = ops.swiglu_bwd(d2, gt, up)
    a3, b3 = ops.swiglu_bwd((d1.float() + d2.float()).to(bf), gt, up)
    assert rel_l2(a3, a1.float() + a2.float()) <= 2e-2 and rel_l2(b3, b1.float() + b2.float()) <= 2e-2
