"""The committed vectors of tests/golden/vectors.npz (made by tests/golden/make_fixtures.py from torch's library
routines in fp64, without the oracle) against the oracle on the CPU and against the HIP kernels on the GPU.  The
reference ships no golden vectors for this path; these pin both sides to the same independent numbers."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import layers as OL
from oracle import optim as OO
from oracle import ring as OR

VEC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz")
ATTN = ("attn_causal_offset", "attn_dense_ragged", "attn_causal_square")


@pytest.fixture(scope="module")
def vec():
    d = np.load(VEC, allow_pickle=False)
    return {k: torch.from_numpy(d[k]) for k in d.files}


def case(vec, name):
    c = {k.split(".", 1)[1]: v for k, v in vec.items() if k.startswith(name + ".")}
    B, Hq, Hkv, Sq, Sk, D, causal, off = (int(x) for x in c.pop("meta"))
    return c, dict(B=B, Hq=Hq, Hkv=Hkv, Sq=Sq, Sk=Sk, D=D, causal=bool(causal), off=off, scale=1.0 / math.sqrt(D))


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def maxabs(a, b):
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


# ------------------------------------------------------------------------------------ oracle vs vectors (CPU)
@pytest.mark.parametrize("name", ATTN)
def test_oracle_attention_matches_vectors(vec, name):
    """Blocks in the order a rank would run them (the diagonal block causal, the earlier keys dense), merged with the
    oracle's update rule, and the oracle's block backward with the merged (out, lse): fp32 against the fp64 vectors."""
    c, m = case(vec, name)
    rep = m["Hq"] // m["Hkv"]
    q, do = c["q"], c["do"]
    k, v = c["k"].repeat_interleave(rep, 1), c["v"].repeat_interleave(rep, 1)   # the reference expands GQA heads
    if m["causal"]:
        assert m["Sk"] == m["off"] + m["Sq"]
        blocks = [(slice(m["off"], m["Sk"]), True)] + ([(slice(0, m["off"]), False)] if m["off"] else [])
    else:
        blocks = [(slice(0, m["Sk"]), False)]
    out = lse = None
    for ks, blk_causal in blocks:
        out, lse = OR.merge(out, lse, *OR.block_forward(q, k[:, :, ks], v[:, :, ks], m["scale"], blk_causal))
    lse = lse.squeeze(-1)
    assert maxabs(out, c["out"]) <= 2e-6 and maxabs(lse, c["lse"]) <= 2e-6
    dq = torch.zeros_like(q)
    dk, dv = torch.zeros_like(k), torch.zeros_like(v)
    for ks, blk_causal in blocks:
        bq, bk, bv = OR.block_backward(do, q, k[:, :, ks], v[:, :, ks], out, lse, m["scale"], blk_causal)
        dq += bq
        dk[:, :, ks] += bk
        dv[:, :, ks] += bv
    fold = lambda t: t.view(m["B"], m["Hkv"], rep, m["Sk"], m["D"]).sum(2)
    assert rel_l2(dq, c["dq"]) <= 1e-5 and rel_l2(fold(dk), c["dk"]) <= 1e-5 and rel_l2(fold(dv), c["dv"]) <= 1e-5
    # the closed-form helper used elsewhere in the tests, on the same case
    o2, l2 = OR.full_attention_closed_form(q, k, v, m["scale"], m["causal"], m["off"])
    assert maxabs(o2, c["out"]) <= 2e-6 and maxabs(l2, c["lse"]) <= 2e-6


def test_oracle_layers_match_vectors(vec):
    y = OL.rmsnorm(vec["rmsnorm.x"], vec["rmsnorm.w"], 1e-5, cast_then_scale=False)
    dx, dw = OL.rmsnorm_backward(vec["rmsnorm.dy"], vec["rmsnorm.x"], vec["rmsnorm.w"], 1e-5)
    assert maxabs(y, vec["rmsnorm.y"]) <= 2e-6 and rel_l2(dx, vec["rmsnorm.dx"]) <= 1e-5 and rel_l2(dw, vec["rmsnorm.dw"]) <= 1e-5
    off, S, D = int(vec["rope.offset"][0]), vec["rope.x"].size(2), vec["rope.x"].size(3)
    cos, sin = OL.get_cos_sin(off + S, D, 10000.0, dtype=torch.float32)
    assert maxabs(OL.apply_rotary_pos_emb(vec["rope.x"], cos[off:], sin[off:]), vec["rope.y"]) <= 2e-6
    assert maxabs(OL.swiglu(vec["swiglu.gate"], vec["swiglu.up"]), vec["swiglu.y"]) <= 2e-6
    dg, du = OL.swiglu_backward(vec["swiglu.dy"], vec["swiglu.gate"], vec["swiglu.up"])
    assert rel_l2(dg, vec["swiglu.dgate"]) <= 1e-5 and rel_l2(du, vec["swiglu.dup"]) <= 1e-5
    tgt = vec["ce.targets"].to(torch.int64)
    loss, lse = OL.cross_entropy(vec["ce.logits"], tgt)
    assert abs(loss.item() - vec["ce.loss"].item()) <= 2e-6 and maxabs(lse, vec["ce.lse"]) <= 2e-6
    assert maxabs(OL.cross_entropy_backward(vec["ce.logits"], tgt), vec["ce.dlogits"]) <= 1e-7
    p, m, v = vec["adamw.p0"].double(), torch.zeros(300, dtype=torch.float64), torch.zeros(300, dtype=torch.float64)
    for step in range(3):
        p, m, v = OO.adamw_step(p, vec[f"adamw.g{step}"].double(), m, v, step + 1, 1e-2, 0.9, 0.95, 1e-8, 0.1)
        assert maxabs(p, vec[f"adamw.p{step + 1}"]) <= 1e-6
    assert maxabs(m, vec["adamw.m3"]) <= 1e-7 and maxabs(v, vec["adamw.v3"]) <= 1e-7


# ------------------------------------------------------------------------------------ HIP kernels vs vectors (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("name", ATTN)
def test_hip_attention_matches_vectors(vec, name, device):
    """One launch per direction with native GQA and the diagonal shifted by q_offset; tolerances of the path:
    forward max-abs 2e-2, lse 1e-3, gradients relative L2 1e-2."""
    from picotron_amd import ops
    c, m = case(vec, name)
    bf = lambda t: t.to(torch.bfloat16).to(device)
    q, k, v, do = bf(c["q"]), bf(c["k"]), bf(c["v"]), bf(c["do"])
    out, lse = ops.attn_fwd(q, k, v, m["scale"], m["causal"], m["off"])
    assert maxabs(out, c["out"]) <= 2e-2 and maxabs(lse, c["lse"]) <= 1e-3
    dq, dk, dv = ops.attn_bwd(do, q, k, v, lse, None, m["scale"], m["causal"], m["off"], out=out)
    assert rel_l2(dq, c["dq"]) <= 1e-2 and rel_l2(dk, c["dk"]) <= 1e-2 and rel_l2(dv, c["dv"]) <= 1e-2


@pytest.mark.gpu
def test_hip_layers_match_vectors(vec, device):
    from picotron_amd import ops
    bf = lambda t: t.to(torch.bfloat16).to(device)
    x, w, dy = bf(vec["rmsnorm.x"]), bf(vec["rmsnorm.w"]), bf(vec["rmsnorm.dy"])
    y, rstd, _ = ops.rmsnorm_fwd(x, w, 1e-5, False)
    dx, dw = ops.rmsnorm_bwd(dy, x, w, rstd)
    assert maxabs(y, vec["rmsnorm.y"]) <= 2e-2 and rel_l2(dx, vec["rmsnorm.dx"]) <= 1e-2 and rel_l2(dw, vec["rmsnorm.dw"]) <= 1e-5
    off, S, D = int(vec["rope.offset"][0]), vec["rope.x"].size(2), vec["rope.x"].size(3)
    cos, sin = OL.get_cos_sin(off + S, D, 10000.0, dtype=torch.float32)
    assert maxabs(ops.rope(bf(vec["rope.x"]), cos.to(device), sin.to(device), pos_offset=off), vec["rope.y"]) <= 2e-2
    g, u, d = bf(vec["swiglu.gate"]), bf(vec["swiglu.up"]), bf(vec["swiglu.dy"])
    assert maxabs(ops.swiglu_fwd(g, u), vec["swiglu.y"]) <= 2e-2 * max(1.0, vec["swiglu.y"].abs().max().item())
    dg, du = ops.swiglu_bwd(d, g, u)
    assert rel_l2(dg, vec["swiglu.dgate"]) <= 1e-2 and rel_l2(du, vec["swiglu.dup"]) <= 1e-2
    logits, tgt = bf(vec["ce.logits"]), vec["ce.targets"].to(torch.int64).to(device)
    loss_rows, lse = ops.cross_entropy_fwd(logits, tgt)
    n = int((tgt != -100).sum())
    assert abs(loss_rows.sum().item() / n - vec["ce.loss"].item()) <= 2e-5 and maxabs(lse, vec["ce.lse"]) <= 2e-5
    dl = ops.cross_entropy_bwd(logits, tgt, lse, torch.full((1,), 1.0 / n, device=device))
    assert maxabs(dl, vec["ce.dlogits"]) <= 2 ** -8 * vec["ce.dlogits"].abs().max().item()
    # AdamW: fp32 master weights follow the fp64 run to fp32 accuracy, the bf16 copy is the rounded master weight
    master = vec["adamw.p0"].to(device)
    m, v = torch.zeros(300, device=device), torch.zeros(300, device=device)
    p_lp = torch.empty(300, dtype=torch.bfloat16, device=device)
    for step in range(3):
        ops.adamw_(p_lp, master, bf(vec[f"adamw.g{step}"]), m, v, step + 1, 1e-2, 0.9, 0.95, 1e-8, 0.1)
        assert maxabs(master, vec[f"adamw.p{step + 1}"]) <= 2e-6
    assert maxabs(m, vec["adamw.m3"]) <= 1e-7 and maxabs(v, vec["adamw.v3"]) <= 1e-7
    assert torch.equal(p_lp, master.to(torch.bfloat16))
