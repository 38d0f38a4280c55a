"""GPU parity of the training step at BASELINE.json's configs[2] (SmolLM-1.7B shape) and configs[3] (Llama-2-7B
shape): the exact per-layer shape, batch and sequence length of the config with the layer count cut to 2, every
default fused path on (one GEMM for q/k/v and one for gate/up, residual stream chained through the RMSNorm
kernels, the cross-entropy kernel, FusedAdamW on bf16 parameters with fp32 moments), against the fp32 CPU oracle
started from the same (bf16-representable) weights.  Reference: ``train.py:29-55`` (step) and ``:209`` (AdamW).

Tolerances.  The GPU step computes in bf16 with fp32 accumulation, the oracle in fp32, so: loss within 3e-2;
parameter gradients within rel-L2 5e-2 (bf16 rounding of every activation along two layers; the kernels alone
meet 1e-2, tests/test_gpu_kernels.py).  The first AdamW step moves every weight by lr * g / (|g| + eps) = +-lr, so
the update itself is compared through its direction (sign agreement where the gradient is not noise), its size
(|new - old| <= lr * (1 + wd) + one bf16 spacing) and the stored result: the oracle's updated fp32 weight, rounded
to bf16 as the in-place update stores it, must be the GPU's weight bit for bit on >= 97 % of the elements (the rest
are gradient-sign flips of elements whose gradient is noise, and rounding ties).  The step as a whole is compared
through the loss of a SECOND step, which both sides take from their own updated weights; the oracle's weights are
rounded to bf16 after its first step because that is what "bf16 parameters updated in place" stores.
"""
import os

import pytest
import torch

from oracle import model as OM

pytestmark = pytest.mark.gpu

LR = 3e-4


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def _copy_weights(ours, oracle):
    with torch.no_grad():
        ours.embedding.weight.copy_(oracle.embedding.weight)
        for a, b in zip(ours.decoder_layers, oracle.layers):
            a.input_layernorm.weight.copy_(b.input_layernorm_weight)
            a.post_attention_layernorm.weight.copy_(b.post_attention_layernorm_weight)
            for n in ("q_proj", "k_proj", "v_proj", "out_proj"):
                getattr(a.attention, n).weight.copy_(getattr(b, n).weight)
            for n in ("up_proj", "gate_proj", "down_proj"):
                getattr(a.mlp, n).weight.copy_(getattr(b, n).weight)
        ours.final_norm.weight.copy_(oracle.final_norm_weight)
        ours.final_proj.weight.copy_(oracle.final_proj.weight)


CONFIGS = {
    # name: (shape with 2 layers, micro-batch, sequence length)
    "configs2_smollm_1p7b": (OM.LlamaShape(2048, 32, 32, 8192, 49152, 2, 1024), 4, 1024),
    "configs3_llama2_7b": (OM.LlamaShape(4096, 32, 32, 11008, 32000, 2, 4096), 1, 4096),
}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_two_layer_training_steps_match_cpu_oracle(device, name):
    import picotron_amd.process_group_manager as pgm
    from picotron_amd.functional import cross_entropy
    from picotron_amd.model import Llama, TritonRMSNorm
    from picotron_amd.optim import FusedAdamW

    cfg, mbs, seq = CONFIGS[name]
    pgm.setup_process_group_manager(1, 1, 1, 1)
    os.environ["CONTEXT_PARALLEL"] = "0"
    for var in ("FLASH_ATTEN", "PICO_FUSED_PROJ", "PICO_FUSED_RESIDUAL"):
        os.environ.pop(var, None)
    torch.set_num_threads(min(16, os.cpu_count() or 1))

    torch.manual_seed(42)
    oracle = OM.OracleLlama(cfg)
    with torch.no_grad():
        for p in oracle.parameters():
            p.copy_(p.to(torch.bfloat16).float())      # both sides start from the same bf16-representable weights
    ours = Llama(cfg)
    _copy_weights(ours, oracle)
    ours = ours.to(torch.bfloat16).to(device)
    assert isinstance(ours.final_norm, TritonRMSNorm)   # the default (fused residual) path is the one under test
    ids, tgt = OM.synthetic_batch(cfg.vocab_size, mbs, seq, seed=0)
    ids_d, tgt_d = ids.to(device), tgt.to(device)

    opt = FusedAdamW(ours.parameters(), lr=LR, master_weights=False, state_dtype=torch.float32)
    opt_o = torch.optim.AdamW(oracle.parameters(), lr=LR)

    def gpu_step():
        opt.zero_grad()
        logits = ours(input_ids=ids_d)
        loss = cross_entropy(logits.view(mbs * seq, -1), tgt_d.reshape(-1))
        loss.backward()
        grads = {n: p.grad.detach().float().cpu() for n, p in ours.named_parameters() if n in watched}
        opt.step()
        return loss.item(), grads

    watched = {"decoder_layers.0.attention.q_proj.weight", "decoder_layers.1.mlp.down_proj.weight",
               "decoder_layers.1.mlp.gate_proj.weight", "final_norm.weight", "embedding.weight"}
    q_before = ours.decoder_layers[0].attention.q_proj.weight.detach().float().cpu().clone()
    loss1, g1 = gpu_step()
    q_after = ours.decoder_layers[0].attention.q_proj.weight.detach().float().cpu().clone()
    loss2, _ = gpu_step()
    torch.cuda.synchronize()

    # the oracle: gradients of step 1 are read before step 2 overwrites them
    print(f"{name}: CPU oracle step 1 ...", flush=True)
    q_before_o = oracle.layers[0].q_proj.weight.detach().clone()
    loss1_o = OM.train_step(oracle, opt_o, ids, tgt)
    g1_o = {
        "decoder_layers.0.attention.q_proj.weight": oracle.layers[0].q_proj.weight.grad.clone(),
        "decoder_layers.1.mlp.down_proj.weight": oracle.layers[1].down_proj.weight.grad.clone(),
        "decoder_layers.1.mlp.gate_proj.weight": oracle.layers[1].gate_proj.weight.grad.clone(),
        "final_norm.weight": oracle.final_norm_weight.grad.clone(),
        "embedding.weight": oracle.embedding.weight.grad.clone(),
    }
    with torch.no_grad():
        for p in oracle.parameters():
            p.copy_(p.to(torch.bfloat16).float())      # the parameters live in bf16 (fp32 moments only)
    q_after_o = oracle.layers[0].q_proj.weight.detach().clone()
    print(f"{name}: CPU oracle step 2 ...", flush=True)
    loss2_o = OM.train_step(oracle, opt_o, ids, tgt)
    print(f"{name}: loss {loss1:.4f} / {loss1_o:.4f}, after one step {loss2:.4f} / {loss2_o:.4f}", flush=True)

    assert abs(loss1 - loss1_o) <= 3e-2, (loss1, loss1_o)
    for n in sorted(watched):
        assert rel_l2(g1[n], g1_o[n]) <= 5e-2, (n, rel_l2(g1[n], g1_o[n]))

    # the AdamW step: size, direction, and what it does to the loss
    assert torch.equal(q_before, q_before_o)
    upd, upd_o = q_after - q_before, q_after_o - q_before_o
    spacing = q_before.abs() * 2.0 ** -7                     # one bf16 spacing at the weight's magnitude (upper bound)
    assert bool(((upd.abs() <= LR * 1.01 + spacing)).all())
    clear = g1_o["decoder_layers.0.attention.q_proj.weight"].abs() > g1_o["decoder_layers.0.attention.q_proj.weight"].abs().median()
    moved = clear & (upd != 0)
    agree = (torch.sign(upd[moved]) == torch.sign(upd_o[moved])).float().mean().item()
    assert agree >= 0.99, agree
    assert (q_after - q_after_o).abs().max().item() <= 2.05 * LR + spacing.max().item()
    same = (q_after == q_after_o).float().mean().item()
    assert same >= 0.97, same
    assert loss2 < loss1 and loss2_o < loss1_o
    assert abs(loss2 - loss2_o) <= 3e-2, (loss2, loss2_o)
    assert abs((loss1 - loss2) - (loss1_o - loss2_o)) <= 0.25 * (loss1_o - loss2_o) + 1e-2
