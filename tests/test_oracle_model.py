"""Pins the CPU oracle's whole model (``oracle.model.OracleLlama``) against an independent implementation of the same
architecture: transformers' ``LlamaForCausalLM`` (a library routine; the reference loads Hugging Face Llama checkpoints
into this very layout, ``checkpoint.py``).  With the same weights the two must give the same logits, loss and gradients;
a wrong RoPE convention, GQA head mapping, residual wiring, norm placement or projection order fails here."""
import pytest
import torch
import torch.nn.functional as F

from oracle import model as OM

tr = pytest.importorskip("transformers")


def _pair(nh, nkv, layers=2, seq=24, hidden=64, inter=96, vocab=101):
    torch.manual_seed(0)
    cfg = OM.LlamaShape(hidden, nh, nkv, inter, vocab, layers, seq, rope_theta=10000.0)
    ours = OM.OracleLlama(cfg, table_dtype=torch.float32)
    hcfg = tr.LlamaConfig(hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers, num_attention_heads=nh,
                          num_key_value_heads=nkv, vocab_size=vocab, max_position_embeddings=seq, rms_norm_eps=1e-5,
                          rope_theta=10000.0, tie_word_embeddings=False, attention_bias=False, mlp_bias=False,
                          attn_implementation="eager")
    hf = tr.LlamaForCausalLM(hcfg).float()
    # norm weights away from 1 so that their placement matters
    with torch.no_grad():
        for p in ours.parameters():
            if p.dim() == 1:
                p.uniform_(0.5, 1.5)
    names = {"model.embed_tokens.weight": ours.embedding.weight, "model.norm.weight": ours.final_norm_weight,
             "lm_head.weight": ours.final_proj.weight}
    for i, layer in enumerate(ours.layers):
        pre = f"model.layers.{i}."
        names.update({pre + "self_attn.q_proj.weight": layer.q_proj.weight, pre + "self_attn.k_proj.weight": layer.k_proj.weight,
                      pre + "self_attn.v_proj.weight": layer.v_proj.weight, pre + "self_attn.o_proj.weight": layer.out_proj.weight,
                      pre + "mlp.gate_proj.weight": layer.gate_proj.weight, pre + "mlp.up_proj.weight": layer.up_proj.weight,
                      pre + "mlp.down_proj.weight": layer.down_proj.weight,
                      pre + "input_layernorm.weight": layer.input_layernorm_weight,
                      pre + "post_attention_layernorm.weight": layer.post_attention_layernorm_weight})
    hf_params = dict(hf.named_parameters())
    assert set(hf_params) == set(names)
    with torch.no_grad():
        for n, p in hf_params.items():
            p.copy_(names[n])
    return cfg, ours, hf, names


@pytest.mark.parametrize("nh,nkv", [(4, 4), (4, 2), (4, 1)])
@pytest.mark.parametrize("cp_world_size", [1, 2])
def test_oracle_model_equals_transformers_llama(nh, nkv, cp_world_size):
    cfg, ours, hf, names = _pair(nh, nkv)
    ids, tgt = OM.synthetic_batch(cfg.vocab_size, 2, cfg.max_position_embeddings, seed=3)
    logits = ours(ids, cp_world_size=cp_world_size)
    want = hf(input_ids=ids).logits
    assert (logits - want).abs().max().item() <= 2e-4 * want.abs().max().item()
    loss = F.cross_entropy(logits.view(-1, cfg.vocab_size), tgt.reshape(-1))
    want_loss = F.cross_entropy(want.view(-1, cfg.vocab_size), tgt.reshape(-1))
    assert abs(loss.item() - want_loss.item()) <= 1e-5
    loss.backward()
    want_loss.backward()
    for n, p in hf.named_parameters():
        g, w = names[n].grad, p.grad
        assert ((g - w).norm() / w.norm().clamp_min(1e-12)).item() <= 1e-3, n


def test_oracle_train_step_equals_transformers_llama_with_torch_adamw():
    """One full step of ``oracle.model.train_step`` (``train.py:29-55,204-209``) moves the weights exactly as the same
    step taken with the library model."""
    cfg, ours, hf, names = _pair(4, 2)
    ids, tgt = OM.synthetic_batch(cfg.vocab_size, 2, cfg.max_position_embeddings, seed=4)
    opt_a = torch.optim.AdamW(ours.parameters(), lr=1e-2)
    opt_b = torch.optim.AdamW(hf.parameters(), lr=1e-2)
    loss_a = OM.train_step(ours, opt_a, ids, tgt)
    opt_b.zero_grad()
    loss_b = F.cross_entropy(hf(input_ids=ids).logits.view(-1, cfg.vocab_size), tgt.reshape(-1))
    loss_b.backward()
    opt_b.step()
    assert abs(loss_a - loss_b.item()) <= 1e-5
    for n, p in hf.named_parameters():
        # the first AdamW step moves every weight by about lr * sign(grad): compare the moves
        assert (names[n] - p).abs().max().item() <= 2e-4, n
