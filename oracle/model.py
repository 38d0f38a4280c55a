"""Oracle (test infrastructure): the reference's ``--use_cpu`` Llama, restated with plain torch ops.

Follows ``picotron/model.py`` with ``FLASH_ATTEN=0`` (forced by ``create_config.py:64-66``):
``LlamaRMSNorm`` (:67-86), ``apply_rotary_pos_emb`` (:12-19), ``F.scaled_dot_product_attention``
(:157) or the explicit-softmax ring blocks when ``cp_world_size > 1`` (:148-151), ``F.silu(gate)*up``
(:186); parameter init distributions and ORDER as in :112-120, :175-182, :201-209, :247-248, :279-289;
loss and optimiser as in ``train.py:29-55`` and ``train.py:209``.

Used (a) as the step-level oracle for the model-shaped GPU tests and (b) as the timed CPU baseline.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import layers, ring


@dataclass
class LlamaShape:
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    vocab_size: int
    num_hidden_layers: int
    max_position_embeddings: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0


def _uniform_fan_in_(w: torch.Tensor):
    bound = math.sqrt(1.0 / w.size(1))
    nn.init.uniform_(w, -bound, bound)


class OracleLayer(nn.Module):
    def __init__(self, cfg: LlamaShape, table_dtype=torch.bfloat16):
        super().__init__()
        h, nh, nkv = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads
        self.cfg = cfg
        self.head_dim = h // nh
        self.input_layernorm_weight = nn.Parameter(torch.empty(h))
        self.q_proj = nn.Linear(h, nh * self.head_dim, bias=False)
        self.k_proj = nn.Linear(h, nkv * self.head_dim, bias=False)
        self.v_proj = nn.Linear(h, nkv * self.head_dim, bias=False)
        self.out_proj = nn.Linear(h, h, bias=False)
        self.post_attention_layernorm_weight = nn.Parameter(torch.empty(h))
        self.up_proj = nn.Linear(h, cfg.intermediate_size, bias=False)
        self.gate_proj = nn.Linear(h, cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, h, bias=False)
        # tables are rounded to bf16 even on the fp32 CPU path because DTYPE is never exported
        cos, sin = layers.get_cos_sin(cfg.max_position_embeddings, self.head_dim, cfg.rope_theta, table_dtype)
        self.register_buffer("cos", cos, persistent=False)
        self.register_buffer("sin", sin, persistent=False)

    def reset_parameters(self):
        # order of model.py:279-289: input norm, attention (q,k,v,out), post norm, mlp (up, gate, down)
        nn.init.ones_(self.input_layernorm_weight)
        for lin in (self.q_proj, self.k_proj, self.v_proj, self.out_proj):
            _uniform_fan_in_(lin.weight)
        nn.init.ones_(self.post_attention_layernorm_weight)
        for lin in (self.up_proj, self.gate_proj, self.down_proj):
            _uniform_fan_in_(lin.weight)

    def attention(self, x, cp_world_size: int):
        b, s, _ = x.shape
        cfg = self.cfg
        q = self.q_proj(x).view(b, s, cfg.num_attention_heads, self.head_dim).transpose(1, 2)
        k = self.k_proj(x).view(b, s, cfg.num_key_value_heads, self.head_dim).transpose(1, 2)
        v = self.v_proj(x).view(b, s, cfg.num_key_value_heads, self.head_dim).transpose(1, 2)
        q = layers.apply_rotary_pos_emb(q, self.cos[:s], self.sin[:s])
        k = layers.apply_rotary_pos_emb(k, self.cos[:s], self.sin[:s])
        rep = cfg.num_attention_heads // cfg.num_key_value_heads
        k = k.repeat_interleave(rep, dim=1)
        v = v.repeat_interleave(rep, dim=1)
        if cp_world_size > 1:
            o, _ = ring.all_ranks_forward(q, k, v, cp_world_size, 1.0 / math.sqrt(self.head_dim), True)
        else:
            o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        o = o.transpose(1, 2).reshape(b, s, cfg.num_attention_heads * self.head_dim)
        return self.out_proj(o)

    def forward(self, x, cp_world_size: int = 1):
        eps = self.cfg.rms_norm_eps
        x = x + self.attention(layers.rmsnorm(x, self.input_layernorm_weight, eps), cp_world_size)
        y = layers.rmsnorm(x, self.post_attention_layernorm_weight, eps)
        return x + self.down_proj(layers.swiglu(self.gate_proj(y), self.up_proj(y)))


class OracleLlama(nn.Module):
    """embedding -> L x layer -> final norm -> untied vocabulary projection (``model.py:253-298``)."""

    def __init__(self, cfg: LlamaShape, table_dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.embedding = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList([OracleLayer(cfg, table_dtype) for _ in range(cfg.num_hidden_layers)])
        self.final_proj = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)
        self.final_norm_weight = nn.Parameter(torch.empty(cfg.hidden_size))
        self.reset_parameters()

    def reset_parameters(self):
        nn.init.normal_(self.embedding.weight, mean=0.0, std=1.0)
        for layer in self.layers:
            layer.reset_parameters()
        nn.init.ones_(self.final_norm_weight)
        _uniform_fan_in_(self.final_proj.weight)

    def forward(self, input_ids, cp_world_size: int = 1):
        x = self.embedding(input_ids)
        for layer in self.layers:
            x = layer(x, cp_world_size)
        x = layers.rmsnorm(x, self.final_norm_weight, self.cfg.rms_norm_eps)
        return self.final_proj(x)


def synthetic_batch(vocab_size: int, batch: int, seq: int, seed: int):
    """Token ids uniform over the vocabulary; targets are the ids shifted by one (``data.py:107-108``)."""
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, vocab_size, (batch, seq + 1), generator=g)
    return ids[:, :-1].contiguous(), ids[:, 1:].contiguous()


def train_step(model: nn.Module, optimizer, input_ids, target_ids, grad_acc_steps: int = 1, **fwd_kw):
    """zero_grad -> forward -> mean CE / grad_acc -> backward -> optimizer.step (``train.py:29-55,223-241``)."""
    optimizer.zero_grad()
    logits = model(input_ids, **fwd_kw)
    b, s = input_ids.shape
    loss = F.cross_entropy(logits.view(b * s, -1).float(), target_ids.reshape(-1), reduction="mean") / grad_acc_steps
    loss.backward()
    optimizer.step()
    return loss.item()


def smollm_135m_2layer(seq: int = 256) -> LlamaShape:
    return LlamaShape(576, 9, 3, 1536, 49152, 2, seq)


def smollm_1p7b(seq: int = 1024) -> LlamaShape:
    return LlamaShape(2048, 32, 32, 8192, 49152, 24, seq)


def llama2_7b(seq: int = 4096) -> LlamaShape:
    return LlamaShape(4096, 32, 32, 11008, 32000, 32, seq)
