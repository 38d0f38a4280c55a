"""Host helpers mirrored from ``picotron/utils.py``: seeding (:23-26), number formatting (:28-38) and the
MFU formula (:43-49) with MI355X's dense bf16 peak in place of the H100 constant."""
from __future__ import annotations

import random
from dataclasses import dataclass

import numpy as np
import torch

MI355X_BF16_DENSE_FLOPS = 2.5e15  # published dense bf16 matrix peak of one MI355X


def set_all_seed(seed):
    for module in [random, np.random]:
        module.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


def to_readable_format(num, precision=2):
    for limit, suffix in ((1e12, "T"), (1e9, "B"), (1e6, "M"), (1e3, "K")):
        if num >= limit:
            return f"{num / limit:.{precision}f}{suffix}"
    return f"{num:.{precision}f}"


def flops_per_token(num_params, num_layers, hidden_dim, seq_len):
    """6*N + 12*L*h*S, the per-token training FLOPs the reference's MFU uses (``utils.py:47``)."""
    return 6 * num_params + 12 * num_layers * hidden_dim * seq_len


def get_mfu(tokens_per_second, num_params, model_config, theoretical_flops=MI355X_BF16_DENSE_FLOPS):
    fpt = flops_per_token(num_params, model_config.num_hidden_layers, model_config.hidden_size,
                          model_config.max_position_embeddings)
    return tokens_per_second * fpt / theoretical_flops * 100


def get_num_params(model):
    return sum(p.numel() for p in model.parameters())


@dataclass
class ModelShape:
    """The fields of a Hugging Face Llama config that ``model.Llama`` reads (the reference builds its config with
    ``AutoConfig.from_pretrained`` and overrides these, ``train.py:154-162``); max_position_embeddings = seq_length."""
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    vocab_size: int
    num_hidden_layers: int
    max_position_embeddings: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0


def smollm_1p7b_shape(seq_length=1024):
    return ModelShape(2048, 32, 32, 8192, 49152, 24, seq_length)


def llama2_7b_shape(seq_length=4096):
    return ModelShape(4096, 32, 32, 11008, 32000, 32, seq_length)


def synthetic_tokens(vocab_size, batch, seq_length, seed):
    """Token ids uniform over the vocabulary; the targets are the ids shifted by one: seq_length + 1 tokens are drawn
    per sample and split, as the reference's collate function does (``data.py:102-116``)."""
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, vocab_size, (batch, seq_length + 1), generator=g)
    return ids[:, :-1].contiguous(), ids[:, 1:].contiguous()
