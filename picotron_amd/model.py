"""The Llama of ``picotron/model.py`` with its hot ops on hand-written gfx950 kernels.

Class and function names, constructor arguments, forward signatures, parameter names, init
distributions and init order are the reference's (``model.py:12-298``); what changes is what runs
underneath:

=====================================  =====================================================
reference (file:line)                  here
=====================================  =====================================================
apply_rotary_pos_emb      :12-19       RoPE kernel (``pico_rope``), strided [B,H,S,D] views
flash_attn rotary         :136-137     same kernel
flash_attention           :33-37       MFMA attention kernels (``pico_attn_fwd`` / ``_bwd``)
F.scaled_dot_product_attention :157    same kernels (there is no CPU / torch attention path)
TritonRMSNorm             :39-65       RMSNorm kernel, fp32 maths + one rounding, optional
                                       fused residual add / prenorm
LlamaRMSNorm              :67-86       RMSNorm kernel, cast-then-scale rounding order
F.silu(gate) * up         :186         SwiGLU kernel
repeat_interleave (GQA)   :142-143     not materialised: the kernels index the kv head
=====================================  =====================================================

The projections, embedding and vocabulary projection stay on torch / hipBLASLt.
Environment switches are read at call time like the reference does: ``FLASH_ATTEN`` picks the
RMSNorm class (:218, :274) and the RoPE call shape (:127-140), ``CONTEXT_PARALLEL`` routes
attention through the ring (:148).
"""
from __future__ import annotations

import math
import os

import torch
import torch.nn as nn
import torch.nn.functional as F

import picotron_amd.process_group_manager as pgm
from picotron_amd.context_parallel import context_parallel
from picotron_amd.functional import (FlashAttnFunc, FusedLinearFunc, QKVAttentionFunc, RMSNormFunc, RMSNormResidualFunc,
                                     RotaryFunc, SwiGLUFunc, SwiGLUFusedFunc, _fused_rope)


def apply_rotary_pos_emb(x, cos, sin):
    """x [B,H,S,D] (any strides with unit D stride), cos/sin [S,D] with duplicated halves."""
    return RotaryFunc.apply(x, cos, sin, 0)


def get_cos_sin(seq_length, head_dim, base=500000.0):
    """[S, D] cos / sin tables, halves duplicated; theta on the CPU, angles in fp32 on the device,
    table dtype from ``DTYPE`` (bf16 unless set otherwise) -- the recipe of ``model.py:21-31``."""
    assert head_dim % 2 == 0
    exponents = torch.arange(0, head_dim, 2, dtype=torch.int64).float().to("cpu") / head_dim
    theta = 1.0 / (base ** exponents)
    dtype = torch.bfloat16 if os.getenv("DTYPE", "bfloat16") == "bfloat16" else torch.float32
    local_rank = int(os.environ.get("LOCAL_RANK", "0"))
    device = torch.device("cuda", local_rank) if os.getenv("DEVICE", "cuda") == "cuda" else torch.device("cpu")
    position = torch.arange(seq_length).to(device).unsqueeze(1).float()
    angle = position * theta.to(device).float()
    return torch.cos(angle).to(dtype).repeat(1, 2), torch.sin(angle).to(dtype).repeat(1, 2)


def flash_attention(q, k, v, causal=True):
    """q [B,Hq,S,D], k/v [B,Hkv,S,D] -> [B,S,Hq,D] (the layout flash_attn_func returns, ``model.py:33-37``)."""
    sm_scale = 1.0 / math.sqrt(q.size(-1))
    return FlashAttnFunc.apply(q, k, v, sm_scale, causal).transpose(1, 2)


class TritonRMSNorm(nn.Module):
    """RMSNorm with fp32 maths and a single rounding; keeps the reference's class name and call shape."""

    def __init__(self, hidden_size, eps=1e-5, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        nn.init.ones_(self.weight)

    def forward(self, hidden_states, residual=None, dropout_p=0.0, prenorm=False, residual_in_fp32=False,
                return_dropout_mask=False):
        """The call shape of flash-attn's ``layer_norm_fn(..., is_rms_norm=True)`` as the reference passes it through
        (``model.py:54-65``): h = dropout(x) + residual, y = rmsnorm(h) * w in x's dtype; ``prenorm`` also returns h
        (in fp32 if ``residual_in_fp32``), ``return_dropout_mask`` appends the keep mask and a None (the second
        input's mask, which does not exist here).  picotron itself calls it without dropout and with residuals in the
        activations' dtype: those calls take the fused kernels; dropout and the fp32 add are torch operations in front
        of the norm kernel."""
        if dropout_p == 0.0 and not return_dropout_mask and not residual_in_fp32:
            if residual is None:
                y = RMSNormFunc.apply(hidden_states, self.weight, self.eps, False)
                return (y, hidden_states) if prenorm else y
            y, h = RMSNormResidualFunc.apply(hidden_states, residual, self.weight, self.eps)
            return (y, h) if prenorm else y
        x = hidden_states
        mask = None
        h = x.float()
        if dropout_p > 0.0:
            mask = torch.rand_like(h) >= dropout_p
            h = h * mask * (1.0 / (1.0 - dropout_p))
        elif return_dropout_mask:
            mask = torch.ones_like(h, dtype=torch.bool)
        if residual is not None:
            h = h + residual.float()
        if residual_in_fp32:
            y = RMSNormFunc.apply(h, self.weight.float(), self.eps, False).to(x.dtype)
        else:
            h = h.to(x.dtype if residual is None else residual.dtype)
            y = RMSNormFunc.apply(h.to(x.dtype), self.weight, self.eps, False)
        out = (y, h) if prenorm else (y,)
        if return_dropout_mask:
            out = out + (mask, None)
        return out if len(out) > 1 else out[0]


class LlamaRMSNorm(nn.Module):
    """RMSNorm that rounds the normalised value to the input dtype before scaling (``model.py:81-86``)."""

    def __init__(self, hidden_size, eps=1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(hidden_size))
        self.variance_epsilon = eps
        self.reset_parameters()

    def reset_parameters(self):
        nn.init.ones_(self.weight)

    def forward(self, hidden_states):
        return RMSNormFunc.apply(hidden_states, self.weight, self.variance_epsilon, True)


def _fused_projections() -> bool:
    """One GEMM for q/k/v and one for gate/up (default); PICO_FUSED_PROJ=0 keeps the reference's separate GEMMs."""
    return os.getenv("PICO_FUSED_PROJ", "1") != "0"


def _fused_residual() -> bool:
    """Residual adds inside the RMSNorm kernels on both passes (default); PICO_FUSED_RESIDUAL=0 keeps them apart."""
    return os.getenv("PICO_FUSED_RESIDUAL", "1") != "0"


def _fused_weight(owner, name, linears):
    """The [sum(out_i), in] buffer that the weights of `linears` alias, row block by row block.  Built on first use
    and rebuilt whenever the Parameters were moved or cast since (``model.to(...)`` gives them fresh storage); the
    Parameters stay separate leaves with their own names, gradients and optimizer state."""
    ws = [m.weight for m in linears]
    buf = owner.__dict__.get(name)
    ok = buf is not None and buf.dtype == ws[0].dtype and buf.device == ws[0].device
    if ok:
        ptr = buf.data_ptr()
        for w in ws:
            ok = ok and w.data_ptr() == ptr and w.is_contiguous()
            ptr += w.numel() * w.element_size()
    if not ok:
        with torch.no_grad():
            buf = torch.cat([w.detach() for w in ws], dim=0).contiguous()
            row = 0
            for w in ws:
                w.data = buf[row:row + w.size(0)]
                row += w.size(0)
        owner.__dict__[name] = buf
    return buf


def _fan_in_uniform_(tensor):
    bound = math.sqrt(1 / tensor.size(1))
    torch.nn.init.uniform_(tensor, -bound, bound)


class Attention(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        mgr = pgm.process_group_manager
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.num_key_values = config.num_key_value_heads
        self.head_dim = self.hidden_size // self.num_heads
        assert config.num_attention_heads % mgr.tp_world_size == 0, "num_attention_heads should be divisible by tp world size"
        assert config.num_key_value_heads % mgr.tp_world_size == 0, "num_key_value_heads should be divisible by  tp world size"
        self.num_local_heads = config.num_attention_heads // mgr.tp_world_size
        self.num_local_kv_heads = config.num_key_value_heads // mgr.tp_world_size

        self.q_proj = nn.Linear(config.hidden_size, self.num_heads * self.head_dim, bias=False)
        self.k_proj = nn.Linear(config.hidden_size, self.num_key_values * self.head_dim, bias=False)
        self.v_proj = nn.Linear(config.hidden_size, self.num_key_values * self.head_dim, bias=False)
        self.out_proj = nn.Linear(config.hidden_size, config.hidden_size, bias=False)
        self.layer_idx = layer_idx
        self.reset_parameters()

    def reset_parameters(self):
        for proj in (self.q_proj, self.k_proj, self.v_proj, self.out_proj):
            _fan_in_uniform_(proj.weight)

    def forward(self, x, cos, sin, attention_mask=None, position_ids=None):
        batch_size, seq_length, _ = x.size()
        context = os.getenv("CONTEXT_PARALLEL", "0") == "1"
        if _fused_projections() and cos.size(0) >= seq_length:
            # one GEMM for q, k and v; RoPE, attention and their backward work on strided views of the fused buffers
            w = _fused_weight(self, "_qkv_weight", (self.q_proj, self.k_proj, self.v_proj))
            qkv = FusedLinearFunc.apply(x, w, self.q_proj.weight, self.k_proj.weight, self.v_proj.weight)
            if not context:
                out = QKVAttentionFunc.apply(qkv, cos, sin, self.num_local_heads, self.num_local_kv_heads, self.head_dim, True)
                return self.out_proj(out)
            nq, nkv = self.num_local_heads * self.head_dim, self.num_local_kv_heads * self.head_dim
            q = qkv[..., :nq].view(batch_size, seq_length, self.num_local_heads, self.head_dim).transpose(1, 2)
            k = qkv[..., nq:nq + nkv].view(batch_size, seq_length, self.num_local_kv_heads, self.head_dim).transpose(1, 2)
            v = qkv[..., nq + nkv:].view(batch_size, seq_length, self.num_local_kv_heads, self.head_dim).transpose(1, 2)
            sm_scale = 1.0 / (self.head_dim ** 0.5)
            whole_cos, whole_sin = getattr(cos, "whole_table", None), getattr(sin, "whole_table", None)
            rank_pos = pgm.process_group_manager.cp_rank * seq_length
            if (_fused_rope() and whole_cos is not None and whole_sin is not None
                    and whole_cos[1] == rank_pos and whole_sin[1] == rank_pos):
                # RoPE inside the ring: q rotated in the attention forward at the rank's absolute positions, k by one
                # launch before its chunk is published, dq / dk un-rotated in the backward kernels' epilogues
                out = context_parallel.ring_attention(q, k, v, sm_scale, True, rope=(whole_cos[0], whole_sin[0]))
            else:
                out = context_parallel.ring_attention(apply_rotary_pos_emb(q, cos, sin), apply_rotary_pos_emb(k, cos, sin), v,
                                                      sm_scale, True)
            return self.out_proj(out.transpose(1, 2).reshape(batch_size, seq_length, nq))
        # [B,S,H*D] -> [B,H,S,D] views over [B,S,H,D] memory; the kernels take the strides as they are
        q = self.q_proj(x).view(batch_size, seq_length, self.num_local_heads, self.head_dim).transpose(1, 2)
        k = self.k_proj(x).view(batch_size, seq_length, self.num_local_kv_heads, self.head_dim).transpose(1, 2)
        v = self.v_proj(x).view(batch_size, seq_length, self.num_local_kv_heads, self.head_dim).transpose(1, 2)
        q = apply_rotary_pos_emb(q, cos, sin)
        k = apply_rotary_pos_emb(k, cos, sin)
        # GQA: no repeat_interleave -- query head h reads kv head h // (Hq/Hkv) inside the kernels

        causal = True if q.size(2) == k.size(2) else False

        if os.getenv("CONTEXT_PARALLEL", "0") == "1":
            sm_scale = 1.0 / (q.size(-1) ** 0.5)
            out = context_parallel.ring_attention(q, k, v, sm_scale, causal).transpose(1, 2)
        else:
            out = flash_attention(q, k, v, causal=causal)  # [B,S,H,D]

        out = out.reshape(batch_size, seq_length, self.num_local_heads * self.head_dim)
        return self.out_proj(out)


class MLP(nn.Module):
    def __init__(self, config) -> None:
        super().__init__()
        self.up_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.gate_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=False)
        self.reset_parameters()

    def reset_parameters(self):
        for proj in (self.up_proj, self.gate_proj, self.down_proj):
            _fan_in_uniform_(proj.weight)

    def forward(self, x):
        if _fused_projections():
            w = _fused_weight(self, "_gate_up_weight", (self.gate_proj, self.up_proj))
            gate_up = FusedLinearFunc.apply(x, w, self.gate_proj.weight, self.up_proj.weight)
            return self.down_proj(SwiGLUFusedFunc.apply(gate_up))
        return self.down_proj(SwiGLUFunc.apply(self.gate_proj(x), self.up_proj(x)))


class FinalProjection(nn.Module):
    def __init__(self, hidden_size, vocab_size, bias=False):
        super().__init__()
        self.in_features = hidden_size
        self.out_features = vocab_size
        self.weight = nn.Parameter(torch.empty(self.out_features, self.in_features))
        self.bias = nn.Parameter(torch.empty(self.out_features)) if bias else None
        self.reset_parameters()

    def reset_parameters(self):
        bound = math.sqrt(1 / self.weight.size(1))
        torch.nn.init.uniform_(self.weight, -bound, bound)
        if self.bias is not None:
            bound_b = math.sqrt(1 / self.bias.size(0)) if self.bias.dim() == 1 else bound
            torch.nn.init.uniform_(self.bias, -bound_b, bound_b)

    def forward(self, x):
        return F.linear(x, self.weight, self.bias)


class DecoderLayer(nn.Module):
    """RMSNorm -> Attention -> residual -> RMSNorm -> MLP -> residual."""

    def __init__(self, config, layer_idx):
        super().__init__()
        RMSNorm = LlamaRMSNorm if os.getenv("FLASH_ATTEN", "1") != "1" else TritonRMSNorm
        self.input_layernorm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.attention = Attention(config, layer_idx=layer_idx)
        self.mlp = MLP(config)
        self.layer_idx = layer_idx
        head_dim = config.hidden_size // config.num_attention_heads
        self.cos, self.sin = get_cos_sin(config.max_position_embeddings, head_dim=head_dim, base=config.rope_theta)
        # context parallelism splits the sequence: keep the rows of this rank's positions
        self.cos, self.sin = context_parallel.update_rope_for_context_parallel(self.cos, self.sin)

    def forward(self, x, attention_mask=None, position_ids=None):
        cos, sin = self.cos, self.sin
        x = x + self.attention(self.input_layernorm(x), cos, sin, attention_mask, position_ids)
        x = x + self.mlp(self.post_attention_layernorm(x))
        return x

    def forward_chained(self, branch, residual, attention_mask=None, position_ids=None):
        """The same layer with the residual stream carried beside the branch output, the way flash-attn's
        layer_norm_fn(residual=..., prenorm=True) is meant to be chained: the layer's input is `branch + residual`
        (`residual` None: just `branch`), each add happens inside the norm kernel that follows it, and the layer
        returns (mlp output, residual stream before it) for the next norm to add.  Forward values are those of
        forward(); in the backward the gradient of the residual stream enters the norm's backward kernel, so no
        separate add runs on either pass."""
        y, residual = self.input_layernorm(branch, residual=residual, prenorm=True)
        a = self.attention(y, self.cos, self.sin, attention_mask, position_ids)
        y, residual = self.post_attention_layernorm(a, residual=residual, prenorm=True)
        return self.mlp(y), residual


class Embedding(nn.Module):
    def __init__(self, num_embeddings, embedding_dim, padding_idx=None):
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.padding_idx = padding_idx
        self.weight = nn.Parameter(torch.empty(num_embeddings, embedding_dim))
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.normal_(self.weight, mean=0.0, std=1.0)

    def forward(self, x):
        return F.embedding(x, self.weight, self.padding_idx)


class Llama(nn.Module):
    def __init__(self, config) -> None:
        super().__init__()
        assert config.hidden_size % config.num_attention_heads == 0
        assert config.num_attention_heads % config.num_key_value_heads == 0
        self.vocab_size = config.vocab_size
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.num_key_values = config.num_key_value_heads
        self.head_dim = self.hidden_size // self.num_heads
        self.max_position_embeddings = config.max_position_embeddings
        self.num_layers = config.num_hidden_layers
        self.model_config = config

        self.embedding = Embedding(self.vocab_size, self.hidden_size)
        self.decoder_layers = nn.ModuleList([DecoderLayer(config, layer_idx=i) for i in range(self.num_layers)])
        self.final_proj = FinalProjection(self.hidden_size, self.vocab_size, bias=False)
        RMSNorm = LlamaRMSNorm if os.getenv("FLASH_ATTEN", "1") != "1" else TritonRMSNorm
        self.final_norm = RMSNorm(self.hidden_size, eps=config.rms_norm_eps)
        self.reset_parameters()

    def reset_parameters(self):
        # same order as the reference (:279-289) so a seed gives the same weights
        self.embedding.reset_parameters()
        for layer in self.decoder_layers:
            layer.input_layernorm.reset_parameters()
            layer.attention.reset_parameters()
            layer.post_attention_layernorm.reset_parameters()
            layer.mlp.reset_parameters()
        self.final_norm.reset_parameters()
        self.final_proj.reset_parameters()

    def set_cp_rank(self, cp_rank: int) -> None:
        """Re-slice every layer's RoPE tables for another virtual cp rank (the reference builds one model per
        process, so its slice is fixed at construction, :228)."""
        mgr = pgm.process_group_manager
        mgr.set_cp_rank(cp_rank)
        for layer in self.decoder_layers:
            head_dim = self.hidden_size // self.num_heads
            if not hasattr(layer, "_full_tables"):
                layer._full_tables = get_cos_sin(self.max_position_embeddings, head_dim=head_dim,
                                                 base=self.model_config.rope_theta)
            layer.cos, layer.sin = context_parallel.update_rope_for_context_parallel(*layer._full_tables)

    def forward(self, input_ids, attention_mask=None, position_ids: torch.Tensor = None):
        x = self.embedding(input_ids)
        if _fused_residual() and isinstance(self.final_norm, TritonRMSNorm) and all(
                isinstance(l.input_layernorm, TritonRMSNorm) for l in self.decoder_layers):
            residual = None
            for layer in self.decoder_layers:
                x, residual = layer.forward_chained(x, residual)
            x = self.final_norm(x, residual=residual)
        else:
            for layer in self.decoder_layers:
                x = layer(x)
            x = self.final_norm(x)
        return self.final_proj(x)
