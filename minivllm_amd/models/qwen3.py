"""Qwen3-style decoder used as the caller of the attention path (src/myvllm/models/qwen3.py).

Single-GPU PyTorch-ROCm: the projections are plain ``F.linear`` (hipBLASLt); the only custom kernels
are behind ``minivllm_amd.layers.attention.Attention``.  Shapes follow the intended semantics where the
reference's own do not work: the QKV projection maps ``hidden_size`` (not ``num_heads*head_dim``,
qwen3.py:37-43) to ``(Hq + 2 Hkv) * D``; ``rms_norm_epsilon`` is honoured (the reference accepts and drops
it); ``Attention`` receives the engine's ``block_size``; weights are seeded N(0, 0.02) instead of
uninitialised memory.  Positions are computed once per step by the model runner, not per layer.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from minivllm_amd.layers.attention import Attention
from minivllm_amd.layers.basic import Linear, RMSNorm, RotaryEmbedding, SiluAndMul
from minivllm_amd.layers.fused import norm_linear_small_m, norm_linear_small_m_takes
from minivllm_amd.utils.context import get_context


class Qwen3Attention(nn.Module):
    def __init__(self, hidden_size, num_heads, head_dim, scale, num_kv_heads, rms_norm_epsilon, qkv_bias,
                 rotary: RotaryEmbedding, block_size, kv_cache_dtype, fused_qk=True, small_rows=0):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.q_size, self.kv_size = num_heads * head_dim, num_kv_heads * head_dim
        self.qkv_projection = Linear(hidden_size, self.q_size + 2 * self.kv_size, bias=qkv_bias, small_rows=small_rows)
        self.qkv_bias = qkv_bias
        self.rms_norm = RMSNorm(head_dim, rms_norm_epsilon)      # one gamma shared by q and k (qwen3.py:50, 104-106)
        self.rotary_emb = rotary
        self.attention = Attention(num_heads, head_dim, scale, num_kv_heads, block_size, kv_cache_dtype)
        self.output_projection = Linear(self.q_size, hidden_size, bias=False, small_rows=small_rows)
        self.fused_qk = fused_qk

    def forward(self, x, positions):
        return self.forward_qkv(self.qkv_projection(x), positions)

    def forward_qkv(self, qkv, positions):
        """Everything after the QKV projection (whose output a caller may have produced fused with the norm)."""
        q, k, v = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
        if self.fused_qk:
            # views of the projection output, no copies; norm + rotation + cache store in one launch
            q = q.unflatten(-1, (self.num_heads, self.head_dim))
            k = k.unflatten(-1, (self.num_kv_heads, self.head_dim))
            v = v.unflatten(-1, (self.num_kv_heads, self.head_dim))
            gamma = None if self.qkv_bias else self.rms_norm.weight_fp32()
            o = self.attention.forward_fused(q, k, v, positions, self.rotary_emb.cos_sin_cache, gamma,
                                             self.rms_norm.eps)
            return self.output_projection(o)
        q = q.reshape(-1, self.num_heads, self.head_dim)
        k = k.reshape(-1, self.num_kv_heads, self.head_dim)
        v = v.reshape(-1, self.num_kv_heads, self.head_dim)
        if not self.qkv_bias:
            q, k = self.rms_norm(q), self.rms_norm(k)
        q, k = self.rotary_emb(positions, q, k)
        return self.output_projection(self.attention(q, k, v))


class Qwen3MLP(nn.Module):
    def __init__(self, hidden_size, intermediate_size, bias, fused=True, small_rows=0):
        super().__init__()
        self.gate_up = Linear(hidden_size, 2 * intermediate_size, bias=bias, small_rows=small_rows)
        self.activation = SiluAndMul(fused)
        self.gate_down = Linear(intermediate_size, hidden_size, bias=bias, small_rows=small_rows)
        self.small_rows, self.fused = small_rows, fused

    def forward(self, x):
        # a decode step's rows: SiluAndMul as the epilogue of the gate/up projection (one launch instead of two)
        if (self.small_rows and self.fused and x.dim() == 2 and x.shape[0] <= self.small_rows and x.is_contiguous()
                and norm_linear_small_m_takes(x, self.gate_up.weight, self.small_rows, norm=False, glu=True)):
            return self.gate_down(norm_linear_small_m(x, self.gate_up.weight, self.gate_up.bias, glu=True))
        return self.gate_down(self.activation(self.gate_up(x)))


class Qwen3DecoderLayer(nn.Module):
    def __init__(self, hidden_size, intermediate_size, ffn_bias, rms_norm_epsilon, fused_elementwise=True,
                 small_rows=0, norm_rows=32, **attn_kwargs):
        super().__init__()
        self.input_layernorm = RMSNorm(hidden_size, rms_norm_epsilon, fused_elementwise)
        self.self_attn = Qwen3Attention(hidden_size=hidden_size, rms_norm_epsilon=rms_norm_epsilon,
                                        small_rows=small_rows, **attn_kwargs)
        self.post_attention_layernorm = RMSNorm(hidden_size, rms_norm_epsilon, fused_elementwise)
        self.mlp = Qwen3MLP(hidden_size, intermediate_size, ffn_bias, fused_elementwise, small_rows)
        # the norm prologue normalises a workgroup's rows once per column tile: it pays up to about 32 rows
        self.norm_rows, self.fused_elementwise = min(small_rows, norm_rows), fused_elementwise

    def _forward_few_rows(self, x, residual, positions):
        """A decode step's few rows: the two residual norms run as the prologues of the projections that follow them
        and SiluAndMul as the epilogue of the gate/up projection (``norm_linear_small_m``): 6 launches per layer
        instead of 9, same roundings."""
        attn, mlp = self.self_attn, self.mlp
        ln1, ln2 = self.input_layernorm, self.post_attention_layernorm
        proj = attn.qkv_projection
        if residual is None:
            qkv = norm_linear_small_m(x, proj.weight, proj.bias, ln1.weight_fp32(), ln1.eps)
            residual = x
        else:
            qkv, residual = norm_linear_small_m(x, proj.weight, proj.bias, ln1.weight_fp32(), ln1.eps, residual, True)
        x = attn.forward_qkv(qkv, positions)
        act, residual = norm_linear_small_m(x, mlp.gate_up.weight, mlp.gate_up.bias, ln2.weight_fp32(), ln2.eps,
                                            residual, True, glu=True)
        return mlp.gate_down(act), residual

    def forward(self, x, residual, positions):
        rows = self.norm_rows
        if (rows and self.fused_elementwise and x.dim() == 2 and x.shape[0] <= rows and x.is_contiguous()
                and norm_linear_small_m_takes(x, self.self_attn.qkv_projection.weight, rows)
                and norm_linear_small_m_takes(x, self.mlp.gate_up.weight, rows, glu=True)):
            return self._forward_few_rows(x, residual, positions)
        if residual is None:
            residual = x
            x = self.input_layernorm(x)
        else:
            x, residual = self.input_layernorm(x, residual)
        x = self.self_attn(x, positions)
        x, residual = self.post_attention_layernorm(x, residual)
        return self.mlp(x), residual


class Qwen3ForCausalLM(nn.Module):
    def __init__(self, vocab_size, hidden_size, num_heads, head_dim=None, scale=1.0, num_kv_heads=None,
                 rms_norm_epsilon=1e-6, qkv_bias=False, base=1_000_000, max_position=4096,
                 intermediate_size=3072, ffn_bias=True, num_layers=8, tie_word_embeddings=True,
                 block_size=256, kv_cache_dtype="auto", fused_qk=True, fused_elementwise=True, small_rows=0,
                 norm_rows=32):
        super().__init__()
        head_dim = head_dim if head_dim is not None else hidden_size // num_heads
        num_kv_heads = num_kv_heads if num_kv_heads is not None else num_heads
        self.embedding_layer = nn.Embedding(vocab_size, hidden_size)
        rotary = RotaryEmbedding(base, head_dim, max_position)
        self.layer_stack = nn.ModuleList([
            Qwen3DecoderLayer(hidden_size, intermediate_size, ffn_bias, rms_norm_epsilon, num_heads=num_heads,
                              head_dim=head_dim, scale=scale, num_kv_heads=num_kv_heads, qkv_bias=qkv_bias,
                              rotary=rotary, block_size=block_size, kv_cache_dtype=kv_cache_dtype,
                              fused_qk=fused_qk, fused_elementwise=fused_elementwise, small_rows=small_rows,
                              norm_rows=norm_rows)
            for _ in range(num_layers)])
        self.final_layernorm = RMSNorm(hidden_size, rms_norm_epsilon, fused_elementwise)
        self.lm_head_weight = self.embedding_layer.weight if tie_word_embeddings else nn.Parameter(
            torch.empty(vocab_size, hidden_size))
        self.max_position = max_position

    def reset_parameters(self, seed: int = 0, std: float = 0.02):
        g = torch.Generator(device="cpu").manual_seed(seed)
        with torch.no_grad():
            for name, p in self.named_parameters():
                if p.dim() >= 2:
                    p.copy_(torch.randn(p.shape, generator=g) * std)
                elif name.endswith("bias"):
                    p.zero_()
                else:
                    p.fill_(1.0)

    def forward(self, input_ids, positions):
        # a decode step's few rows by plain indexing: the embedding operator's small-batch kernel takes 11 us for 16
        # rows, the gather 4
        x = self.embedding_layer.weight[input_ids] if input_ids.numel() <= 256 else self.embedding_layer(input_ids)
        residual = None
        for layer in self.layer_stack:
            x, residual = layer(x, residual, positions)
        x, _ = self.final_layernorm(x, residual)
        return x

    def compute_logits(self, hidden):
        context = get_context()
        if context.is_prefill:                         # last token of every packed sequence (embedding_head.py:57-62)
            hidden = hidden[(context.cu_seqlens_q[1:] - 1).long()].contiguous()
        return F.linear(hidden, self.lm_head_weight)
