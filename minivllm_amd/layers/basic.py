"""Counterparts of the reference's small layers around the attention path, as chains of PyTorch-ROCm tensor
operations and, with ``fused=True``, as single HIP launches (minivllm_amd.layers.fused): RMSNorm with fused residual (layers/layernorm.py:9-28), NeoX half-split RoPE
(layers/rotary_embedding.py:4-83), SiluAndMul (layers/activation.py:15-18) and the temperature /
exponential-race sampler (layers/sampler.py:14-19)."""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from minivllm_amd.layers.fused import add_rms_norm, linear_small_m, linear_small_m_takes, silu_and_mul


class Linear(nn.Linear):
    """``nn.Linear`` (layers/linear.py) whose calls with at most ``small_rows`` rows (a decode step) run as one HIP
    launch built for that size (``linear_small_m``); everything else, prefill included, is the library GEMM."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, small_rows: int = 0):
        super().__init__(in_features, out_features, bias=bias)
        self.small_rows = small_rows

    def forward(self, x):
        if self.small_rows and linear_small_m_takes(x, self.weight, self.small_rows):
            return linear_small_m(x, self.weight, self.bias)
        return F.linear(x, self.weight, self.bias)


class RMSNorm(nn.Module):
    """x / sqrt(mean(x^2) + eps) * weight over the last dim, optionally after adding a residual
    (layers/layernorm.py:9-28).  ``fused=True`` runs it as one HIP launch (``add_rms_norm``), otherwise as the
    chain of tensor operations; both round where the chain rounds."""

    def __init__(self, size: int, eps: float = 1e-6, fused: bool = False):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(size))
        self.eps = eps
        self.fused = fused
        self._w32 = None

    def weight_fp32(self):
        """float32 copy of the weight for the HIP kernels (made once; weights do not change while serving)."""
        if self._w32 is None or self._w32.device != self.weight.device:
            self._w32 = self.weight.detach().float().contiguous()
        return self._w32

    def _norm(self, x):
        xf = x.float()
        xf = xf / torch.sqrt(xf.pow(2).mean(dim=-1, keepdim=True) + self.eps)
        return (xf * self.weight.float()).to(x.dtype)

    def forward(self, x, residual=None):
        if self.fused and x.dim() == 2:
            return add_rms_norm(x, self.weight_fp32(), self.eps, residual)
        if residual is None:
            return self._norm(x)
        x = x + residual
        return self._norm(x), x


class RotaryEmbedding(nn.Module):
    def __init__(self, base: float, rotary_dim: int, max_position: int):
        super().__init__()
        self.base, self.rotary_dim, self.max_position = base, rotary_dim, max_position
        self.register_buffer("cos_sin_cache", self._table(), persistent=False)

    def _table(self):
        inv_freq = 1.0 / (self.base ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim))
        freqs = torch.outer(torch.arange(self.max_position, dtype=torch.float32), inv_freq)
        return torch.cat([freqs.cos(), freqs.sin()], dim=-1)

    def _apply(self, fn, recurse=True):
        # the table stays float32 whatever dtype the model is cast to (rotary_embedding.py:61-70 builds it
        # from float positions): rebuild it on the device the cast left it on
        super()._apply(fn, recurse)
        self.cos_sin_cache = self._table().to(self.cos_sin_cache.device)
        return self

    @staticmethod
    def _rotate(x, cos, sin):
        x1, x2 = x.float().chunk(2, dim=-1)
        return torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).to(x.dtype)

    def forward(self, positions, query, key):
        cos, sin = self.cos_sin_cache[positions].chunk(2, dim=-1)      # (T, D/2) each, fp32
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
        return self._rotate(query, cos, sin), self._rotate(key, cos, sin)


class SiluAndMul(nn.Module):
    def __init__(self, fused: bool = False):
        super().__init__()
        self.fused = fused

    def forward(self, x):
        if self.fused and x.dim() == 2:
            return silu_and_mul(x)
        a, b = x.chunk(2, dim=-1)
        return F.silu(a) * b


class Sampler(nn.Module):
    """argmax(softmax(logits / T) / E), E ~ Exp(1): one draw from the tempered distribution."""

    def forward(self, logits, temperatures, generator=None):
        probs = torch.softmax(logits.float() / temperatures.unsqueeze(-1), dim=-1)
        noise = torch.empty_like(probs).exponential_(1.0, generator=generator).clamp_min_(1e-10)
        return probs.div_(noise).argmax(dim=-1)
