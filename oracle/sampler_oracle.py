"""CPU restatement of the reference's sampler and of the counter-based noise the HIP sampler draws.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

* ``sampler_oracle``            src/myvllm/layers/sampler.py:14-19, with the noise passed in instead of drawn.
                                Pinned by its distribution: over many independent noise tensors the frequency of
                                each token approaches softmax(logits / T) (tests/test_oracle_pins.py).
* ``philox4x32_10_oracle``      Philox4x32-10 of Salmon et al., "Parallel random numbers: as easy as 1, 2, 3"
                                (SC'11); the reference has no counterpart (torch draws its noise).  Pinned by the
                                known-answer vectors published with the Random123 library.
* ``exponential_noise_oracle``  the Exp(1) tensor the kernel generates for (seed, offset): counter
                                (i // 4, b, offset_lo, offset_hi), key (seed_lo, seed_hi), word i % 4,
                                u = ((x >> 8) + 0.5) * 2^-24, E = -log(u).  Pinned by mean / variance / range.
"""
from __future__ import annotations

import numpy as np
import torch

_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10_oracle(counters: np.ndarray, key) -> np.ndarray:
    """counters: uint32 [N, 4]; key: two uint32.  Returns uint32 [N, 4]."""
    c = [counters[:, i].astype(np.uint64) for i in range(4)]
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = _M0 * c[0]
        p1 = _M1 * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & _MASK
        hi1, lo1 = p1 >> np.uint64(32), p1 & _MASK
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0 = (k0 + _W0) & 0xFFFFFFFF
        k1 = (k1 + _W1) & 0xFFFFFFFF
    return np.stack(c, axis=1).astype(np.uint32)


def exponential_noise_oracle(seed: int, offset: int, batch: int, vocab: int) -> torch.Tensor:
    groups = (vocab + 3) // 4
    gi, b = np.meshgrid(np.arange(groups, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
    ctr = np.stack([gi.ravel(), b.ravel(),
                    np.full(gi.size, offset & 0xFFFFFFFF, dtype=np.uint32),
                    np.full(gi.size, (offset >> 32) & 0xFFFFFFFF, dtype=np.uint32)], axis=1)
    words = philox4x32_10_oracle(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    u = ((words >> np.uint32(8)).astype(np.float32) + np.float32(0.5)) * np.float32(2.0 ** -24)
    e = -np.log(u.astype(np.float32))
    return torch.from_numpy(e.reshape(batch, groups * 4)[:, :vocab].astype(np.float32).copy())


def sampler_oracle(logits: torch.Tensor, temperatures: torch.Tensor, noise: torch.Tensor) -> torch.Tensor:
    """logits / T -> softmax -> divide by the Exp(1) noise clamped at 1e-10 -> argmax (sampler.py:15-18)."""
    scaled = logits.float() / temperatures.float().unsqueeze(-1)
    probs = torch.softmax(scaled, dim=-1)
    return probs.div(noise.float().clamp_min(1e-10)).argmax(dim=-1)
