"""CPU oracle for the paged-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this
module; it is used by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported CPU baseline.
"""
from .attention_oracle import (  # noqa: F401
    store_kvcache_oracle,
    quantize_int8_oracle,
    store_kvcache_int8_oracle,
    dequantize_cache_oracle,
    decode_naive_oracle,
    decode_vectorised_oracle,
    decode_int8_oracle,
    prefill_standard_oracle,
    prefill_paged_oracle,
    gather_sequence_kv,
    rms_norm_oracle,
    rope_cos_sin_cache_oracle,
    rope_oracle,
    qk_norm_rope_store_oracle,
    add_rms_norm_oracle,
    silu_and_mul_oracle,
)
from .producers_oracle import (  # noqa: F401
    prefill_metadata_oracle,
    decode_metadata_oracle,
)
from .sampler_oracle import (  # noqa: F401
    philox4x32_10_oracle,
    exponential_noise_oracle,
    sampler_oracle,
)
