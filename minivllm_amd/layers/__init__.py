from .attention import (  # noqa: F401
    Attention,
    flash_attention_prefill,
    paged_attention_decode,
    paged_attention_decode_int8,
    store_kvcache,
    store_kvcache_int8,
)
