"""minivllm_amd: MI355X (gfx950) implementation of a MinivLLM-style paged-attention path.

Public surface mirrors the reference package layout:
``minivllm_amd.utils`` (Context), ``minivllm_amd.layers.attention`` (operators),
``minivllm_amd.engine`` (metadata producers, scheduler, block manager).
"""
__version__ = "0.1.0"
