from .qwen3 import Qwen3ForCausalLM  # noqa: F401
