from . import qwen2  # registers Qwen2ForCausalLM

__all__ = ["qwen2"]
