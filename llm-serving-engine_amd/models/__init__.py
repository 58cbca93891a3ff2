from . import dafutar, qwen2  # register Dafutar and Qwen2ForCausalLM

__all__ = ["dafutar", "qwen2"]
