from . import dafutar, qwen2, sozavik  # register Dafutar, Qwen2ForCausalLM and Sozavik

__all__ = ["dafutar", "qwen2", "sozavik"]
