from . import dafutar, katenex, qwen2, sozavik  # register Dafutar, Katenex, Qwen2ForCausalLM and Sozavik

__all__ = ["dafutar", "katenex", "qwen2", "sozavik"]
