from . import dafutar, katenex, qwen2, sozavik, vagozen  # register Dafutar, Katenex, Qwen2ForCausalLM, Sozavik and Vagozen

__all__ = ["dafutar", "katenex", "qwen2", "sozavik", "vagozen"]
