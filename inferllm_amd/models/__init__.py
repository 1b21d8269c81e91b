from . import kukupel, llama, rabapel  # registers Kukupel, LlamaForCausalLM and Rabapel

__all__ = ["kukupel", "llama", "rabapel"]
