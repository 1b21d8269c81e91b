from . import llama, rabapel  # registers LlamaForCausalLM and Rabapel

__all__ = ["llama", "rabapel"]
