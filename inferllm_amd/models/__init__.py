from . import dotorax, kukupel, llama, rabapel, sabipel  # registers Dotorax, Kukupel, LlamaForCausalLM, Rabapel and Sabipel

__all__ = ["dotorax", "kukupel", "llama", "rabapel", "sabipel"]
