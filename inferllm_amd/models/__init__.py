from . import kukupel, llama, rabapel, sabipel  # registers Kukupel, LlamaForCausalLM, Rabapel and Sabipel

__all__ = ["kukupel", "llama", "rabapel", "sabipel"]
