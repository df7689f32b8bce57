"""Small Llama / Qwen3 / GPT-2 module trees with the reference's attribute names,
so that the Linear swap is exercised on the structures it will meet."""
from .families import GPT2, GPT2Config, Llama, LlamaConfig, Qwen3, Qwen3Config

__all__ = ["GPT2", "GPT2Config", "Llama", "LlamaConfig", "Qwen3", "Qwen3Config"]
