"""The models wired from the shared decoder: Llama and Granite."""

from .granite import Granite, GraniteConfig
from .llama import Llama, LlamaConfig

__all__ = ["Granite", "GraniteConfig", "Llama", "LlamaConfig"]
