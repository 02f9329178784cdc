"""The models wired from the shared decoder: Llama, Granite and Gemma 4's text decoder."""

from .gemma4 import Gemma4, Gemma4Config
from .granite import Granite, GraniteConfig
from .llama import Llama, LlamaConfig

__all__ = ["Gemma4", "Gemma4Config", "Granite", "GraniteConfig", "Llama", "LlamaConfig"]
