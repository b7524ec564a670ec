"""A small MI355X-native inference engine for decoder models built from parts; the
architecture it ships is the Qwen3 dense decoder."""
from .api import LLM, generate
from .config import ConfigError, Qwen3Config, load_config, register_architecture
from .parts import DecoderModel, register_part
from .weights import WeightError, write_random_model

__all__ = ["LLM", "generate", "ConfigError", "Qwen3Config", "load_config", "register_architecture", "DecoderModel",
           "register_part", "WeightError", "write_random_model"]
