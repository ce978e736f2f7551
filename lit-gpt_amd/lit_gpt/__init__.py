"""MI355X-native decode path behind the lit_gpt API (reference lit_gpt/__init__.py:27)."""

from lit_gpt.config import Config, LayeredConfig, load_config, model_class

__all__ = ["GPT", "Config", "LayeredConfig", "LayeredGPT", "Tokenizer", "load_config", "model_class"]


def __getattr__(name):
    if name == "GPT":
        from lit_gpt.model import GPT

        return GPT
    if name == "LayeredGPT":
        from lit_gpt.layered import LayeredGPT

        return LayeredGPT
    if name == "Tokenizer":
        from lit_gpt.tokenizer import Tokenizer

        return Tokenizer
    raise AttributeError(name)
