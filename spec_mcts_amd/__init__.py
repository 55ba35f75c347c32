"""MI355X-native Q4_0 CodeLlama hot path with the Python model API of hongyihuang/spec-mcts."""
from .hf_model_q40_kv_shared import ModelArgs, Transformer, LinearQ4_0  # noqa: F401
from .load_q40 import load_q40  # noqa: F401

__all__ = ["ModelArgs", "Transformer", "LinearQ4_0", "load_q40"]
