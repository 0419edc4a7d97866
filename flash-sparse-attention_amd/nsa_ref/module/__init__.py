from .rope import RopeConfig, RotaryEmbedding

__all__ = ["RopeConfig", "RotaryEmbedding"]
