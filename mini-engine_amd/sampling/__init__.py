from .sampler import Sampler, draw_key, mix64

__all__ = ["Sampler", "draw_key", "mix64"]
