from .sampler import Sampler, draw_key

__all__ = ["Sampler", "draw_key"]
