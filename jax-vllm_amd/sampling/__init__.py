from .keys import draw_key

__all__ = ["Sampler", "draw_key"]


def __getattr__(name):
    if name == "Sampler":  # pulls in torch and the kernels
        from .sampler import Sampler

        return Sampler
    raise AttributeError(name)
