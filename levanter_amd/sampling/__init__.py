from .sampler import Sampler, fold_in, make_key

__all__ = ["Sampler", "fold_in", "make_key"]
