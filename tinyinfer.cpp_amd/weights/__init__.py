from .loader import load_weights, WeightsError
from ..native import FileError


def write_model_folder(*args, **kwargs):
    """A random-weights model folder from a config and a seed (weights/random_init.py, which is
    also a command: `python -m tinyinfer_amd.weights.random_init`; it is imported at the call, so
    that running it as a command does not find it imported already)."""
    from .random_init import write_model_folder as write
    return write(*args, **kwargs)
