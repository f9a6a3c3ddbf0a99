from ..spec import ModelSpec, LayerSpec, PartSpec, TensorNeed, PagedKVNeed, StateNeed
from .model import Model
from . import qwen3  # noqa: F401  (registers the architecture)
