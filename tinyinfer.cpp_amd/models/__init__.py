from ..spec import ModelSpec, LayerSpec, PartSpec, TensorNeed, PagedKVNeed, StateNeed
from .model import Model
