from ..spec import ModelSpec, LayerSpec, PartSpec, TensorNeed, PagedKVNeed, PagedRowsNeed, StateNeed
from .model import Model
