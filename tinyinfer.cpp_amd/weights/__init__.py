from .loader import load_weights, WeightsError
from .random_init import write_model_folder
from ..native import FileError
