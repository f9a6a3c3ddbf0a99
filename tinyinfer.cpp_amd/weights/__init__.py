from .loader import load_weights, WeightsError
from .random_init import random_tensors, write_model_folder
from .safetensors_io import SafetensorsFile, write_safetensors, open_model_files, SafetensorsError
