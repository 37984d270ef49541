from .safetensors_io import SafetensorsFile, SafetensorsError, write_safetensors
from .loader import TensorSpec, WeightError, open_folder, check_against, load_folder
from .random_init import random_tensors, write_model_folder
