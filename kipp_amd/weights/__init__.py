from .loader import WeightError, check_tensors, read_model_tensors
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, read_file, write_file
