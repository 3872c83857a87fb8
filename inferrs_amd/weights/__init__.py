from .safetensors_io import SafetensorsError, SafetensorsFile, weight_files, write_safetensors
from .loader import TensorSpec, WeightError, load_weights
from .random_init import random_tensors, write_random_model
