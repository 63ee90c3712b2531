from .loader import WeightsError, build_model, expected_tensors, load_model, load_weights
from .random_init import fill_random, random_tensors, write_random_model
from .safetensors_io import SafetensorsFile, list_safetensors, write_safetensors
