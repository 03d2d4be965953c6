from .loader import WeightError, check_against, load_weights
from .random_init import random_tensors, random_weights_on_device, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_tensors, write_safetensors
