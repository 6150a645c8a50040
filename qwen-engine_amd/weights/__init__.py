from .loader import WeightError, read_checked, safetensors_files
from .random_init import random_tensors, write_model_folder
