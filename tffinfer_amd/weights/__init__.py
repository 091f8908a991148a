from .loader import WeightError, check_weights, normalize_stored
from .random_init import random_tensor, write_random_model
from .safetensors_io import WeightFileError, load_file, load_model_dir, save_file
