from .safetensors_io import SafetensorsFile, SafetensorsError, save_file, open_model_files
from .loader import (Checkpoint, WeightLoadError, load_weights, init_random_weights, write_random_model, random_tensor,
                     check_against, target_dtype)
