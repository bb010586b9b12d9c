from .safetensors_io import SafetensorsFile, SafetensorsError, write_safetensors
from .loader import (Checkpoint, WeightError, check_tensors, load_config, load_model,
                     read_config, keep_dtype)
from .random_init import RandomCheckpoint, random_tensors, write_random_model
