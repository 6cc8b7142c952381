from .loader import (WeightError, load_weights, random_tensor, storage_dtype, tensor_seed,
                     write_random_model)
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, write_safetensors
