from .loader import (DictSource, SafetensorsFolder, TensorSource, WeightError, expected_tensors, load_model_folder,
                     load_weights)
from .random_init import RandomSource, random_state_dict, write_random_model

__all__ = ["DictSource", "SafetensorsFolder", "TensorSource", "WeightError", "expected_tensors",
           "load_model_folder", "load_weights", "RandomSource", "random_state_dict", "write_random_model"]
