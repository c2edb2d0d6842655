from .binding import WeightBindingError, WeightSpec, bind_weights, stored_to_resident
from .safetensors_io import (ModelFiles, SafetensorsError, SafetensorsFile, TensorDict,
                             write_safetensors)
from .random_init import random_tensors, write_random_model

__all__ = ["WeightBindingError", "WeightSpec", "bind_weights", "stored_to_resident", "ModelFiles",
           "SafetensorsError", "SafetensorsFile", "TensorDict", "write_safetensors",
           "random_tensors", "write_random_model"]
