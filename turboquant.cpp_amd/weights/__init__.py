from .loader import Binding, TensorDict, WeightError, check, expected_tensors, load_bindings, stored_dtype
from .random_init import random_tensor, random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFolder, SafetensorsWriter, write_safetensors
