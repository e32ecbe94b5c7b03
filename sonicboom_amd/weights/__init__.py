from .loader import LazyTensors, WeightError, check_against_spec, load_tensors, open_tensors  # noqa: F401
from .random_init import random_arrays, random_source, random_tensors, write_random_model  # noqa: F401
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors  # noqa: F401
