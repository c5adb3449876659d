from .loader import check_tensors, load_tensors  # noqa: F401
from .random_init import random_tensors, write_random_model  # noqa: F401
from .safetensors_io import SafetensorsFile, open_model_files, write_safetensors  # noqa: F401
