from .loader import WeightError, WeightSpec, load_weights, storage_dtype
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_folder, shard_files, write_file
