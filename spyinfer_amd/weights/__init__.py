from .loader import WeightError, WeightSpec, load_weights, storage_dtype
from .random_init import random_tensors, random_tensors_on_device, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_folder, shard_files, write_file
