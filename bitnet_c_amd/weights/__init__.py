from .loader import TensorSource, TensorSpec, WeightError, load_tensors, open_tensors
from .random_init import random_tensors, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, write_file
