from .loader import GAIN, MATRIX, TABLE, TensorSpec, check_folder, load_checked
from .random_init import random_tensor, random_tensors, write_random_model
from .safetensors_io import ModelFolder, SafeTensorFile, save_file

__all__ = ["GAIN", "MATRIX", "TABLE", "TensorSpec", "check_folder", "load_checked", "random_tensor",
           "random_tensors", "write_random_model", "ModelFolder", "SafeTensorFile", "save_file"]
