from .loader import FolderSource, TensorWant, WeightError, check_names_and_shapes, load_tensors
from .random_init import RandomSource, parse_shape, random_model_folder, write_model_folder
from .safetensors_io import read_folder_header, read_header, write_file

__all__ = [
    "FolderSource",
    "RandomSource",
    "TensorWant",
    "WeightError",
    "check_names_and_shapes",
    "load_tensors",
    "parse_shape",
    "random_model_folder",
    "read_folder_header",
    "read_header",
    "write_file",
    "write_model_folder",
]
