from .loader import WeightsError, load_folder, place_all
from .random_init import InitRule, random_tensors, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, save_file

__all__ = ["WeightsError", "load_folder", "place_all", "InitRule", "random_tensors", "write_model_folder",
           "SafetensorsError", "SafetensorsFile", "open_model_files", "save_file"]
