from .loader import held_dtype, load_tensors, random_tensors, write_model_folder
from .safetensors_io import SafetensorsFile, open_model_files, write_safetensors
