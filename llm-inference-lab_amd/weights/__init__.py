from .safetensors_io import SafetensorsFile, ModelFiles, save_safetensors
from .loader import (TensorSpec, MATRIX, VECTOR, INT_TABLE, INIT_NORMAL, INIT_NORM, INIT_ZEROS, INIT_ONES,
                     kept_dtype, load_tensors, place_tensors, check_names_and_shapes)
from .random_init import random_tensors, write_model_dir
