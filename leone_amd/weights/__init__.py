from .loader import (INT_TABLE, MATRIX, VECTOR, TensorSpec, WeightsError, load_from_dir, load_from_tensors)
from .safetensors_io import ModelFiles, SafetensorsError, write_file
