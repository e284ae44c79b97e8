from .spec import TensorSpec
from .safetensors_io import Checkpoint, SafetensorsFile, SafetensorsError, write_safetensors
from .loader import WeightsError, load_tensors, bind_tensors, check_tensors, engine_dtype, convert_for_engine
from .random_init import random_tensors, random_tensor, write_model_folder
