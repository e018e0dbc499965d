from .source import DeviceTensors, DictSource, SafetensorsSource, TensorSource, storage_dtype
from .loader import WeightError, check_tensors, open_model_folder
from .random_init import random_tensor, random_tensors, write_model_folder
