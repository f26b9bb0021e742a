from .loader import ParamSpec, TensorSource, WeightsError
from .random_init import write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_file

__all__ = ["ParamSpec", "TensorSource", "WeightsError", "write_random_model", "SafetensorsError", "SafetensorsFile",
           "write_file"]
