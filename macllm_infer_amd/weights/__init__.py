from .loader import Expect, WeightError, WeightSource, bind
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["Expect", "SafetensorsError", "SafetensorsFile", "WeightError", "WeightSource", "bind",
           "write_safetensors"]
