from .loader import Expect, Float16Narrowed, WeightError, WeightSource, bind
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["Expect", "Float16Narrowed", "SafetensorsError", "SafetensorsFile", "WeightError", "WeightSource", "bind",
           "write_safetensors"]
