from .loader import (INTEGER, MATRIX, TABLE, VECTOR, ParamSpec, WeightError, WeightSource,
                     load_parameters, target_dtype)
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = [
    "INTEGER", "MATRIX", "TABLE", "VECTOR", "ParamSpec", "SafetensorsError", "SafetensorsFile",
    "WeightError", "WeightSource", "load_parameters", "target_dtype", "write_safetensors",
]
