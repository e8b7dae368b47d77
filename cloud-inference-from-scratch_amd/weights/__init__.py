from .loader import (
    INIT_STD,
    RandomSource,
    SafetensorsSource,
    WeightError,
    torch_dtype,
    write_model_folder,
    write_tensors,
)
from .tensors import TensorSpec

__all__ = [
    "INIT_STD", "RandomSource", "SafetensorsSource", "TensorSpec", "WeightError",
    "torch_dtype", "write_model_folder", "write_tensors",
]
