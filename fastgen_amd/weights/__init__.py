from .folder import write_model_folder
from .source import (
    DictSource,
    RandomSource,
    SafetensorsSource,
    TensorSource,
    WeightError,
    check_against_specs,
    safetensors_files,
)

__all__ = [
    "DictSource", "RandomSource", "SafetensorsSource", "TensorSource", "WeightError",
    "check_against_specs", "safetensors_files", "write_model_folder",
]
