from .safetensors_io import SafetensorsError, SafetensorsFile, resolve_shards, save_file
from .source import TensorSpec, WeightSource, FolderSource, DictSource, RandomSource, tensor_seed
from .loader import WeightError, check_source, load_weights, kept_dtype
from .random_init import write_random_model

__all__ = ["SafetensorsError", "SafetensorsFile", "resolve_shards", "save_file", "TensorSpec", "WeightSource",
           "FolderSource", "DictSource", "RandomSource", "tensor_seed", "WeightError", "check_source",
           "load_weights", "kept_dtype", "write_random_model"]
