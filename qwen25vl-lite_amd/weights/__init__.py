from .loader import WeightsError, kept_dtype, load_weights
from .random_init import fill_random, random_tensors, write_random_model
from .safetensors_io import SafetensorsFile, checkpoint_shards, write_safetensors

__all__ = ["WeightsError", "kept_dtype", "load_weights", "fill_random", "random_tensors", "write_random_model",
           "SafetensorsFile", "checkpoint_shards", "write_safetensors"]
