from .arena import ResidentWeights, WeightArena, keep_in
from .random_init import random_tensors, resident_random_tensors, write_random_model
from .safetensors_io import SafetensorsFile, write_safetensors
from .store import WeightStore, to_kept_precision

__all__ = ["ResidentWeights", "WeightArena", "keep_in", "random_tensors", "resident_random_tensors", "write_random_model", "SafetensorsFile", "write_safetensors", "WeightStore",
           "to_kept_precision"]
