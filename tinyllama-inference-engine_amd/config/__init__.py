from .llama import LlamaConfig, read_config_json
from .spec import LayerSpec, ModelSpec, PartSpec, Run, TensorSpec

__all__ = ["LlamaConfig", "read_config_json", "LayerSpec", "ModelSpec", "PartSpec", "Run", "TensorSpec"]
