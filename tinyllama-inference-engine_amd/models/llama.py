"""Registers the Llama dense decoder: the name in config.json -> its configuration class."""
from ..config.llama import LlamaConfig
from ..registry import register

register("architecture", "LlamaForCausalLM")(LlamaConfig)
