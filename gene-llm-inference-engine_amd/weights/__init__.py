"""Safetensors reading and writing, binding by name, random weights."""
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors
from .loader import TensorNeed, WeightsError, load_tensors, merge_needs
from .random_init import formula_tensors, formula_values, random_tensors, tensor_key, write_random_model
