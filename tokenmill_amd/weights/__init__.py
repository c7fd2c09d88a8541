from tokenmill_amd.weights.loader import TensorSpec, WeightsError, read_checkpoint
from tokenmill_amd.weights.random_init import random_tensors, write_random_model

__all__ = ["TensorSpec", "WeightsError", "read_checkpoint", "random_tensors", "write_random_model"]
