from .random_init import RandomSource, load_random_model, random_tensors, write_random_model
from .reader import CheckpointReader, WeightsError, place
from .spec import TensorSpec

__all__ = ["CheckpointReader", "WeightsError", "TensorSpec", "place", "random_tensors", "write_random_model",
           "RandomSource", "load_random_model"]
