from .loader import WeightError, load_weights
from .random_init import load_random_weights, random_tensor, random_tensors, write_random_model
