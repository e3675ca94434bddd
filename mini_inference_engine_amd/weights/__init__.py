from .loader import CheckpointFiles, WeightError, load_weights, storage_dtype
from .random_init import random_tensors, write_random_model
