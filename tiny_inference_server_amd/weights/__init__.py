from .loader import WeightError, check_names_and_shapes, load_tensors, spec_tensors
from .random_init import random_tensors, write_random_model
