from tensorline_amd.weights.loader import WeightError, load_checkpoint, load_from_getter  # noqa: F401
from tensorline_amd.weights.random_init import random_tensor, write_random_model  # noqa: F401
