from tokasaurus_amd.weights.loader import WeightError, read_tensors  # noqa: F401
from tokasaurus_amd.weights.random_init import draw_tensors, write_random_model  # noqa: F401
