from atomserve_amd.weights.loader import Stack, Take, WeightsError, bind_checkpoint, load_model, load_weights
from atomserve_amd.weights.random_init import random_checkpoint, write_random_model

__all__ = ["Stack", "Take", "WeightsError", "bind_checkpoint", "load_model", "load_weights", "random_checkpoint",
           "write_random_model"]  # fmt: skip
