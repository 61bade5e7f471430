from .loader import WeightError, load_weights, checkpoint_layout
from .random_weights import write_random_model, random_checkpoint, fill_random_

__all__ = ["WeightError", "load_weights", "checkpoint_layout", "write_random_model", "random_checkpoint",
           "fill_random_"]
