from .loader import Checkpoint, TensorDict, WeightsError, check, load_tensors, target_dtype
from .random_init import random_tensors, write_random_model
