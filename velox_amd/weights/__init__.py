from .loader import WeightsError, bind_from_checkpoint, held_dtype, list_weight_files  # noqa: F401
from .random_init import bind_random, random_tensors, write_random_model  # noqa: F401
