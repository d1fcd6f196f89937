from .loader import TensorSource, WeightsError, bind, bind_from_checkpoint, held_dtype, list_weight_files, named_tensors  # noqa: F401
from .random_init import RandomSource, bind_random, random_tensors, write_random_model  # noqa: F401
