"""Checkpoint reading, the declared-tensor check, and the random-weights writer."""
from .loader import (COMPUTE, FLOAT32, INT32, TensorDecl, WeightError, WeightStore,
                     check_table, load_weights, table_of)
from .random_init import random_tensor, random_weights_on_device, write_random_model
from .safetensors_io import SafetensorsFile, open_checkpoint, write_safetensors
