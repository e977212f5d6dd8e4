from clockwork_amd.weights.checkpoint import CheckpointIndex, WeightMismatchError
from clockwork_amd.weights.loader import load_parameters, read_config_json
from clockwork_amd.weights.random_init import random_checkpoint_tensors, write_random_model

__all__ = [
    "CheckpointIndex",
    "WeightMismatchError",
    "load_parameters",
    "read_config_json",
    "random_checkpoint_tensors",
    "write_random_model",
]
