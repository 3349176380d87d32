"""DAP initialisation at world size 1 (reference: fastfold/distributed/core.py:7-40)."""
import os

_DAP_SIZE = 1


def ensure_divisibility(numerator, denominator):
    assert numerator % denominator == 0, "{} is not divisible by {}".format(numerator, denominator)


def init_dap(tensor_model_parallel_size_=None):
    """Reference: fastfold/distributed/core.py:17-40.  Only size 1 is supported here."""
    if tensor_model_parallel_size_ is None:
        tensor_model_parallel_size_ = int(os.environ.get("WORLD_SIZE", "1"))
    if tensor_model_parallel_size_ != 1:
        raise RuntimeError("fastfold_amd runs on one GPU: DAP size must be 1, got %d"
                           % tensor_model_parallel_size_)


def get_world_size():
    return _DAP_SIZE


def get_rank():
    return 0
