"""Dynamic Axial Parallelism shims at world size 1.

This build runs the Evoformer on one GPU (DAP size 1).  Every communication primitive of
the reference's ``fastfold.distributed`` is the identity at that size
(fastfold/distributed/comm.py:19-20,31-32,43-44,147-148; comm_async.py:67-68,90-95,130-131,
186-191); they are kept so code written against the reference imports and runs unchanged.
"""
import os

_DAP_SIZE = 1


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


def scatter(input, dim=-1):
    return input


def gather(input, dim=-1):
    return input


def reduce(input):
    return input


def copy(input):
    return input


def row_to_col(input):
    return input


def col_to_row(input):
    return input


def gather_async(input, dim=-1):
    return input, None


def gather_async_opp(output, work, dim=-1):
    return output


__all__ = ["init_dap", "get_world_size", "get_rank", "scatter", "gather", "reduce", "copy", "row_to_col",
           "col_to_row", "gather_async", "gather_async_opp"]
