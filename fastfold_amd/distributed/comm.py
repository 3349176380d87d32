"""Synchronous DAP primitives at world size 1: every one is the identity, as in the reference when
``gpc.get_world_size(ParallelMode.TENSOR) == 1`` (fastfold/distributed/comm.py:18-20,30-32,42-44,146-148)."""


def divide(numerator, denominator):
    assert numerator % denominator == 0, "{} is not divisible by {}".format(numerator, denominator)
    return numerator // denominator


def _reduce(tensor):
    return tensor


def _split(tensor, dim=-1):
    return tensor


def _gather(tensor, dim=-1):
    return tensor


def _all_to_all(tensor, in_dim=-1, out_dim=-1):
    return tensor


def copy(input):
    return input


def scatter(input, dim=-1):
    return input


def reduce(input):
    return input


def gather(input, dim=-1):
    return input


def col_to_row(input_):
    return input_


def row_to_col(input_):
    return input_
