"""Asynchronous DAP primitives at world size 1 (fastfold/distributed/comm_async.py:58-199): the "async" half
returns its input and ``work = None``, the "opp" half returns the tensor it is given - exactly what the
reference's functions do when the tensor-parallel world has one member (``:66-68,90-95,129-131,186-191``)."""
import torch

from .core import get_rank, get_world_size  # noqa: F401  (comm_async.py:58-63 exports both)


def _gather_async(tensor, dim=-1):
    return tensor, None


def gather_async(input, dim=-1):
    return input, None


def gather_async_opp(output, work, dim=-1):
    if work:
        work.wait()
    return output


def _all_to_all_async(tensor, in_dim=-1, out_dim=-1):
    return tensor, None


class All_to_All_Async(torch.autograd.Function):
    """``m, work = All_to_All_Async.apply(m, 1, 2)`` (fastnn/evoformer.py:67): identity, ``work`` is None."""

    @staticmethod
    def forward(ctx, input_, in_dim=-1, out_dim=-1):
        return input_, None

    @staticmethod
    def backward(ctx, grad_output, grad_work=None):
        return grad_output, None, None


class All_to_All_Async_Opp(torch.autograd.Function):
    """``m = All_to_All_Async_Opp.apply(m, work, 1, 2)`` (fastnn/evoformer.py:69): waits for ``work`` if there is
    one; the regrouping ``n (x h) w c -> n h (x w) c`` with x = 1 is the identity."""

    @staticmethod
    def forward(ctx, output, work, in_dim=-1, out_dim=-1):
        if work:
            work.wait()
        return output

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None, None, None
