"""Dynamic Axial Parallelism shims at world size 1.

This build runs the Evoformer on one GPU (DAP size 1).  Every communication primitive of the reference's
``fastfold.distributed`` is the identity at that size (fastfold/distributed/comm.py:19-20,31-32,43-44,147-148;
comm_async.py:67-68,90-95,130-131,186-191); they are kept, under the reference's module paths (``core``,
``comm``, ``comm_async``), so that code written against the reference imports and runs unchanged.
"""
from .core import init_dap, get_world_size, get_rank
from .comm import _reduce, _split, _gather, copy, scatter, reduce, gather, col_to_row, row_to_col
from .comm_async import All_to_All_Async, All_to_All_Async_Opp, gather_async, gather_async_opp

__all__ = ["init_dap", "_reduce", "_split", "_gather", "copy", "scatter", "reduce", "gather", "col_to_row",
           "row_to_col", "get_world_size", "get_rank", "gather_async", "gather_async_opp", "All_to_All_Async",
           "All_to_All_Async_Opp"]
