"""Import surface the reference's callers rely on (CPU: nothing here launches a kernel)."""
import subprocess
import sys

import torch


def test_distributed_module_paths_and_identities():
    """fastfold/distributed/{core,comm,comm_async}.py at world size 1 (comm.py:18-20,30-32,42-44,146-148;
    comm_async.py:66-68,90-95,129-131,153-199): every primitive returns its tensor, the async halves return
    ``work = None``."""
    from fastfold_amd.distributed import col_to_row, gather, init_dap, row_to_col, scatter
    from fastfold_amd.distributed.comm import _all_to_all, _gather, _reduce, _split, copy, reduce
    from fastfold_amd.distributed.comm_async import (All_to_All_Async, All_to_All_Async_Opp, gather_async,
                                                     gather_async_opp, get_rank, get_world_size)
    from fastfold_amd.distributed.core import ensure_divisibility
    init_dap(1)
    ensure_divisibility(8, 1)
    assert get_world_size() == 1 and get_rank() == 0
    x = torch.arange(24.0).reshape(1, 2, 3, 4)
    for f in (scatter, gather, col_to_row, row_to_col, _reduce, _split, _gather, _all_to_all, copy, reduce):
        assert f(x) is x
    y, work = gather_async(x, dim=1)
    assert y is x and work is None and gather_async_opp(y, work, dim=1) is x
    # the call pattern of fastnn/evoformer.py:67-69
    m, work = All_to_All_Async.apply(x, 1, 2)
    assert work is None and torch.equal(m, x)
    assert torch.equal(All_to_All_Async_Opp.apply(m, work, 1, 2), x)
    # and it is transparent to autograd
    g = x.clone().requires_grad_(True)
    m, work = All_to_All_Async.apply(g, 1, 2)
    All_to_All_Async_Opp.apply(m, work, 1, 2).sum().backward()
    assert torch.equal(g.grad, torch.ones_like(x))


def test_fastfold_alias_is_opt_in():
    """``install_as_fastfold()`` makes the reference's import lines work (benchmark/perf.py:7-8,
    fastnn/evoformer.py:12-13, inference.py:42); without it no ``fastfold`` module exists."""
    code = (
        "import importlib.util, sys\n"
        "sys.path = [p for p in sys.path if 'reference' not in p]\n"
        "assert importlib.util.find_spec('fastfold') is None\n"
        "import fastfold_amd\n"
        "fastfold_amd.install_as_fastfold()\n"
        "from fastfold.model.fastnn import Evoformer, EvoformerStack, set_chunk_size\n"
        "from fastfold.model.fastnn.kernel import fused_softmax, LayerNorm, bias_dropout_add, bias_sigmod_ele, "
        "bias_ele_dropout_residual, fused_attention_core\n"
        "from fastfold.distributed import init_dap\n"
        "from fastfold.distributed.comm import gather, scatter, col_to_row\n"
        "from fastfold.distributed.comm_async import All_to_All_Async, All_to_All_Async_Opp\n"
        "from fastfold.utils.inject_fastnn import inject_fastnn\n"
        "import fastfold_amd.model.fastnn as real\n"
        "assert Evoformer is real.Evoformer\n"
        "print('ok')\n")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stderr


def test_slab_weight_gradient_on_cpu():
    """``_weight_grad`` (the differentiable Linear's dW): bf16 activations with many rows are reduced slab by slab through
    a batched GEMM and summed in fp32; other inputs take the plain product.  Both against float64."""
    from fastfold_amd.model.fastnn.ops import _LinearFn, _weight_grad
    g = torch.Generator().manual_seed(0)
    dy = torch.randn(32768, 24, generator=g)
    x = torch.randn(32768, 40, generator=g)
    ref = dy.double().t() @ x.double()
    assert torch.allclose(_weight_grad(dy, x).double(), ref, rtol=1e-4, atol=1e-2)            # fp32: plain product
    got = _weight_grad(dy.bfloat16(), x.bfloat16())                                            # 8 slabs of 4096 rows
    assert got.dtype == torch.bfloat16
    ref16 = dy.bfloat16().double().t() @ x.bfloat16().double()
    assert float((got.double() - ref16).norm() / ref16.norm()) < 1e-2
    odd = _weight_grad(dy[:4099].bfloat16(), x[:4099].bfloat16())                              # no even split: plain
    assert float((odd.double() - dy[:4099].bfloat16().double().t() @ x[:4099].bfloat16().double()).norm()) < 5.0
    # the autograd function against float64 autograd of F.linear
    xi = torch.randn(3, 7, 10, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(5, 10, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(5, generator=g, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(_LinearFn.apply, (xi, w, b))
    assert torch.autograd.gradcheck(lambda a, c: _LinearFn.apply(a, c, None), (xi, w))
