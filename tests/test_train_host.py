"""Host-side checks of the differentiable path (run on the CPU): the guard in front of every library batched GEMM,
and the address arithmetic of the operand views that were handed to the library in the two runs at N_res = 1024
that ended in a GPU memory fault inside its batched NT GEMM (bf16, 128 x 1024^3)."""
import pytest
import torch

from fastfold_amd.model.fastnn import _fused as F_
from fastfold_amd.model.fastnn import ops


def _span_elems(shape, stride, offset):
    return offset, offset + sum((n - 1) * st for n, st in zip(shape, stride)) + 1


def test_faulting_views_were_inside_their_allocation():
    """Both faulting launches took their operands from the padded buffer of the fused triangle multiplication,
    ``lr = [2, c, r * kpad + pad]`` (channel planes ``cs`` elements apart, operand ``side`` at ``side * c * cs``),
    viewed as [c, r, kpad] with strides (cs, kpad, 1), and wrote to ``p = [c, cs]`` viewed the same way.  Largest
    element offset each view addresses, against the allocation: all inside - the callers' indexing is cleared."""
    r, c = 1024, 128
    kpad = F_.round_up(r, 8)
    cs = r * kpad + F_._TRIMUL_CHAN_PAD
    lr_elems, p_elems = 2 * c * cs, c * cs
    for side in range(2):
        lo, hi = _span_elems((c, r, kpad), (cs, kpad, 1), side * c * cs)
        assert lo == side * c * cs and hi <= lr_elems
        # the NT product reads the second operand through a transposed view: same elements
        lo_t, hi_t = _span_elems((c, kpad, r), (cs, 1, kpad), side * c * cs)
        assert (lo_t, hi_t) == (lo, hi)
    # the two operands do not overlap each other
    assert _span_elems((c, r, kpad), (cs, kpad, 1), 0)[1] <= c * cs
    lo, hi = _span_elems((c, r, r), (cs, kpad, 1), 0)
    assert hi <= p_elems
    # the same through torch's own bookkeeping (meta tensors: no memory is touched)
    lr = torch.empty(2, c, cs, dtype=torch.bfloat16, device="meta")
    for side in range(2):
        v = lr[side][:, :r * kpad].view(c, r, kpad)
        assert v.stride() == (cs, kpad, 1) and v.storage_offset() == side * c * cs
        assert ops._storage_span(v)[1] <= lr_elems * 2
        assert ops._storage_span(v.transpose(1, 2))[1] <= lr_elems * 2


def test_library_gemm_guard_rejects_views_of_one_allocation():
    buf = torch.zeros(2, 4, 40)
    a, b = buf[0].view(4, 5, 8), buf[1].view(4, 5, 8)
    with pytest.raises(RuntimeError, match="views of one allocation"):
        ops._check_library_gemm_operands(a, b.transpose(1, 2), "test")
    ops._check_library_gemm_operands(a, b.clone(), "test")
    # a view whose storage was shrunk underneath it addresses more than the allocation holds
    t = torch.zeros(4, 4)
    v = t.view(4, 4)
    t.untyped_storage().resize_(32)
    with pytest.raises(RuntimeError, match="bytes of a"):
        ops._check_library_gemm_operands(v, torch.zeros(4, 4), "test")


def test_weight_grad_never_hands_the_library_one_allocation(monkeypatch):
    """Slab weight gradient (bf16, >= 8192 rows -> the batched GEMM branch): with dy and x sliced from ONE tensor the
    operands reach torch.bmm in two allocations, and the result is the plain product."""
    seen = []
    real_bmm = torch.bmm

    def spy(a, b):
        seen.append(a.untyped_storage().data_ptr() != b.untyped_storage().data_ptr())
        return real_bmm(a, b)
    monkeypatch.setattr(torch, "bmm", spy)
    g = torch.Generator().manual_seed(0)
    both = torch.randn(16384, 48, generator=g).to(torch.bfloat16)
    dy, x = both[:, :16], both[:, 16:]
    got = ops._weight_grad(dy, x)
    assert seen == [True]
    want = dy.double().t() @ x.double()
    assert float((got.double() - want).norm() / want.norm()) < 1e-2


def test_chan_major_copies_are_separate_and_padded():
    g = torch.Generator().manual_seed(1)
    lr = torch.randn(1, 6, 6, 8, generator=g)
    left, right = lr.chunk(2, dim=-1)
    L, R = ops._chan_major(left, (2, 0, 1)), ops._chan_major(right, (2, 0, 1))
    assert L.shape == (4, 6, 8) and L.is_contiguous() and R.is_contiguous()
    assert L.untyped_storage().data_ptr() != R.untyped_storage().data_ptr()
    assert torch.equal(L[..., :6], left[0].permute(2, 0, 1)) and float(L[..., 6:].abs().max()) == 0.0
    Li = ops._chan_major(left, (2, 1, 0))                 # incoming: L[c, i, k] = left[k, i, c]
    assert torch.equal(Li[..., :6], left[0].permute(2, 1, 0))
