"""GPU parity of the row-wise kernels through the C ABI, against the float64 numpy oracle.

Shapes, dtypes and tolerances follow the reference's own op tests
(tests/test_fastnn/test_softmax.py:7-38, tests/test_fastnn/test_layernorm.py:13-40)."""
import numpy as np
import pytest
import torch

from oracle import ops_np

pytestmark = pytest.mark.gpu

SOFTMAX_TOL = {torch.float32: 1e-6, torch.float16: 2e-4, torch.bfloat16: 1e-3}   # test_softmax.py:14
LN_TOL = {torch.float32: 1e-4, torch.float16: 1e-1, torch.bfloat16: 1e-1}        # test_layernorm.py:20


def _np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


@pytest.mark.parametrize("seq", [31, 32, 128, 129, 256, 259, 512, 700, 1024])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_fused_softmax_reference_cases(dev, seq, dtype):
    from fastfold_amd.model.fastnn.kernel import fused_softmax
    g = torch.Generator().manual_seed(seq)
    x = torch.rand(1, 8, 4, seq, seq, generator=g).to(dev, dtype)
    mask = (torch.rand(1, 8, seq, generator=g) > 0.1).to(dev, dtype)
    mask[..., 0] = 1
    bias = torch.rand(1, 1, 4, seq, seq, generator=g).to(dev, dtype)
    for m_, b_ in ((mask, bias), (mask, None), (None, None)):
        out = fused_softmax(x, m_, b_) if b_ is not None else (fused_softmax(x, m_) if m_ is not None else fused_softmax(x))
        ref = ops_np.fused_softmax(_np(x), None if m_ is None else _np(m_), None if b_ is None else _np(b_))
        err = np.abs(_np(out) - ref).max()
        assert err < SOFTMAX_TOL[dtype], (seq, dtype, err)
        if m_ is not None and dtype == torch.float32:
            assert float(out[0, :, :, :, :][(m_[0] == 0)[:, None, None, :].expand_as(out[0])].abs().max()) == 0.0


def test_fused_softmax_inplace_and_backward(dev):
    from fastfold_amd.model.fastnn.kernel import fused_softmax
    from fastfold_amd.model.fastnn.kernel.softmax import fused_softmax_
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 5, 2, 40, 40, generator=g).to(dev)
    mask = (torch.rand(1, 5, 40, generator=g) > 0.2).float().to(dev)
    mask[..., 3] = 1
    bias = torch.randn(1, 1, 2, 40, 40, generator=g).to(dev)
    xr, br = x.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    ref = torch.softmax(xr + br + 1e9 * (mask - 1)[:, :, None, None, :], -1)
    xf, bf = x.clone().requires_grad_(True), bias.clone().requires_grad_(True)
    out = fused_softmax(xf, mask, bf)
    assert (out - ref).abs().max().item() < 1e-6
    dy = torch.rand_like(out)
    ref.backward(dy)
    out.backward(dy)
    assert (xf.grad - xr.grad).abs().max().item() < 1e-6
    assert (bf.grad - br.grad).abs().max().item() < 1e-5
    y = x.clone()
    r = fused_softmax_(y, mask, bias)
    assert r.data_ptr() == y.data_ptr() and (y - ref.detach()).abs().max().item() < 1e-6


@pytest.mark.parametrize("shape", [(64, 64), (64, 128), (64, 129), (64, 1024), (3, 5, 256), (1000, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_layernorm_reference_cases(dev, shape, dtype):
    from fastfold_amd.model.fastnn.kernel import LayerNorm
    g = torch.Generator().manual_seed(shape[-1])
    x = torch.rand(*shape, generator=g).to(dev, dtype)
    ln = LayerNorm(shape[-1]).to(dev, dtype)
    with torch.no_grad():
        ln.weight.copy_(1 + 0.1 * torch.randn(shape[-1], generator=g))
        ln.bias.copy_(0.1 * torch.randn(shape[-1], generator=g))
    out = ln(x)
    ref = ops_np.layer_norm(_np(x), _np(ln.weight), _np(ln.bias), 1e-5)
    assert out.shape == x.shape and out.dtype == dtype
    assert np.abs(_np(out) - ref).max() < LN_TOL[dtype]
    if dtype == torch.float32:
        assert np.abs(_np(out) - ref).max() < 2e-6


def test_layernorm_backward(dev):
    from fastfold_amd.model.fastnn.kernel import LayerNorm
    g = torch.Generator().manual_seed(1)
    x = torch.randn(37, 129, generator=g).to(dev)
    ln = LayerNorm(129).to(dev)
    ref = torch.nn.LayerNorm(129).to(dev)
    with torch.no_grad():
        ln.weight.copy_(1 + 0.1 * torch.randn(129, generator=g))
        ref.weight.copy_(ln.weight)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    dy = torch.rand(37, 129, generator=g).to(dev)
    ln(xa).backward(dy)
    ref(xb).backward(dy)
    assert (xa.grad - xb.grad).abs().max().item() < 1e-4     # test_layernorm.py:20 (fp32)
    assert (ln.weight.grad - ref.weight.grad).abs().max().item() < 1e-4
    assert (ln.bias.grad - ref.bias.grad).abs().max().item() < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols", [(65, 64), (1000, 128), (37, 256), (4096 + 3, 384), (513, 512), (70, 1024),
                                       (33, 2048), (40, 72)])
def test_layernorm_backward_shapes(dev, dtype, rows, cols):
    """Both backward kernels (the vector form for rows of exactly lanes x vectors x 16 bytes up to 1024 elements, the
    general one otherwise) against float64 autograd of torch's layer_norm on the same rounded inputs; row counts that
    leave ragged row groups, enough rows for several grid-stride passes."""
    from fastfold_amd.model.fastnn.kernel import LayerNorm
    g = torch.Generator().manual_seed(rows + cols)
    x = torch.randn(rows, cols, generator=g).to(dev, dtype)
    dy = torch.randn(rows, cols, generator=g).to(dev, dtype)
    ln = LayerNorm(cols).to(dev, dtype)
    with torch.no_grad():
        ln.weight.copy_(1 + 0.2 * torch.randn(cols, generator=g))
        ln.bias.copy_(0.1 * torch.randn(cols, generator=g))
    xa = x.clone().requires_grad_(True)
    ln(xa).backward(dy)
    xr = x.double().cpu().requires_grad_(True)
    wr, br = ln.weight.detach().double().cpu().requires_grad_(True), ln.bias.detach().double().cpu().requires_grad_(True)
    torch.nn.functional.layer_norm(xr, (cols,), wr, br, ln.eps).backward(dy.double().cpu())
    tol = 1e-5 if dtype == torch.float32 else (1.5e-2 if dtype == torch.bfloat16 else 2e-3)

    def rel(a, b):
        return float((a.double().cpu() - b).abs().max() / b.abs().max())
    assert rel(xa.grad, xr.grad) <= tol, rel(xa.grad, xr.grad)
    assert rel(ln.weight.grad, wr.grad) <= tol, rel(ln.weight.grad, wr.grad)
    assert rel(ln.bias.grad, br.grad) <= tol, rel(ln.bias.grad, br.grad)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [128, 36, 7])
def test_elementwise_fusions(dev, dtype, C):
    from fastfold_amd.model.fastnn.kernel import bias_dropout_add, bias_sigmod_ele, bias_ele_dropout_residual
    g = torch.Generator().manual_seed(C)
    sh = (1, 6, 9, C)
    y, z, r = (torch.randn(*sh, generator=g).to(dev, dtype) for _ in range(3))
    b = torch.randn(C, generator=g).to(dev, dtype)
    tol = 1e-5 if dtype == torch.float32 else 4e-2
    out = bias_sigmod_ele(y, b, z)
    assert np.abs(_np(out) - ops_np.bias_sigmod_ele(_np(y), _np(b), _np(z))).max() < tol
    for dm in (torch.ones_like(y[:, 0:1, :, :]), torch.ones_like(y[:, :, 0:1, :])):
        dm = dm * 0.5   # any multiplier must be applied as given in eval mode
        out = bias_dropout_add(y, b, dm, r, prob=0.25, training=False)
        assert np.abs(_np(out) - ops_np.bias_dropout_add(_np(y), _np(b), _np(dm), _np(r))).max() < tol
        out = bias_ele_dropout_residual(y, b, z, dm, r, prob=0.25, training=False)
        assert np.abs(_np(out) - ops_np.bias_ele_dropout_residual(_np(y), _np(b), _np(z), _np(dm), _np(r))).max() < tol


def test_errors_raise_runtime_error(dev):
    from fastfold_amd.model.fastnn.kernel import fused_softmax
    with pytest.raises(RuntimeError):
        fused_softmax(torch.rand(2, 3, 4), torch.ones(2, 4))                       # CPU tensors
    x = torch.rand(1, 2, 2, 4, 4, device=dev)
    with pytest.raises(RuntimeError):
        fused_softmax(x, torch.ones(1, 2, 5, device=dev))                          # wrong mask shape
    with pytest.raises(RuntimeError):
        fused_softmax(x.double())                                                  # unsupported dtype
