"""fused_softmax: softmax(where(mask == 0, -1e9, x + bias), dim=-1) on the HIP kernel.

Mirrors the reference's ``fastfold/model/fastnn/kernel/softmax.py:21-58``
(``FusedSoftmaxFunc`` / ``fused_softmax``): same call signature, same autograd
contract (grad for ``input`` and ``bias``, none for ``mask``; the bias gradient is the
input gradient summed over dim 1).
"""
from functools import reduce
from operator import mul

import torch

from fastfold_amd import _lib


def _softmax_forward(input_, mask_, bias_, out=None):
    _lib.check_device(input_, mask_, bias_)
    tag = _lib.dtype_tag(input_.dtype)
    if mask_ is not None or bias_ is not None:
        if input_.dim() != 5:
            raise RuntimeError("fused_softmax: masked / biased softmax expects a 5-D input "
                               "[B1, B2, H, Nq, Nk], got %s" % (tuple(input_.shape),))
        B1, B2, H, Nq, Nk = input_.shape
        if mask_ is not None:
            if tuple(mask_.shape) != (B1, B2, Nk) or mask_.dtype != input_.dtype:
                raise RuntimeError("fused_softmax: mask must be [B1, B2, Nk] of the input dtype, got %s %s"
                                   % (tuple(mask_.shape), mask_.dtype))
        if bias_ is not None:
            if tuple(bias_.shape) != (B1, 1, H, Nq, Nk) or bias_.dtype != input_.dtype:
                raise RuntimeError("fused_softmax: bias must be [B1, 1, H, Nq, Nk] of the input dtype, got %s %s"
                                   % (tuple(bias_.shape), bias_.dtype))
    else:
        Nk = input_.shape[-1]
        B1, B2, H, Nq = 1, 1, 1, reduce(mul, input_.shape[:-1], 1)
    if out is None:
        out = torch.empty_like(input_)
    if input_.numel() == 0:
        return out
    _lib.call("ffk_softmax_fwd", _lib.ptr(out), _lib.ptr(input_), _lib.ptr(mask_), _lib.ptr(bias_),
              B1, B2, H, Nq, Nk, tag, _lib.stream_ptr())
    return out


class FusedSoftmaxFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, mask=None, bias=None):
        input_ = input.contiguous()
        mask_ = mask.contiguous() if mask is not None else None
        bias_ = bias.contiguous() if bias is not None else None
        ctx.use_bias = bias is not None
        ctx.cols = input_.shape[-1]
        ctx.rows = reduce(mul, input.shape[:-1], 1)
        output = _softmax_forward(input_, mask_, bias_)
        ctx.save_for_backward(output)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        (output,) = ctx.saved_tensors
        _lib.check_device(grad_output, output)
        grad_input = torch.empty_like(output)
        _lib.call("ffk_softmax_bwd", _lib.ptr(grad_input), _lib.ptr(grad_output), _lib.ptr(output),
                  ctx.rows, ctx.cols, _lib.dtype_tag(output.dtype), _lib.stream_ptr())
        grad_bias = torch.sum(grad_input, dim=1, keepdim=True) if ctx.use_bias else None
        return grad_input, None, grad_bias


fused_softmax = FusedSoftmaxFunc.apply


def fused_softmax_(input, mask=None, bias=None):
    """In-place variant (no autograd): overwrites ``input`` with the probabilities, as the
    reference's CUDA kernels do (softmax_cuda_kernel.cu:438-440,521)."""
    return _softmax_forward(input, mask, bias, out=input)
