"""LayerNorm module backed by the HIP kernel.

Mirrors the reference's ``fastfold/model/fastnn/kernel/layer_norm.py:19-60``
(``FusedLayerNorm``, exported as ``kernel.LayerNorm``): ``normalized_shape``/``eps``
constructor, ``weight``/``bias`` parameters initialised to 1/0, forward over the
trailing ``normalized_shape`` dims, biased variance.
"""
import numbers
from functools import reduce
from operator import mul

import torch
from torch.nn.parameter import Parameter

from fastfold_amd import _lib


class FusedLayerNormAffineFunction(torch.autograd.Function):
    """Same argument order as the reference's autograd function
    (kernel/cuda_native/layer_norm.py:8-35)."""

    @staticmethod
    def forward(ctx, input, weight, bias, normalized_shape, eps):
        ctx.normalized_shape = normalized_shape
        ctx.eps = eps
        input_ = input.contiguous()
        weight_ = weight.contiguous()
        bias_ = bias.contiguous()
        _lib.check_device(input_, weight_, bias_)
        cols = reduce(mul, normalized_shape, 1)
        if tuple(input_.shape[input_.dim() - len(normalized_shape):]) != tuple(normalized_shape):
            raise RuntimeError("LayerNorm: expected trailing dims %s, got input shape %s"
                               % (tuple(normalized_shape), tuple(input_.shape)))
        if weight_.numel() != cols or bias_.numel() != cols:
            raise RuntimeError("LayerNorm: weight/bias must have %d elements" % cols)
        if weight_.dtype != input_.dtype or bias_.dtype != input_.dtype:
            weight_ = weight_.to(input_.dtype)
            bias_ = bias_.to(input_.dtype)
        rows = input_.numel() // cols if cols else 0
        output = torch.empty_like(input_)
        need_stats = input.requires_grad or weight.requires_grad or bias.requires_grad
        mean = torch.empty(rows, dtype=torch.float32, device=input_.device) if need_stats else None
        rstd = torch.empty(rows, dtype=torch.float32, device=input_.device) if need_stats else None
        if rows > 0:
            _lib.call("ffk_layernorm_fwd", _lib.ptr(output), _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(input_),
                      _lib.ptr(weight_), _lib.ptr(bias_), rows, cols, float(eps),
                      _lib.dtype_tag(input_.dtype), _lib.stream_ptr())
        if need_stats:
            ctx.save_for_backward(input_, weight_, mean, rstd)
        ctx.dims = (rows, cols)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        input_, weight_, mean, rstd = ctx.saved_tensors
        rows, cols = ctx.dims
        g = grad_output.contiguous()
        dx = torch.empty_like(input_)
        dgamma = torch.zeros(cols, dtype=torch.float32, device=input_.device)
        dbeta = torch.zeros(cols, dtype=torch.float32, device=input_.device)
        _lib.call("ffk_layernorm_bwd", _lib.ptr(dx), _lib.ptr(dgamma), _lib.ptr(dbeta), _lib.ptr(g),
                  _lib.ptr(input_), _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(weight_), rows, cols,
                  _lib.dtype_tag(input_.dtype), _lib.stream_ptr())
        shape = tuple(ctx.normalized_shape)
        return dx, dgamma.to(weight_.dtype).view(shape), dbeta.to(weight_.dtype).view(shape), None, None


class FusedLayerNorm(torch.nn.Module):

    def __init__(self, normalized_shape, eps=1e-5):
        super(FusedLayerNorm, self).__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.weight = Parameter(torch.empty(*normalized_shape))
        self.bias = Parameter(torch.empty(*normalized_shape))
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)
        torch.nn.init.zeros_(self.bias)

    def forward(self, input):
        return self.kernel_forward(input)

    def kernel_forward(self, input):
        return FusedLayerNormAffineFunction.apply(input, self.weight, self.bias, self.normalized_shape,
                                                  self.eps)

    def extra_repr(self):
        return "{}, eps={}".format(tuple(self.normalized_shape), self.eps)
