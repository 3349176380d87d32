"""The three elementwise fusions of the reference's ``kernel/jit/fused_ops.py:5-22``,
each one HIP launch instead of a TorchScript fusion group.  Signatures are identical.
Dropout masks are drawn with torch's generator in training mode (the mask tensor is
tiny: one row or column of the activation) and applied inside the kernel.  The backward
passes are elementwise torch expressions on the saved operands.
"""
import torch
import torch.nn.functional as F

from fastfold_amd import _lib


def _as4d(t):
    if t.dim() == 4:
        return t
    if t.dim() < 1:
        raise RuntimeError("expected a tensor with a channel dimension")
    lead = t.shape[:-1]
    rows = 1
    for d in lead:
        rows *= d
    return t.reshape(1, 1, rows, t.shape[-1])


def _dm_strides(dm, like):
    """Element strides of the (broadcast) dropout mask over the first three dims of `like`."""
    if tuple(dm.shape) == tuple(like.shape):
        dm = dm.contiguous()
        B, I, J, C = like.shape
        return dm, (I * J * C, J * C, C)
    dm = dm.contiguous()
    st = []
    for d in range(3):
        if dm.shape[d] == like.shape[d]:
            st.append(dm.stride(d))
        elif dm.shape[d] == 1:
            st.append(0)
        else:
            raise RuntimeError("dropout mask shape %s does not broadcast to %s"
                               % (tuple(dm.shape), tuple(like.shape)))
    if dm.shape[3] != like.shape[3]:
        raise RuntimeError("dropout mask must have the full channel dimension")
    return dm, tuple(st)


def _sum_to_bias(t, bias):
    """Column sums of ``t`` over every leading row, in fp32, as the gradient of a per-channel bias."""
    return t.reshape(-1, t.shape[-1]).sum(0, dtype=torch.float32).to(bias.dtype).view(bias.shape)


def _bias_sigmod_ele_kernel(y, bias, z):
    y_, z_, b_ = y.contiguous(), z.contiguous(), bias.contiguous().to(y.dtype)
    _lib.check_device(y_, z_, b_)
    C = y_.shape[-1]
    out = torch.empty_like(y_)
    if y_.numel():
        _lib.call("ffk_bias_sigmoid_mul", _lib.ptr(out), _lib.ptr(y_), _lib.ptr(b_), _lib.ptr(z_),
                  y_.numel() // C, C, _lib.dtype_tag(y_.dtype), _lib.stream_ptr())
    return out


class _BiasSigmodEle(torch.autograd.Function):

    @staticmethod
    def forward(ctx, y, bias, z):
        ctx.save_for_backward(y, bias, z)
        return _bias_sigmod_ele_kernel(y, bias, z)

    @staticmethod
    def backward(ctx, dout):
        y, bias, z = ctx.saved_tensors
        s = torch.sigmoid(y.float() + bias.float())
        d = dout.float()
        dz = (d * s).to(z.dtype) if ctx.needs_input_grad[2] else None
        dy = db = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            dy32 = d * z.float() * s * (1.0 - s)
            dy = dy32.to(y.dtype)
            db = _sum_to_bias(dy32, bias) if ctx.needs_input_grad[1] else None
        return dy, db, dz


def bias_sigmod_ele(y, bias, z):
    """sigmoid(y + bias) * z   (fused_ops.py:5-7).  One launch forward; differentiable in y, bias and z."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in (y, bias, z)):
        return _BiasSigmodEle.apply(y, bias, z)
    return _bias_sigmod_ele_kernel(y, bias, z)


def _bias_dropout_add_kernel(x, bias, dm, residual):
    x4, r4 = _as4d(x.contiguous()), _as4d(residual.contiguous())
    b_ = bias.contiguous().to(x.dtype)
    dm4, (sb, si, sj) = _dm_strides(_as4d(dm) if dm.dim() != 4 else dm, x4)
    _lib.check_device(x4, r4, b_, dm4)
    B, I, J, C = x4.shape
    out = torch.empty_like(x4)
    if x4.numel():
        _lib.call("ffk_bias_dropout_add", _lib.ptr(out), _lib.ptr(x4), _lib.ptr(b_), _lib.ptr(dm4),
                  _lib.ptr(r4), B, I, J, C, sb, si, sj, _lib.dtype_tag(x4.dtype), _lib.stream_ptr())
    return out.view(x.shape)


class _BiasDropoutAdd(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, bias, dm, residual):
        ctx.save_for_backward(bias, dm)
        return _bias_dropout_add_kernel(x, bias, dm, residual)

    @staticmethod
    def backward(ctx, dout):
        bias, dm = ctx.saved_tensors
        dx = db = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            dx = dout * dm
            db = _sum_to_bias(dx, bias) if ctx.needs_input_grad[1] else None
        return dx, db, None, (dout if ctx.needs_input_grad[3] else None)


def bias_dropout_add(x: torch.Tensor, bias: torch.Tensor, dropmask: torch.Tensor, residual: torch.Tensor,
                     prob: float, training: bool) -> torch.Tensor:
    """residual + (x + bias) * dropout(dropmask)   (fused_ops.py:10-15).  One launch forward; differentiable in
    x, bias and residual."""
    dm = F.dropout(dropmask, p=prob, training=training)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (x, bias, residual)):
        return _BiasDropoutAdd.apply(x, bias, dm.detach(), residual)
    return _bias_dropout_add_kernel(x, bias, dm, residual)


def _bias_ele_dropout_residual_kernel(ab, b, g, dm, Z_raw):
    ab4, g4, z4 = _as4d(ab.contiguous()), _as4d(g.contiguous()), _as4d(Z_raw.contiguous())
    b_ = b.contiguous().to(ab.dtype)
    dm4, (sb, si, sj) = _dm_strides(_as4d(dm) if dm.dim() != 4 else dm, ab4)
    _lib.check_device(ab4, g4, z4, b_, dm4)
    B, I, J, C = ab4.shape
    out = torch.empty_like(ab4)
    if ab4.numel():
        _lib.call("ffk_bias_ele_dropout_res", _lib.ptr(out), _lib.ptr(ab4), _lib.ptr(b_), _lib.ptr(g4),
                  _lib.ptr(dm4), _lib.ptr(z4), B, I, J, C, sb, si, sj, _lib.dtype_tag(ab4.dtype),
                  _lib.stream_ptr())
    return out.view(ab.shape)


class _BiasEleDropoutResidual(torch.autograd.Function):

    @staticmethod
    def forward(ctx, ab, b, g, dm, Z_raw):
        ctx.save_for_backward(ab, b, g, dm)
        return _bias_ele_dropout_residual_kernel(ab, b, g, dm, Z_raw)

    @staticmethod
    def backward(ctx, dout):
        ab, b, g, dm = ctx.saved_tensors
        d = dout * dm
        dab = db = dg = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            dab = d * g
            db = _sum_to_bias(dab, b) if ctx.needs_input_grad[1] else None
        if ctx.needs_input_grad[2]:
            dg = d * (ab + b.to(ab.dtype))
        return dab, db, dg, None, (dout if ctx.needs_input_grad[4] else None)


def bias_ele_dropout_residual(ab: torch.Tensor, b: torch.Tensor, g: torch.Tensor, dropout_mask: torch.Tensor,
                              Z_raw: torch.Tensor, prob: float, training: bool) -> torch.Tensor:
    """Z_raw + dropout(dropout_mask) * (g * (ab + b))   (fused_ops.py:18-22).  One launch forward; differentiable
    in ab, b, g and Z_raw."""
    dm = F.dropout(dropout_mask, p=prob, training=training)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (ab, b, g, Z_raw)):
        return _BiasEleDropoutResidual.apply(ab, b, g, dm.detach(), Z_raw)
    return _bias_ele_dropout_residual_kernel(ab, b, g, dm, Z_raw)
