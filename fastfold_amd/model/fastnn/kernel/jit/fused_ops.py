"""The three elementwise fusions of the reference's ``kernel/jit/fused_ops.py:5-22``,
each one HIP launch instead of a TorchScript fusion group.  Signatures are identical.
Dropout masks are drawn with torch's generator in training mode (the mask tensor is
tiny: one row or column of the activation) and applied inside the kernel.
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


def _forward_only(name, *tensors):
    """The three ops launch forward kernels only; the reference's TorchScript versions are differentiable.  Rather
    than return outputs without a grad_fn (gradients would silently vanish), refuse inputs that require grad."""
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise NotImplementedError("%s: the HIP path implements the forward pass only; run it under torch.no_grad()" % name)


def bias_sigmod_ele(y, bias, z):
    """sigmoid(y + bias) * z   (fused_ops.py:5-7)."""
    _forward_only("bias_sigmod_ele", y, bias, z)
    y_, z_, b_ = y.contiguous(), z.contiguous(), bias.contiguous().to(y.dtype)
    _lib.check_device(y_, z_, b_)
    C = y_.shape[-1]
    out = torch.empty_like(y_)
    if y_.numel():
        _lib.call("ffk_bias_sigmoid_mul", _lib.ptr(out), _lib.ptr(y_), _lib.ptr(b_), _lib.ptr(z_),
                  y_.numel() // C, C, _lib.dtype_tag(y_.dtype), _lib.stream_ptr())
    return out


def bias_dropout_add(x: torch.Tensor, bias: torch.Tensor, dropmask: torch.Tensor, residual: torch.Tensor,
                     prob: float, training: bool) -> torch.Tensor:
    """residual + (x + bias) * dropout(dropmask)   (fused_ops.py:10-15)."""
    _forward_only("bias_dropout_add", x, bias, residual)
    x4, r4 = _as4d(x.contiguous()), _as4d(residual.contiguous())
    b_ = bias.contiguous().to(x.dtype)
    dm = F.dropout(dropmask, p=prob, training=training)
    dm4, (sb, si, sj) = _dm_strides(_as4d(dm) if dm.dim() != 4 else dm, x4)
    _lib.check_device(x4, r4, b_, dm4)
    B, I, J, C = x4.shape
    out = torch.empty_like(x4)
    if x4.numel():
        _lib.call("ffk_bias_dropout_add", _lib.ptr(out), _lib.ptr(x4), _lib.ptr(b_), _lib.ptr(dm4),
                  _lib.ptr(r4), B, I, J, C, sb, si, sj, _lib.dtype_tag(x4.dtype), _lib.stream_ptr())
    return out.view(x.shape)


def bias_ele_dropout_residual(ab: torch.Tensor, b: torch.Tensor, g: torch.Tensor, dropout_mask: torch.Tensor,
                              Z_raw: torch.Tensor, prob: float, training: bool) -> torch.Tensor:
    """Z_raw + dropout(dropout_mask) * (g * (ab + b))   (fused_ops.py:18-22)."""
    _forward_only("bias_ele_dropout_residual", ab, b, g, Z_raw)
    ab4, g4, z4 = _as4d(ab.contiguous()), _as4d(g.contiguous()), _as4d(Z_raw.contiguous())
    b_ = b.contiguous().to(ab.dtype)
    dm = F.dropout(dropout_mask, p=prob, training=training)
    dm4, (sb, si, sj) = _dm_strides(_as4d(dm) if dm.dim() != 4 else dm, ab4)
    _lib.check_device(ab4, g4, z4, b_, dm4)
    B, I, J, C = ab4.shape
    out = torch.empty_like(ab4)
    if ab4.numel():
        _lib.call("ffk_bias_ele_dropout_res", _lib.ptr(out), _lib.ptr(ab4), _lib.ptr(b_), _lib.ptr(g4),
                  _lib.ptr(dm4), _lib.ptr(z4), B, I, J, C, sb, si, sj, _lib.dtype_tag(ab4.dtype),
                  _lib.stream_ptr())
    return out.view(ab.shape)
