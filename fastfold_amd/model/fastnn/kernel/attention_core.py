"""``fused_attention_core`` with the reference's interface
(fastfold/model/fastnn/kernel/attention_core.py:17-52):

    softmax(q * d**-0.5 @ k^T + bias + BIG * (mask - 1)) @ v   ->   [b1, b2, n, h*d]

for q, k, v ``[b1, b2, h, n, d]``, mask ``[b1, b2, n]`` (0/1, over keys) and bias ``[b1, h, n, n]``.
The logits are never materialised: the operands are re-tiled into the 32x32 MFMA order and handed to
the flash attention kernel (``ffk_attention_fwd``); the backward pass (``ffk_attention_bwd``) recomputes them the
same way.  The tuned kernel is the Evoformer's head dim (32); narrower heads (8 and 16, the extra-MSA and template
stacks) are zero-padded to 32 channels, which changes neither the scores nor the used output channels; the other
widths the reference's Triton kernel takes (64 and 128, triton/attention_core.py:142), which no module of the path
uses, run on a plain one-wave-per-query-tile instantiation that cuts the head into 32-channel parts.
Dtypes: bf16 and fp32 (forward and backward); fp16 raises here, before anything is launched.
"""
import math

import torch

from .... import _lib
from . import layouts


def _attention_core(q, k, v, mask=None, bias=None):
    for t in (q, k, v, mask, bias):          # any strides: the operands are re-tiled as they lie
        if t is not None and not t.is_cuda:
            raise RuntimeError("fastfold_amd: tensor must be a CUDA/HIP tensor (got %s)" % t.device)
    if q.dim() != 5 or q.shape != k.shape or q.shape != v.shape:
        raise RuntimeError("fused_attention_core: q, k, v must be [b1, b2, h, n, d] of one shape, got %s %s %s"
                           % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    b1, b2, h, n, d = q.shape
    if d not in (8, 16, 32, 64, 128):
        raise RuntimeError("fused_attention_core: head dim %d is not supported (8, 16, 32, 64 or 128)" % d)
    if q.dtype not in (torch.bfloat16, torch.float32) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("fused_attention_core: q, k, v must share one dtype, bfloat16 or float32 (got %s, %s, %s)"
                           % (q.dtype, k.dtype, v.dtype))
    if mask is not None and tuple(mask.shape) != (b1, b2, n):
        raise RuntimeError("fused_attention_core: mask must be [b1, b2, n], got %s" % (tuple(mask.shape),))
    if bias is not None and tuple(bias.shape) != (b1, h, n, n):
        raise RuntimeError("fused_attention_core: bias must be [b1, h, n, n], got %s" % (tuple(bias.shape),))
    # zero channels past d add nothing to q.k and give zero output channels, which are dropped at the end
    dk = max(d, 32)                        # head width the kernel sees
    out = torch.empty(b1, b2, n, h * dk, dtype=q.dtype, device=q.device)
    if out.numel() == 0:
        return out.view(b1, b2, n, h, dk)[..., :d].reshape(b1, b2, n, h * d)
    nt = layouts.n_tiles(n)
    scale = _lib.LOG2E / math.sqrt(d)      # the kernel exponentiates in base 2
    kb = torch.empty(b2, nt * 32, dtype=torch.float32, device=q.device)
    fl = torch.empty(b2, nt, dtype=torch.int32, device=q.device)
    for i in range(b1):
        mk = mask[i].to(q.dtype).contiguous() if mask is not None else torch.ones(b2, n, dtype=q.dtype, device=q.device)
        _lib.key_bias(kb, fl, mk, B=b2, N=n, mask_sb=n, mask_sn=1)
        bt = layouts.tile_bias((bias[i].float() * _lib.LOG2E).to(q.dtype)) if bias is not None else None
        _lib.attention_fwd(out[i].view(b2 * n, h * dk), _lib.tile_pack(q[i], _lib.FFK_TILE_QK, scale),
                           _lib.tile_pack(k[i], _lib.FFK_TILE_QK), _lib.tile_pack(v[i], _lib.FFK_TILE_V), bt, kb, fl,
                           None, B2=b2, H=h, Nq=n, Nk=n, D=dk)
    if d < 32:
        return out.view(b1, b2, n, h, 32)[..., :d].reshape(b1, b2, n, h * d)
    return out


def _attention_core_backward(q, k, v, mask, bias, out, dout, need_dbias):
    """dq, dk, dv (shapes of q, k, v) and dbias ([b1, h, n, n] or None) through ``ffk_attention_bwd``."""
    b1, b2, h, n, d = q.shape
    dt, dev = q.dtype, q.device
    QK, ACC = _lib.FFK_TILE_QK, _lib.FFK_TILE_V
    nt = layouts.n_tiles(n)
    dk_ = max(d, 32)
    scale = _lib.LOG2E / math.sqrt(d)
    dq, dk, dv = (torch.empty(b1, b2, h, n, dk_, dtype=dt, device=dev) for _ in range(3))
    dbias = torch.zeros(b1, h, n, n, dtype=torch.float32, device=dev) if (need_dbias and bias is not None) else None
    kb = torch.empty(b2, nt * 32, dtype=torch.float32, device=dev)
    fl = torch.empty(b2, nt, dtype=torch.int32, device=dev)
    lse = torch.empty(b2 * h * nt * 32, dtype=torch.float32, device=dev)
    dsum = torch.empty_like(lse)
    for i in range(b1):
        mk = mask[i].to(dt).contiguous() if mask is not None else torch.ones(b2, n, dtype=dt, device=dev)
        _lib.key_bias(kb, fl, mk, B=b2, N=n, mask_sb=n, mask_sn=1)
        bt = layouts.tile_bias((bias[i].float() * _lib.LOG2E).to(dt)) if bias is not None else None
        do_ = dout[i].view(b2, n, h, d).permute(0, 2, 1, 3)          # [b2, h, n, d] views: re-tiled as they lie
        o_ = out[i].view(b2, n, h, d).permute(0, 2, 1, 3)
        _lib.attention_bwd(dq[i], dk[i], dv[i], None if dbias is None else dbias[i], lse, dsum,
                           _lib.tile_pack(q[i], QK, scale), _lib.tile_pack(q[i], ACC, scale),     # as the forward saw q
                           _lib.tile_pack(k[i], QK), _lib.tile_pack(k[i], ACC), _lib.tile_pack(v[i], QK),
                           bt, kb,
                           _lib.tile_pack(do_, QK), _lib.tile_pack(do_, ACC), _lib.tile_pack(o_, QK),
                           B2=b2, H=h, Nq=n, Nk=n, D=dk_, dq_scale=1.0 / math.sqrt(d), dk_scale=1.0 / _lib.LOG2E)
    if d < 32:
        dq, dk, dv = (t[..., :d] for t in (dq, dk, dv))
    return dq, dk, dv, (None if dbias is None else dbias.to(dt))


class FusedAttenionCoreFunc(torch.autograd.Function):
    """Name (including its spelling) as in the reference (attention_core.py:34).  The reference's function has no
    backward (training goes through matmul / fused_softmax / matmul there, fastnn/ops.py:310-322); this one has:
    dq, dk, dv and dbias from ``ffk_attention_bwd``, which recomputes the logits tile by tile."""

    @staticmethod
    def forward(ctx, q, k, v, mask=None, bias=None):
        out = _attention_core(q, k, v, mask, bias)
        if any(t is not None and t.requires_grad for t in (q, k, v, bias)):
            ctx.save_for_backward(q, k, v, mask, bias, out)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, mask, bias, out = ctx.saved_tensors
        dq, dk, dv, dbias = _attention_core_backward(q, k, v, mask, bias, out.contiguous(), dout.contiguous(),
                                                     bias is not None and ctx.needs_input_grad[4])
        return dq, dk, dv, None, dbias


fused_attention_core = FusedAttenionCoreFunc.apply
