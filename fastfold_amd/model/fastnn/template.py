"""Template pair stack (Algorithm 16) with the reference's interface
(fastfold/model/fastnn/template.py:185-434): per template, triangle attention around the starting and
the ending node, outgoing and incoming triangle multiplication and the pair transition at the template
width (c_t = 64, 4 heads of 16, multiplication width 64, transition factor 2), then a LayerNorm.

The modules are the ones of the Evoformer pair stack at other widths: the attention kernel takes the
16-wide heads zero-padded to 32 channels, the projections run on the generic kernel variants.
As for ``Evoformer``, the reference's padding by one residue between blocks is kept as an interface only.
"""
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from fastfold_amd.model.fastnn.kernel import LayerNorm
from fastfold_amd import _lib
from . import _fused as F_
from .ops import (AsyncChunkTriangleMultiplicationIncoming, AsyncChunkTriangleMultiplicationOutgoing,
                  ChunkTransition, ChunkTriangleAttentionEndingNode, ChunkTriangleAttentionStartingNode, Linear,
                  _PackMixin, _needs_grad, _no_grad_guard)


class _PointwiseProjections(nn.Module):
    """Parameter holder with the names of the reference's generic ``Attention`` (nn/primitives.py:333-338),
    gating off: ``linear_q`` / ``linear_k`` / ``linear_v`` without bias, ``linear_o`` with bias."""

    def __init__(self, c_q, c_kv, c_hidden, no_heads):
        super(_PointwiseProjections, self).__init__()
        hc = c_hidden * no_heads
        self.linear_q = Linear(c_q, hc, use_bias=False)
        self.linear_k = Linear(c_kv, hc, use_bias=False)
        self.linear_v = Linear(c_kv, hc, use_bias=False)
        self.linear_o = Linear(hc, c_q, initializer='zeros')


class TemplatePointwiseAttention(nn.Module, _PackMixin):
    """Algorithm 17 (fastfold/model/fastnn/template.py:33-182): every pair position attends over the
    templates' embeddings at that position.  Two projection launches (q from z, k and v from t), one
    streaming kernel for the softmax over at most 8 templates, one output projection; the update is zero
    when no template is valid, as in the reference."""

    def __init__(self, c_t, c_z, c_hidden, no_heads, inf, **kwargs):
        super(TemplatePointwiseAttention, self).__init__()
        self.c_t, self.c_z, self.c_hidden, self.no_heads, self.inf = c_t, c_z, c_hidden, no_heads, inf
        self.mha = _PointwiseProjections(c_z, c_t, c_hidden, no_heads)

    def _run(self, t, z, template_mask, resid):
        F_.check_cuda(t, z, template_mask)
        _no_grad_guard(self, t, z)
        if t.dim() != 4 or z.dim() != 3 or t.shape[1:3] != z.shape[:2] or t.shape[-1] != self.c_t or z.shape[-1] != self.c_z:
            raise RuntimeError("TemplatePointwiseAttention: expected t [N_templ, r, r, %d] and z [r, r, %d], got %s / %s"
                               % (self.c_t, self.c_z, tuple(t.shape), tuple(z.shape)))
        NT, r = t.shape[0], t.shape[1]
        if NT > 8:
            raise RuntimeError("TemplatePointwiseAttention: at most 8 templates per launch, got %d" % NT)
        dt, dev = z.dtype, z.device
        H, D = self.no_heads, self.c_hidden
        hc = H * D
        P = r * r
        m = self.mha
        wq, wkv, wo, bo = self._packed(("pw", dt, dev), [m.linear_q.weight, m.linear_k.weight, m.linear_v.weight,
                                                          m.linear_o.weight, m.linear_o.bias], lambda: (
            F_.pack_rows([m.linear_q.weight.detach() * (float(D) ** -0.5)], dt, dev),
            F_.pack_rows([m.linear_k.weight, m.linear_v.weight], dt, dev),
            F_.pack_rows([m.linear_o.weight], dt, dev), F_.pack_vec([m.linear_o.bias], dt, dev)))
        if template_mask is None:
            template_mask = t.new_ones(NT)
        tm = template_mask.to(device=dev, dtype=torch.float32).reshape(NT)
        bias = (self.inf * (tm - 1.0)).contiguous()
        any_valid = (tm.sum() > 0).to(torch.float32).reshape(1)            # stays on the device: no host round trip
        q = F_.linear(z.contiguous().view(P, self.c_z), wq, None, hc)
        kv = F_.linear(t.contiguous().view(NT * P, self.c_t), wkv, None, 2 * hc)
        o = torch.empty(P, hc, dtype=dt, device=dev)
        _lib.pointwise_attention_core(o, q, kv, bias, P=P, H=H, D=D, NT=NT, kv_st=P * 2 * hc, kv_sp=2 * hc, v_off=hc,
                                      out_scale=any_valid)
        del q, kv
        out = F_.linear(o, wo, (bo * any_valid).to(dt), self.c_z, out=resid, resid=resid)   # in place with a residual
        return out.view(r, r, self.c_z)

    def _train(self, t, z, template_mask):
        """template.py:100-127 with the generic attention of nn/primitives.py:390-440 written out (gating off): the
        softmax runs over at most 8 templates per pair position, in fp32."""
        m, H, D = self.mha, self.no_heads, self.c_hidden
        if template_mask is None:
            template_mask = t.new_ones(t.shape[0])
        tm = template_mask.to(device=z.device, dtype=torch.float32)
        q = m.linear_q(z).unflatten(-1, (H, D)) * (float(D) ** -0.5)           # [r, r, H, D]
        k = m.linear_k(t).unflatten(-1, (H, D))                               # [NT, r, r, H, D]
        v = m.linear_v(t).unflatten(-1, (H, D))
        logits = (q.unsqueeze(0).float() * k.float()).sum(-1) + (self.inf * (tm - 1.0)).view(-1, 1, 1, 1)
        w = torch.softmax(logits, dim=0).to(v.dtype)                           # [NT, r, r, H]
        o = (w.unsqueeze(-1) * v).sum(0).flatten(-2)                           # [r, r, H * D]
        return m.linear_o(o) * (tm.sum() > 0).to(z.dtype)

    def forward(self, t: torch.Tensor, z: torch.Tensor, template_mask: Optional[torch.Tensor] = None,
                chunk_size: Optional[int] = None) -> torch.Tensor:
        """t [N_templ, N_res, N_res, C_t], z [N_res, N_res, C_z], template_mask [N_templ]
        -> the pair update [N_res, N_res, C_z] (not yet added to z)."""
        if _needs_grad(self, t, z):
            F_.check_cuda(t, z, template_mask)
            return self._train(t, z, template_mask)
        return self._run(t, z, template_mask, None)

    def inplace(self, t: torch.Tensor, z: torch.Tensor, template_mask: Optional[torch.Tensor] = None,
                chunk_size: Optional[int] = None) -> torch.Tensor:
        """Same, with the update added to z in place; returns z."""
        zc = z.contiguous()
        out = self._run(t, zc, template_mask, zc.view(-1, self.c_z))
        if zc.data_ptr() != z.data_ptr():
            z.copy_(out)
            return z
        return out


class TemplatePairBlock(nn.Module):

    def __init__(self, c_t: int, c_hidden_tri_att: int, c_hidden_tri_mul: int, no_heads: int,
                 pair_transition_n: int, dropout_rate: float, inf: float, first_block: bool, last_block: bool,
                 **kwargs):
        super(TemplatePairBlock, self).__init__()
        self.first_block = first_block
        self.last_block = last_block
        self.c_t = c_t
        self.c_hidden_tri_att = c_hidden_tri_att
        self.c_hidden_tri_mul = c_hidden_tri_mul
        self.n_head = no_heads
        self.p_drop = dropout_rate
        self.hidden_c = int(c_t / self.n_head)
        self.TriangleMultiplicationOutgoing = AsyncChunkTriangleMultiplicationOutgoing(
            self.c_t, p_drop=self.p_drop, c=self.c_hidden_tri_mul)
        self.TriangleMultiplicationIncoming = AsyncChunkTriangleMultiplicationIncoming(
            self.c_t, p_drop=self.p_drop, c=self.c_hidden_tri_mul)
        self.TriangleAttentionStartingNode = ChunkTriangleAttentionStartingNode(
            self.c_t, p_drop=self.p_drop, c=self.c_hidden_tri_att, n_head=self.n_head)
        self.TriangleAttentionEndingNode = ChunkTriangleAttentionEndingNode(
            self.c_t, p_drop=self.p_drop, c=self.c_hidden_tri_att, n_head=self.n_head)
        self.PairTransition = ChunkTransition(d=self.c_t, n=pair_transition_n)

    def _core(self, z, mask, inplace: bool):
        """z [1, r, r, c_t] contiguous, mask [1, r, r]; order as template.py:248-256."""
        F_.check_nonempty("TemplatePairBlock", z)
        if _needs_grad(self, z):
            z = self.TriangleAttentionStartingNode(z, mask)
            z = self.TriangleAttentionEndingNode(z, mask)
            z = self.TriangleMultiplicationOutgoing(z, mask)
            z = self.TriangleMultiplicationIncoming(z, mask)
            return self.PairTransition(z)
        out = z if inplace else torch.empty_like(z)
        self.TriangleAttentionStartingNode._run(z, mask, out)
        self.TriangleAttentionEndingNode._run(out, mask, out)
        self.TriangleMultiplicationOutgoing._run(out, mask, out)
        self.TriangleMultiplicationIncoming._run(out, mask, out)
        self.PairTransition._run(out, out)
        return out

    def _enter(self, z, r):
        if z.dim() != 4 or z.shape[0] != 1:
            raise RuntimeError("TemplatePairBlock: expected one template, [1, r, r, c_t], got %s" % (tuple(z.shape),))
        if self.first_block:
            return z.contiguous()
        if z.shape[1] != r + 1:
            raise RuntimeError("TemplatePairBlock: a non-first block expects the padded [1, r+1, r+1, c_t] input, "
                               "got %s" % (tuple(z.shape),))
        return z[:, :r, :r, :].contiguous()

    def _leave(self, z):
        return z if self.last_block else F.pad(z, (0, 0, 0, 1, 0, 1))

    def forward(self, z: torch.Tensor, mask: torch.Tensor, chunk_size: Optional[int] = None,
                _mask_trans: bool = True):
        r = mask.size(-1)
        return self._leave(self._core(self._enter(z, r), mask, inplace=not self.first_block))

    def inplace(self, z, mask: torch.Tensor, chunk_size: Optional[int] = None, _mask_trans: bool = True):
        r = mask.size(-1)
        z[0] = self._leave(self._core(self._enter(z[0], r), mask, inplace=True))
        return z


class TemplatePairStack(nn.Module):
    """Implements Algorithm 16."""

    def __init__(self, c_t, c_hidden_tri_att, c_hidden_tri_mul, no_blocks, no_heads, pair_transition_n,
                 dropout_rate, blocks_per_ckpt, inf=1e9, **kwargs):
        super(TemplatePairStack, self).__init__()
        self.blocks_per_ckpt = blocks_per_ckpt
        self.blocks = nn.ModuleList()
        for block_id in range(no_blocks):
            self.blocks.append(TemplatePairBlock(
                c_t=c_t, c_hidden_tri_att=c_hidden_tri_att, c_hidden_tri_mul=c_hidden_tri_mul, no_heads=no_heads,
                pair_transition_n=pair_transition_n, dropout_rate=dropout_rate, inf=inf,
                first_block=(block_id == 0), last_block=(block_id == no_blocks - 1)))
        self.layer_norm = LayerNorm(c_t)

    def _run(self, t, mask, inplace: bool):
        if t.dim() != 4:
            raise RuntimeError("TemplatePairStack: expected [N_templ, r, r, c_t], got %s" % (tuple(t.shape),))
        if mask.shape[-3] == 1:
            mask = mask.expand(t.shape[0], *mask.shape[-2:])
        if _needs_grad(self, t):
            outs = []
            for i in range(t.shape[0]):
                z = t[i:i + 1]
                for b in self.blocks:
                    z = b._core(z, mask[i:i + 1], inplace=False)
                outs.append(self.layer_norm(z[0]))
            return torch.stack(outs, 0)
        out = t if (inplace and t.is_contiguous()) else torch.empty_like(t, memory_format=torch.contiguous_format)
        for i in range(t.shape[0]):
            with F_.mask_cache():
                z = t[i:i + 1].contiguous()
                own = z.data_ptr() != t[i].data_ptr()          # a fresh copy may be overwritten
                for k, b in enumerate(self.blocks):
                    z = b._core(z, mask[i:i + 1], inplace=(inplace or own or k > 0))
            out[i] = self.layer_norm(z[0])
        return out

    def forward(self, t: torch.tensor, mask: torch.tensor, chunk_size: int, _mask_trans: bool = True):
        """t [N_templ, N_res, N_res, C_t], mask [N_templ or 1, N_res, N_res] -> update of the same shape;
        the input is left untouched."""
        return self._run(t, mask, inplace=False)

    def inplace(self, t, mask: torch.tensor, chunk_size: int, _mask_trans: bool = True):
        """``t`` is a one-element list whose tensor is overwritten (template.py:404-434)."""
        t[0] = self._run(t[0], mask, inplace=True)
        return t
