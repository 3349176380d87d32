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
from . import _fused as F_
from .ops import (AsyncChunkTriangleMultiplicationIncoming, AsyncChunkTriangleMultiplicationOutgoing,
                  ChunkTransition, ChunkTriangleAttentionEndingNode, ChunkTriangleAttentionStartingNode)


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
