"""Pair stack of the Evoformer block (fastfold/model/fastnn/triangle.py:216-271)."""
import torch
import torch.nn as nn

from .ops import (AsyncChunkTriangleMultiplicationIncoming, AsyncChunkTriangleMultiplicationOutgoing,
                  ChunkTransition, ChunkTriangleAttentionEndingNode, ChunkTriangleAttentionStartingNode, _needs_grad)


class PairCore(nn.Module):

    def __init__(self, d_pair, p_drop=0.25):
        super(PairCore, self).__init__()
        self.d_pair = d_pair
        self.n_head = 4
        self.hidden_c = int(d_pair / self.n_head)

        self.TriangleMultiplicationOutgoing = AsyncChunkTriangleMultiplicationOutgoing(d_pair, p_drop=p_drop, c=d_pair)
        self.TriangleMultiplicationIncoming = AsyncChunkTriangleMultiplicationIncoming(d_pair, p_drop=p_drop, c=d_pair)
        self.TriangleAttentionStartingNode = ChunkTriangleAttentionStartingNode(d_pair, p_drop=p_drop,
                                                                                c=self.hidden_c, n_head=self.n_head)
        self.TriangleAttentionEndingNode = ChunkTriangleAttentionEndingNode(d_pair, p_drop=p_drop,
                                                                            c=self.hidden_c, n_head=self.n_head)
        self.PairTransition = ChunkTransition(d=d_pair)

    def forward(self, pair, pair_mask, xtail=None, drops=None):
        """pair [1, r, r, d_pair], pair_mask [1, r, r] -> new pair (input untouched).  ``xtail``: int8 tail of the
        pair tensor as an extended residual stream (read with the input, rewritten for the output).  ``drops``: None,
        or a dict with the dropout multipliers of a training-mode call drawn by the caller (keys "tmo", "tmi", "tas":
        [1, 1, r, d_pair]; "tae": [1, r, 1, d_pair])."""
        d = drops or {}
        if _needs_grad(self, pair):
            if xtail is not None:
                raise RuntimeError("PairCore: the extended residual stream is forward-only")
            if drops is not None:
                pair = self.TriangleMultiplicationOutgoing._train(pair, pair_mask, drop=d.get("tmo"))
                pair = self.TriangleMultiplicationIncoming._train(pair, pair_mask, drop=d.get("tmi"))
                pair = self.TriangleAttentionStartingNode._train(pair, pair_mask, drop=d.get("tas"))
                pair = self.TriangleAttentionEndingNode._train(pair, pair_mask, drop=d.get("tae"))
                return self.PairTransition(pair)
            pair = self.TriangleMultiplicationOutgoing(pair, pair_mask)
            pair = self.TriangleMultiplicationIncoming(pair, pair_mask)
            pair = self.TriangleAttentionStartingNode(pair, pair_mask)
            pair = self.TriangleAttentionEndingNode(pair, pair_mask)
            return self.PairTransition(pair)
        pair = pair.contiguous()
        out = torch.empty_like(pair)
        self.TriangleMultiplicationOutgoing._run(pair, pair_mask, out, xtail, drop=d.get("tmo"))
        self._rest(out, pair_mask, xtail, d)
        return out

    def _rest(self, z, pair_mask, xtail=None, d=None):
        d = d or {}
        self.TriangleMultiplicationIncoming._run(z, pair_mask, z, xtail, drop=d.get("tmi"))
        self.TriangleAttentionStartingNode._run(z, pair_mask, z, xtail, drop=d.get("tas"))
        self.TriangleAttentionEndingNode._run(z, pair_mask, z, xtail, drop=d.get("tae"))
        self.PairTransition._run(z, z, xtail)

    def inplace(self, pair, pair_mask, xtail=None, drops=None):
        pair[0] = pair[0].contiguous()
        self.TriangleMultiplicationOutgoing._run(pair[0], pair_mask, pair[0], xtail, drop=(drops or {}).get("tmo"))
        self._rest(pair[0], pair_mask, xtail, drops)
        return pair
