"""MSA stack of the Evoformer block: row attention with pair bias, column attention,
transition - same classes and parameters as fastfold/model/fastnn/msa.py:33-151."""
import math

import torch
import torch.nn as nn

from fastfold_amd.model.fastnn.kernel import LayerNorm
from . import _fused as F_
from .ops import SelfAttention, Transition, _PackMixin, _ln_pair, _mask_like, _no_grad_guard


class MSARowAttentionWithPairBias(nn.Module, _PackMixin):

    def __init__(self, d_node, d_pair, c=32, n_head=8, p_drop=0.15):
        super(MSARowAttentionWithPairBias, self).__init__()
        self.d_node = d_node
        self.d_pair = d_pair
        self.c = c
        self.n_head = n_head
        self.p_drop = p_drop

        self.layernormM = LayerNorm(d_node)
        self.layernormZ = LayerNorm(d_pair)

        _init_weights = torch.nn.init.normal_(torch.zeros([n_head, d_pair]), std=1.0 / math.sqrt(d_pair))
        self.linear_b_weights = nn.parameter.Parameter(data=_init_weights, requires_grad=True)

        self.attention = SelfAttention(qkv_dim=d_node, c=c, n_head=n_head, out_dim=d_node, gating=True,
                                       last_bias_fuse=True)
        self.out_bias = nn.parameter.Parameter(data=torch.zeros((d_node,)), requires_grad=True)

    def _run(self, M_raw, Z, M_mask, out):
        F_.check_cuda(M_raw, Z, M_mask)
        _no_grad_guard(self, M_raw, Z)
        dt, dev = M_raw.dtype, M_raw.device
        self.attention._check(dt)
        if M_raw.dim() != 4 or M_raw.shape[0] != 1:
            raise RuntimeError("MSARowAttentionWithPairBias: expected [1, s, r, C], got %s" % (tuple(M_raw.shape),))
        _, s, r, C = M_raw.shape
        Cz = Z.shape[-1]
        if not F_.fits_fused(Cz, dt):
            raise RuntimeError("MSARowAttentionWithPairBias: unsupported pair width %d" % Cz)
        wb = self._packed(("wb", dt, dev), [self.linear_b_weights],
                          lambda: F_.pack_rows([self.linear_b_weights], dt, dev))
        ob = self._packed(("ob", dt, dev), [self.out_bias], lambda: F_.pack_vec([self.out_bias], dt, dev))
        w_pk, gb_pk, wo_pk = self.attention.packed(dt, dev)
        pbs = self._packed(("pbs", dt, dev), [self.linear_b_weights, self.layernormZ.weight, self.layernormZ.bias],
                           lambda: F_.PairBiasScratch(Cz, dev))
        bias_t = F_.pair_bias(Z.contiguous(), r=r, C=Cz, H=self.n_head, ln=_ln_pair(self.layernormZ, dt), wb_pk=wb,
                              pb_scratch=pbs)
        mask = _mask_like(M_mask, M_raw)[0]
        F_.attention(M_raw, out, M_raw, B2=s, N=r, C=C, H=self.n_head, a_map=(s * r, 0, C),
                     ln=_ln_pair(self.layernormM, dt), w_pk=w_pk, gate_bias_pk=gb_pk, wo_pk=wo_pk, out_bias_pk=ob,
                     c_out=C, mask=mask, mask_sb=r, mask_sn=1, bias_t=bias_t)
        return out

    def forward(self, M_raw, Z, M_mask):
        M_raw = M_raw.contiguous()
        return self._run(M_raw, Z, M_mask, torch.empty_like(M_raw))


class MSAColumnAttention(nn.Module, _PackMixin):

    def __init__(self, d_node, c=32, n_head=8):
        super(MSAColumnAttention, self).__init__()
        self.d_node = d_node
        self.c = c
        self.n_head = n_head

        self.layernormM = LayerNorm(d_node)
        self.attention = SelfAttention(qkv_dim=d_node, c=c, n_head=n_head, out_dim=d_node, gating=True)

    def _run(self, M_raw, M_mask, out):
        F_.check_cuda(M_raw, M_mask)
        _no_grad_guard(self, M_raw)
        dt, dev = M_raw.dtype, M_raw.device
        self.attention._check(dt)
        if M_raw.dim() != 4 or M_raw.shape[0] != 1:
            raise RuntimeError("MSAColumnAttention: expected [1, s, r, C], got %s" % (tuple(M_raw.shape),))
        _, s, r, C = M_raw.shape
        w_pk, gb_pk, wo_pk = self.attention.packed(dt, dev)
        ob = self._packed(("ob", dt, dev), [self.attention.o_linear.bias],
                          lambda: F_.pack_vec([self.attention.o_linear.bias], dt, dev))
        mask = _mask_like(M_mask, M_raw)[0]            # [s, r]; keys run along s for each residue
        # logical row (j, s') reads m[s', j]
        F_.attention(M_raw, out, M_raw, B2=r, N=s, C=C, H=self.n_head, a_map=(s, C, r * C),
                     ln=_ln_pair(self.layernormM, dt), w_pk=w_pk, gate_bias_pk=gb_pk, wo_pk=wo_pk, out_bias_pk=ob,
                     c_out=C, mask=mask, mask_sb=1, mask_sn=r)
        return out

    def forward(self, M_raw, M_mask):
        M_raw = M_raw.contiguous()
        return self._run(M_raw, M_mask, torch.empty_like(M_raw))


class MSACore(nn.Module):

    def __init__(self, d_node, d_pair, p_drop=0.15):
        super(MSACore, self).__init__()
        self.MSARowAttentionWithPairBias = MSARowAttentionWithPairBias(d_node=d_node, d_pair=d_pair, p_drop=p_drop)
        self.MSAColumnAttention = MSAColumnAttention(d_node=d_node)
        self.MSATransition = Transition(d=d_node)

    def forward(self, node, pair, node_mask):
        """node [1, s, r, d_node], pair [1, r, r, d_pair], node_mask [1, s, r] -> new node
        (the input tensor is left untouched; the two later updates run in place on the copy)."""
        node = node.contiguous()
        out = torch.empty_like(node)
        self.MSARowAttentionWithPairBias._run(node, pair, node_mask, out)
        self.MSAColumnAttention._run(out, node_mask, out)
        self.MSATransition._run(out, out)
        return out

    def inplace(self, node, pair, node_mask):
        self.MSARowAttentionWithPairBias._run(node, pair, node_mask, node)
        self.MSAColumnAttention._run(node, node_mask, node)
        self.MSATransition._run(node, node)
        return node
