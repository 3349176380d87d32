"""MSA stack of the Evoformer block: row attention with pair bias, column attention,
transition - same classes and parameters as fastfold/model/fastnn/msa.py:33-151 - and the
extra-MSA core / block / stack (msa.py:154-464), whose column attention is the global one."""
import math
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from fastfold_amd.model.fastnn.kernel import LayerNorm
from . import _fused as F_
from .ops import (ChunkMSAColumnGlobalAttention, ChunkTransition, OutProductMean, SelfAttention, Transition,
                  _PackMixin, _budget, _check_tail, _ln_pair, _mask_like, _needs_grad, _no_grad_guard)
from .triangle import PairCore


def _private_copy(view, owner):
    out = view.contiguous()
    return out.clone() if out.data_ptr() == owner.data_ptr() else out


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

    def _run(self, M_raw, Z, M_mask, out, xtail=None, drop=None):
        """``drop``: None or the [1, 1, r, C] dropout multipliers of a training-mode call (drawn by the caller)."""
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
                     c_out=C, mask=mask, mask_sb=r, mask_sn=1, bias_t=bias_t, head_dim=self.c, budget=_budget(),
                     xtail=_check_tail(xtail, M_raw), drop=None if drop is None else drop.reshape(r, C).contiguous())
        return out

    def _train(self, M_raw, Z, M_mask, drop=None):
        """msa.py:60-74, operator by operator.  ``drop``: dropout multipliers drawn by the caller; None = drawn here."""
        from .kernel import bias_dropout_add
        M = self.layernormM(M_raw)
        b = F.linear(self.layernormZ(Z), self.linear_b_weights.to(Z.dtype))
        M = self.attention(M, M_mask, (b, None))
        if drop is not None:
            return bias_dropout_add(M, self.out_bias, drop, M_raw, prob=0.0, training=False)
        dropout_mask = torch.ones_like(M[:, 0:1, :, :])
        return bias_dropout_add(M, self.out_bias, dropout_mask, M_raw, prob=self.p_drop, training=self.training)

    def forward(self, M_raw, Z, M_mask):
        if _needs_grad(self, M_raw, Z):
            return self._train(M_raw, Z, M_mask)
        M_raw = M_raw.contiguous()
        return self._run(M_raw, Z, M_mask, torch.empty_like(M_raw))


class ChunkMSARowAttentionWithPairBias(MSARowAttentionWithPairBias):
    """Same computation (ops.py:751-867); logits are never materialised, and the operand tiles are built a
    bounded slab of sequences at a time."""

    def inplace(self, M_raw, Z, M_mask):
        M_raw[0] = M_raw[0].contiguous()
        self._run(M_raw[0], Z, M_mask, M_raw[0])
        return M_raw


class MSAColumnAttention(nn.Module, _PackMixin):

    def __init__(self, d_node, c=32, n_head=8):
        super(MSAColumnAttention, self).__init__()
        self.d_node = d_node
        self.c = c
        self.n_head = n_head

        self.layernormM = LayerNorm(d_node)
        self.attention = SelfAttention(qkv_dim=d_node, c=c, n_head=n_head, out_dim=d_node, gating=True)

    def _run(self, M_raw, M_mask, out, xtail=None):
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
                     c_out=C, mask=mask, mask_sb=1, mask_sn=r, head_dim=self.c, budget=_budget(),
                     xtail=_check_tail(xtail, M_raw))
        return out

    def _train(self, M_raw, M_mask):
        """msa.py:92-104, operator by operator."""
        M = self.layernormM(M_raw.transpose(-2, -3))
        M = self.attention(M, M_mask.transpose(-1, -2))
        return M_raw + M.transpose(-2, -3)

    def forward(self, M_raw, M_mask):
        if _needs_grad(self, M_raw):
            return self._train(M_raw, M_mask)
        M_raw = M_raw.contiguous()
        return self._run(M_raw, M_mask, torch.empty_like(M_raw))


class MSACore(nn.Module):

    def __init__(self, d_node, d_pair, p_drop=0.15):
        super(MSACore, self).__init__()
        self.MSARowAttentionWithPairBias = MSARowAttentionWithPairBias(d_node=d_node, d_pair=d_pair, p_drop=p_drop)
        self.MSAColumnAttention = MSAColumnAttention(d_node=d_node)
        self.MSATransition = Transition(d=d_node)

    def forward(self, node, pair, node_mask, xtail=None, drops=None):
        """node [1, s, r, d_node], pair [1, r, r, d_pair], node_mask [1, s, r] -> new node
        (the input tensor is left untouched; the two later updates run in place on the copy).
        ``xtail``: int8 tail of the *new* node tensor as an extended residual stream (zero on entry when the input
        is a plain bf16 tensor).  ``drops``: None, or a dict with the dropout multipliers of a training-mode call
        drawn by the caller (key "row": [1, 1, r, d_node])."""
        drop = None if drops is None else drops.get("row")
        if _needs_grad(self, node, pair):
            if xtail is not None:
                raise RuntimeError("MSACore: the extended residual stream is forward-only")
            if drop is not None:
                node = self.MSARowAttentionWithPairBias._train(node, pair, node_mask, drop=drop)
            else:
                node = self.MSARowAttentionWithPairBias(node, pair, node_mask)
            node = self.MSAColumnAttention(node, node_mask)
            return self.MSATransition(node)
        node = node.contiguous()
        out = torch.empty_like(node)
        self.MSARowAttentionWithPairBias._run(node, pair, node_mask, out, xtail, drop=drop)
        self.MSAColumnAttention._run(out, node_mask, out, xtail)
        self.MSATransition._run(out, out, xtail)
        return out

    def inplace(self, node, pair, node_mask, xtail=None):
        self.MSARowAttentionWithPairBias._run(node, pair, node_mask, node, xtail)
        self.MSAColumnAttention._run(node, node_mask, node, xtail)
        self.MSATransition._run(node, node, xtail)
        return node


class ExtraMSACore(nn.Module):
    """Row attention with pair bias (head dim 8), global column attention, transition (msa.py:154-187)."""

    def __init__(self, d_node, d_pair, p_drop=0.15):
        super(ExtraMSACore, self).__init__()
        self.MSARowAttentionWithPairBias = ChunkMSARowAttentionWithPairBias(d_node=d_node, d_pair=d_pair,
                                                                            p_drop=p_drop, c=8)
        self.MSAColumnAttention = ChunkMSAColumnGlobalAttention(d_node=d_node, c=8)
        self.MSATransition = ChunkTransition(d=d_node)

    def forward(self, node, pair, node_mask):
        if _needs_grad(self, node, pair):
            node = self.MSARowAttentionWithPairBias(node, pair, node_mask)
            node = self.MSAColumnAttention(node, node_mask)
            return self.MSATransition(node)
        node = node.contiguous()
        out = torch.empty_like(node)
        self.MSARowAttentionWithPairBias._run(node, pair, node_mask, out)
        self.MSAColumnAttention._run(out, node_mask, out)
        self.MSATransition._run(out, out)
        return out

    def inplace(self, node, pair, node_mask):
        """``node`` is a one-element list; ``pair`` a tensor (msa.py:176-187)."""
        node[0] = node[0].contiguous()
        self.MSARowAttentionWithPairBias._run(node[0], pair, node_mask, node[0])
        self.MSAColumnAttention._run(node[0], node_mask, node[0])
        self.MSATransition._run(node[0], node[0])
        return node


class ExtraMSABlock(nn.Module):
    """One block of the extra-MSA stack (msa.py:190-345).  As for ``Evoformer``, the reference's padding
    by one sequence and one residue between blocks is kept as an interface (shapes in and out) while the
    computation runs on the un-padded region, whose results cannot depend on the masked padding."""

    def __init__(self, c_m: int, c_z: int, first_block: bool, last_block: bool, is_multimer=False):
        super(ExtraMSABlock, self).__init__()
        self.first_block = first_block
        self.last_block = last_block
        self.msa_stack = ExtraMSACore(c_m, c_z, p_drop=0.15)
        self.communication = OutProductMean(n_feat=c_m, n_feat_out=c_z, n_feat_proj=32)
        self.pair_stack = PairCore(d_pair=c_z)
        self.is_multimer = is_multimer

    def _core(self, m, z, msa_mask, pair_mask, inplace: bool):
        """m [1, s, r, c_m], z [1, r, r, c_z] contiguous, masks [1, s, r] / [1, r, r]."""
        F_.check_nonempty("ExtraMSABlock", m, z)
        if _needs_grad(self, m, z):
            # the reference's operator sequence (msa.py:226-258), nothing in place
            if self.is_multimer:
                z = self.communication(m, msa_mask, z)
                m = self.msa_stack(m, z, msa_mask)
                return m, self.pair_stack(z, pair_mask)
            m = self.msa_stack(m, z, msa_mask)
            z = self.communication(m, msa_mask, z)
            return m, self.pair_stack(z, pair_mask)
        if self.is_multimer:
            # msa.py:252-258, 321-332: outer product mean first, the MSA stack reads the pair tensor it leaves,
            # the pair stack runs last
            z_new = z if inplace else torch.empty_like(z)
            self.communication._run(m, msa_mask, z, z_new)
            m = self.msa_stack.inplace([m], z_new, msa_mask)[0] if inplace else self.msa_stack.forward(m, z_new, msa_mask)
            self.pair_stack.inplace([z_new], pair_mask)
            return m, z_new
        if inplace:
            m = self.msa_stack.inplace([m], z, msa_mask)[0]
            self.communication._run(m, msa_mask, z, z)
            self.pair_stack.inplace([z], pair_mask)
            return m, z
        m = self.msa_stack.forward(m, z, msa_mask)
        z = self.communication.forward(m, msa_mask, z)
        self.pair_stack.inplace([z], pair_mask)
        return m, z

    def _enter(self, m, z, s, r):
        if self.first_block:
            return m.unsqueeze(0).contiguous(), z.unsqueeze(0).contiguous()
        if m.dim() != 4 or z.dim() != 4 or m.shape[1] != s + 1 or m.shape[2] != r + 1 or z.shape[1] != r + 1:
            raise RuntimeError("ExtraMSABlock: a non-first block expects padded [1, s+1, r+1, c] / [1, r+1, r+1, c] "
                               "inputs, got %s / %s" % (tuple(m.shape), tuple(z.shape)))
        # private copies (the core runs in place) even where the slice is contiguous as it stands
        return _private_copy(m[:, :s, :r, :], m), _private_copy(z[:, :r, :r, :], z)

    def _leave(self, m, z):
        if self.last_block:
            return m.squeeze(0), z.squeeze(0)
        return F.pad(m, (0, 0, 0, 1, 0, 1)), F.pad(z, (0, 0, 0, 1, 0, 1))

    def forward(self, m: torch.Tensor, z: torch.Tensor, msa_mask: torch.Tensor, pair_mask: torch.Tensor,
                chunk_size: Optional[int] = None, _mask_trans: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
        s, r = msa_mask.size(-2), pair_mask.size(-1)
        m, z = self._enter(m, z, s, r)
        m, z = self._core(m, z, msa_mask.unsqueeze(0), pair_mask.unsqueeze(0), inplace=not self.first_block)
        return self._leave(m, z)

    def inplace(self, m, z, msa_mask: torch.Tensor, pair_mask: torch.Tensor, chunk_size: Optional[int] = None,
                _mask_trans: bool = True):
        s, r = msa_mask.size(-2), pair_mask.size(-1)
        mm, zz = self._enter(m[0], z[0], s, r)
        mm, zz = self._core(mm, zz, msa_mask.unsqueeze(0), pair_mask.unsqueeze(0), inplace=True)
        m[0], z[0] = self._leave(mm, zz)
        return m, z


class ExtraMSAStack(nn.Module):
    """Algorithm 18 (msa.py:347-464): ``no_blocks`` extra-MSA blocks; returns the pair representation."""

    def __init__(self, c_m: int, c_z: int, no_blocks: int, clear_cache_between_blocks: bool = False,
                 is_multimer: bool = False, **kwargs):
        super(ExtraMSAStack, self).__init__()
        self.clear_cache_between_blocks = clear_cache_between_blocks
        self.blocks = nn.ModuleList()
        for block_id in range(no_blocks):
            self.blocks.append(ExtraMSABlock(c_m=c_m, c_z=c_z, first_block=(block_id == 0),
                                             last_block=(block_id == no_blocks - 1), is_multimer=is_multimer))

    def _run(self, m, z, msa_mask, pair_mask, inplace_first: bool):
        mm, zz = m.unsqueeze(0).contiguous(), z.unsqueeze(0).contiguous()
        mk, pk = msa_mask.unsqueeze(0), pair_mask.unsqueeze(0)
        with F_.mask_cache():
            for i, b in enumerate(self.blocks):
                mm, zz = b._core(mm, zz, mk, pk, inplace=(inplace_first or i > 0))
                if self.clear_cache_between_blocks:
                    torch.cuda.empty_cache()
        return zz.squeeze(0)

    def forward(self, m: torch.Tensor, z: torch.Tensor, chunk_size: int, msa_mask: Optional[torch.Tensor] = None,
                pair_mask: Optional[torch.Tensor] = None, _mask_trans: bool = True) -> torch.Tensor:
        """m [N_extra, N_res, C_m], z [N_res, N_res, C_z], msa_mask [N_extra, N_res], pair_mask
        [N_res, N_res] -> z.  Inputs are left untouched."""
        msa_mask, pair_mask = self._masks(m, z, msa_mask, pair_mask)
        return self._run(m, z, msa_mask, pair_mask, inplace_first=False)

    def inplace(self, m, z, chunk_size: int, msa_mask: Optional[torch.Tensor] = None,
                pair_mask: Optional[torch.Tensor] = None, _mask_trans: bool = True):
        """``m`` / ``z`` are one-element lists; returns the list ``z`` as the reference does (msa.py:433-464)."""
        msa_mask, pair_mask = self._masks(m[0], z[0], msa_mask, pair_mask)
        contiguous = m[0].is_contiguous() and z[0].is_contiguous()
        z[0] = self._run(m[0], z[0], msa_mask, pair_mask, inplace_first=contiguous)
        return z

    @staticmethod
    def _masks(m, z, msa_mask, pair_mask):
        if msa_mask is None:
            msa_mask = m.new_ones(m.shape[:-1])
        if pair_mask is None:
            pair_mask = z.new_ones(z.shape[:-1])
        return msa_mask, pair_mask
