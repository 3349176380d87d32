"""Evoformer block and 48-block stack with the reference's interface
(fastfold/model/fastnn/evoformer.py:17-332), single GPU (DAP size 1).

Padding contract.  The reference pads the residue axis by ``padding_size = 1`` in the first
block even at DAP size 1, carries ``[1, s, r+1, c]`` / ``[1, r+1, r+1, c]`` tensors between
blocks and strips the pad in the last block (evoformer.py:42-62,78-89).  The padded key is
masked in every attention and every masked projection, and padded rows are discarded, so
results on the un-padded region do not depend on it.  ``Evoformer.forward`` keeps that
*interface* (same shapes in and out for first / middle / last blocks) but computes on the
un-padded region only; ``EvoformerStack`` never materialises the pad at all.
"""
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _fused as F_
from .msa import MSACore
from .ops import Linear, OutProductMean, _needs_grad
from .triangle import PairCore


def _private_copy(view, owner):
    out = view.contiguous()
    return out.clone() if out.data_ptr() == owner.data_ptr() else out


class _BlockRecompute(torch.autograd.Function):
    """One Evoformer block as its own checkpoint: the forward pass runs the fused launches (nothing of it is kept but
    the two inputs and the dropout multipliers, which are drawn here so that both passes see the same ones); the
    backward pass re-runs the block operator by operator with autograd on, the way block checkpointing re-runs it
    (fastfold/utils/checkpointing.py:55-73; evoformer.py:262-266), and back-propagates through that."""

    @staticmethod
    def forward(ctx, block, msa_mask, pair_mask, drops, _grad_anchor, m, z):
        ctx.block, ctx.masks, ctx.drops = block, (msa_mask, pair_mask), drops
        ctx.save_for_backward(m, z)
        return block._core(m.contiguous(), z.contiguous(), msa_mask, pair_mask, inplace=False, drops=drops)

    @staticmethod
    def backward(ctx, dm, dz):
        m, z = ctx.saved_tensors
        with torch.enable_grad():
            m_, z_ = m.detach().requires_grad_(True), z.detach().requires_grad_(True)
            mo, zo = ctx.block._core_train(m_, z_, *ctx.masks, drops=ctx.drops if ctx.drops is not None else {})
        torch.autograd.backward((mo, zo), (dm, dz))        # parameter gradients accumulate here, as under checkpointing
        return None, None, None, None, None, m_.grad, z_.grad


class Evoformer(nn.Module):

    # A call that autograd has to see runs the fused forward and re-runs the block in the backward pass
    # (_BlockRecompute).  False: the forward itself is the operator-by-operator composition, every intermediate is
    # kept, and the backward pass re-runs nothing.
    recompute_in_backward = True

    def __init__(self, c_m: int, c_z: int, first_block: bool, last_block: bool, is_multimer: bool = False):
        super(Evoformer, self).__init__()
        self.first_block = first_block
        self.last_block = last_block
        self.msa = MSACore(c_m, c_z, p_drop=0.15)
        self.communication = OutProductMean(n_feat=c_m, n_feat_out=c_z, n_feat_proj=32)
        self.pair = PairCore(d_pair=c_z)
        self.is_multimer = is_multimer

    # -- un-padded core on [1, s, r, c_m] / [1, r, r, c_z] / [1, s, r] / [1, r, r] ----------
    def _core(self, m, z, msa_mask, pair_mask, inplace: bool, tails=(None, None), drops=None):
        """``tails = (m_tail, z_tail)``: int8 tails of m / z as extended residual streams (the stack's bf16 mode),
        or None for the plain stream of the reference.  ``drops``: None, or the dropout multipliers of a training-mode
        pass (``_draw_drops``; out-of-place only)."""
        F_.check_nonempty("Evoformer", m, z)
        mt, zt = tails
        if self.is_multimer:
            # multimer order (evoformer.py:70-76, 133-137): outer product mean first, the MSA stack reads the
            # pair tensor it leaves, the pair stack runs last
            z_new = z if inplace else torch.empty_like(z)
            self.communication._run(m, msa_mask, z, z_new, zt)
            m = self.msa.inplace(m, z_new, msa_mask, mt) if inplace else self.msa.forward(m, z_new, msa_mask, mt, drops=drops)
            self.pair.inplace([z_new], pair_mask, zt, drops=drops)
            return m, z_new
        if inplace:
            m = self.msa.inplace(m, z, msa_mask, mt)
            self.communication._run(m, msa_mask, z, z, zt)
            self.pair.inplace([z], pair_mask, zt)
            return m, z
        m = self.msa.forward(m, z, msa_mask, mt, drops=drops)
        z_new = torch.empty_like(z)
        self.communication._run(m, msa_mask, z, z_new, zt)
        self.pair.inplace([z_new], pair_mask, zt, drops=drops)
        return m, z_new

    def _core_train(self, m, z, msa_mask, pair_mask, drops=None):
        """The differentiable block (evoformer.py:64-76) on the un-padded tensors: every update is out of place and
        made of operators with a backward pass.  ``drops``: None (every module draws its own dropout mask in training
        mode) or the multipliers drawn by the caller (a dict, possibly empty: no dropout)."""
        F_.check_nonempty("Evoformer", m, z)
        if self.is_multimer:
            z_ori = self.communication(m, msa_mask, z)
            z = self.pair(z_ori, pair_mask, drops=drops)
            return self.msa(m, z_ori, msa_mask, drops=drops), z
        m = self.msa(m, z, msa_mask, drops=drops)
        z = self.communication(m, msa_mask, z)
        return m, self.pair(z, pair_mask, drops=drops)

    def _draw_drops(self, m, z):
        """Dropout multipliers (0 or 1 / (1 - p)) of one training-mode pass of this block, one tensor per update that
        the reference drops (msa.py:70-73; triangle.py:66-75,122-131,168-173,215-222): shared along the rows, except for
        the ending-node attention, which shares them along the columns.  None in eval mode."""
        if not self.training:
            return None
        r = z.shape[-2]

        def draw(p, shape):
            return F.dropout(torch.ones(shape, dtype=z.dtype, device=z.device), p=p, training=True) if p > 0 else None
        pair = self.pair
        d = {"row": draw(self.msa.MSARowAttentionWithPairBias.p_drop, (1, 1, r, m.shape[-1])),
             "tmo": draw(pair.TriangleMultiplicationOutgoing.p_drop, (1, 1, r, z.shape[-1])),
             "tmi": draw(pair.TriangleMultiplicationIncoming.p_drop, (1, 1, r, z.shape[-1])),
             "tas": draw(pair.TriangleAttentionStartingNode.p_drop, (1, 1, r, z.shape[-1])),
             "tae": draw(pair.TriangleAttentionEndingNode.p_drop, (1, r, 1, z.shape[-1]))}
        return {k: v for k, v in d.items() if v is not None}

    def _run_grad(self, m, z, msa_mask, pair_mask):
        """The block under autograd, on the un-padded [1, ...] tensors."""
        if not self.recompute_in_backward:
            return self._core_train(m, z, msa_mask, pair_mask)
        anchor = torch.empty(0, device=m.device, requires_grad=True)     # outputs need a gradient even when m and z do not
        return _BlockRecompute.apply(self, msa_mask, pair_mask, self._draw_drops(m, z), anchor, m, z)

    def _enter(self, m, z, r):
        if self.first_block:
            return m.unsqueeze(0).contiguous(), z.unsqueeze(0).contiguous()
        if m.dim() != 4 or z.dim() != 4 or m.shape[2] != r + 1 or z.shape[1] != r + 1:
            raise RuntimeError("Evoformer: a non-first block expects padded [1, s, r+1, c] / [1, r+1, r+1, c] "
                               "inputs, got %s / %s" % (tuple(m.shape), tuple(z.shape)))
        # the core runs in place on these: they must be copies even where the un-padding slice is already
        # contiguous (a single sequence, a single residue) and ``.contiguous()`` would hand back the caller's memory
        return _private_copy(m[:, :, :r, :], m), _private_copy(z[:, :r, :r, :], z)

    def _leave(self, m, z):
        if self.last_block:
            return m.squeeze(0), z.squeeze(0)
        return F.pad(m, (0, 0, 0, 1)), F.pad(z, (0, 0, 0, 1, 0, 1))

    def forward(self, m: torch.Tensor, z: torch.Tensor, msa_mask: torch.Tensor, pair_mask: torch.Tensor,
                chunk_size: Optional[int] = None, _mask_trans: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
        """``chunk_size`` and ``_mask_trans`` are accepted and ignored, as in the reference
        (evoformer.py:36-37): chunking is the process-global ``set_chunk_size`` and transitions
        are never masked."""
        r = pair_mask.size(-1)
        if _needs_grad(self, m, z):
            if self.first_block:
                m, z = m.unsqueeze(0), z.unsqueeze(0)
            else:
                m, z = m[:, :, :r, :], z[:, :r, :r, :]
            return self._leave(*self._run_grad(m, z, msa_mask.unsqueeze(0), pair_mask.unsqueeze(0)))
        m, z = self._enter(m, z, r)
        m, z = self._core(m, z, msa_mask.unsqueeze(0), pair_mask.unsqueeze(0), inplace=not self.first_block)
        return self._leave(m, z)

    def inplace(self, m, z, msa_mask: torch.Tensor, pair_mask: torch.Tensor, chunk_size: Optional[int] = None,
                _mask_trans: bool = True):
        """List-passing variant (evoformer.py:93-152): ``m`` and ``z`` are one-element lists whose
        tensors are updated / rebound."""
        r = pair_mask.size(-1)
        if self.first_block:
            mm, zz = m[0].unsqueeze(0), z[0].unsqueeze(0)
            if not mm.is_contiguous() or not zz.is_contiguous():
                mm, zz = mm.contiguous(), zz.contiguous()
        else:
            mm, zz = self._enter(m[0], z[0], r)
        mm, zz = self._core(mm, zz, msa_mask.unsqueeze(0), pair_mask.unsqueeze(0), inplace=True)
        m[0], z[0] = self._leave(mm, zz)
        return m, z


class EvoformerStack(nn.Module):
    """Main Evoformer trunk (Algorithm 6): ``no_blocks`` blocks, then ``s = Linear(c_m, c_s)(m[0])``."""

    # bf16 / fp16 runs keep eight extra mantissa bits of both residual streams in int8 side tensors between the
    # blocks (see "extended residual stream" in include/ffk.h): rounding m and z to bf16 after each of the ~430
    # sub-updates of 48 blocks alone costs 2e-2 .. 3e-2 relative L2 at the output.  False = the reference's plain stream.
    extended_residual = True

    def __init__(self, c_m: int, c_z: int, c_s: int, no_blocks: int, blocks_per_ckpt: int,
                 clear_cache_between_blocks: bool = False, is_multimer: bool = False, **kwargs):
        super(EvoformerStack, self).__init__()
        self.blocks_per_ckpt = blocks_per_ckpt
        self.clear_cache_between_blocks = clear_cache_between_blocks
        self.blocks = nn.ModuleList()
        for block_id in range(no_blocks):
            self.blocks.append(Evoformer(c_m=c_m, c_z=c_z, first_block=(block_id == 0),
                                         last_block=(block_id == no_blocks - 1), is_multimer=is_multimer))
        self.linear = Linear(c_m, c_s)

    def _run(self, m, z, msa_mask, pair_mask, inplace_first: bool):
        mm, zz = m.unsqueeze(0), z.unsqueeze(0)
        mk, pk = msa_mask.unsqueeze(0), pair_mask.unsqueeze(0)
        tails = (None, None)
        if self.extended_residual and mm.dtype == torch.bfloat16 and mm.is_cuda:
            # zero tails: the inputs are exact bf16 values; the tails die with this call, the bf16 tensors they
            # leave are the correctly rounded results
            tails = (torch.zeros(mm.shape, dtype=torch.int8, device=mm.device),
                     torch.zeros(zz.shape, dtype=torch.int8, device=zz.device))
        with F_.mask_cache():          # key biases / normalisers depend on the masks only: once per stack, not per block
            for i, b in enumerate(self.blocks):
                if self.clear_cache_between_blocks:
                    torch.cuda.empty_cache()
                mm, zz = b._core(mm.contiguous(), zz.contiguous(), mk, pk, inplace=(inplace_first or i > 0), tails=tails)
        return mm.squeeze(0), zz.squeeze(0)

    def _run_train(self, m, z, msa_mask, pair_mask):
        """The differentiable stack: plain residual stream, blocks re-run in the backward pass in groups of
        ``blocks_per_ckpt`` while the module is in training mode (evoformer.py:262-266)."""
        from torch.utils.checkpoint import checkpoint
        mm, zz = m.unsqueeze(0), z.unsqueeze(0)
        mk, pk = msa_mask.unsqueeze(0), pair_mask.unsqueeze(0)
        blocks = list(self.blocks)
        per = self.blocks_per_ckpt if (self.training and self.blocks_per_ckpt) else None

        def run(group, a, b):
            for blk in group:
                if self.clear_cache_between_blocks:
                    torch.cuda.empty_cache()
                a, b = blk._core_train(a, b, mk, pk)
            return a, b
        if per is None:
            mm, zz = run(blocks, mm, zz)
        elif all(blk.recompute_in_backward for blk in blocks):
            # every block its own checkpoint, with a fused forward (at least as fine as groups of blocks_per_ckpt)
            for blk in blocks:
                if self.clear_cache_between_blocks:
                    torch.cuda.empty_cache()
                mm, zz = blk._run_grad(mm, zz, mk, pk)
        else:
            for i in range(0, len(blocks), per):
                mm, zz = checkpoint(run, blocks[i:i + per], mm, zz, use_reentrant=False)
        return mm.squeeze(0), zz.squeeze(0)

    def forward(self, m: torch.Tensor, z: torch.Tensor, msa_mask: torch.Tensor, pair_mask: torch.Tensor,
                chunk_size: int = None, _mask_trans: bool = True
                ) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
        """
        m [N_seq, N_res, C_m], z [N_res, N_res, C_z], msa_mask [N_seq, N_res], pair_mask [N_res, N_res]
        -> (m, z, s [N_res, C_s]).  Inputs are left untouched.
        """
        if _needs_grad(self, m, z):
            m, z = self._run_train(m, z, msa_mask, pair_mask)
            return m, z, self.linear(m[..., 0, :, :])
        m, z = self._run(m, z, msa_mask, pair_mask, inplace_first=False)
        s = self.linear(m[..., 0, :, :])
        return m, z, s

    def inplace(self, m, z, msa_mask: torch.Tensor, pair_mask: torch.Tensor, chunk_size: int = None,
                _mask_trans: bool = True):
        """``m`` / ``z`` are one-element lists; their tensors are overwritten (evoformer.py:280-332)."""
        contiguous = m[0].is_contiguous() and z[0].is_contiguous()
        mm, zz = self._run(m[0], z[0], msa_mask, pair_mask, inplace_first=contiguous)
        m[0], z[0] = mm, zz
        s = self.linear(m[0][..., 0, :, :])
        return m, z, s
