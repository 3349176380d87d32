"""Input and recycling embedders with the reference's interface (fastfold/model/fastnn/ops.py:1046-1145,
1238-1334; the reference's ``inject_embedder`` swaps exactly these two, utils/inject_fastnn.py:376-416), and
the three Linear-only feature embedders of fastnn/embedders.py:257-372 (template angle / pair, extra MSA).

The r x r x c_z parts run in one launch of ``ffk_pair_embed`` each: a Linear on a one-hot vector is a pick of
one weight column, so neither the [r, r, 65] relative-position one-hot nor the [r, r, 15] distogram one-hot
is formed.  The small feature projections run on the projection kernels after zero-padding their ragged
input widths (22, 49) to a multiple of 32 on the host, target features concatenated to the MSA features so
that ``linear_msa_m(msa) + linear_tf_m(tf)`` is a single GEMM.
"""
from typing import Tuple

import torch
import torch.nn as nn

from fastfold_amd import _lib
from fastfold_amd.model.fastnn.kernel import LayerNorm
from . import _fused as F_
from . import ops as _ops
from .ops import Linear, _PackMixin, _needs_grad


def _pad_cols(x, k):
    return x if x.shape[-1] == k else torch.nn.functional.pad(x, (0, k - x.shape[-1]))


class InputEmbedder(nn.Module, _PackMixin):
    """Embeds a subset of the input features: Algorithms 3 (InputEmbedder) and 4 (relpos)."""

    def __init__(self, tf_dim: int, msa_dim: int, c_z: int, c_m: int, relpos_k: int, **kwargs):
        super(InputEmbedder, self).__init__()
        self.tf_dim = tf_dim
        self.msa_dim = msa_dim
        self.c_z = c_z
        self.c_m = c_m
        self.linear_tf_z_i = Linear(tf_dim, c_z)
        self.linear_tf_z_j = Linear(tf_dim, c_z)
        self.linear_tf_m = Linear(tf_dim, c_m)
        self.linear_msa_m = Linear(msa_dim, c_m)
        self.relpos_k = relpos_k
        self.no_bins = 2 * relpos_k + 1
        self.linear_relpos = Linear(self.no_bins, c_z)

    def _pk(self, dt, dev):
        ps = [p for l in (self.linear_tf_z_i, self.linear_tf_z_j, self.linear_tf_m, self.linear_msa_m, self.linear_relpos)
              for p in (l.weight, l.bias)]
        ktf = F_.round_up(self.tf_dim, 32)
        kmsa = F_.round_up(self.msa_dim + self.tf_dim, 32)

        def build():
            wi = F_.pack_rows([_pad_cols(self.linear_tf_z_i.weight.detach(), ktf)], dt, dev)
            wj = F_.pack_rows([_pad_cols(self.linear_tf_z_j.weight.detach(), ktf)], dt, dev)
            wm = F_.pack_rows([_pad_cols(torch.cat([self.linear_msa_m.weight.detach(), self.linear_tf_m.weight.detach()], 1),
                                         kmsa)], dt, dev)
            return (wi, F_.pack_vec([self.linear_tf_z_i.bias], dt, dev), wj, F_.pack_vec([self.linear_tf_z_j.bias], dt, dev),
                    wm, F_.pack_vec([self.linear_msa_m.bias.detach().float() + self.linear_tf_m.bias.detach().float()], dt, dev),
                    self.linear_relpos.weight.detach().t().to(dt).contiguous(),
                    self.linear_relpos.bias.detach().to(dt).contiguous())
        return (ktf, kmsa) + self._packed(("ie", dt, dev), ps, build)

    def _train(self, tf, ri, msa):
        """embedders.py:99-135, operator by operator; the one-hot of the clipped offset selects a row of the
        relative-position table."""
        dt = self.linear_relpos.weight.dtype
        tf, msa = tf.to(dt), msa.to(dt)
        pair_emb = self.linear_tf_z_i(tf)[..., None, :] + self.linear_tf_z_j(tf)[..., None, :, :]
        d = ri.to(torch.float32)
        d = (d[..., None] - d[..., None, :]).clamp(-self.relpos_k, self.relpos_k)
        d = torch.ceil(d - 0.5).long() + self.relpos_k                      # nearest offset, the lower one on a tie
        pair_emb = pair_emb + (self.linear_relpos.weight.t()[d] + self.linear_relpos.bias)
        msa_emb = self.linear_msa_m(msa) + self.linear_tf_m(tf).unsqueeze(-3)
        return msa_emb, pair_emb

    def forward(self, tf: torch.Tensor, ri: torch.Tensor, msa: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """tf [N_res, tf_dim], ri [N_res], msa [N_clust, N_res, msa_dim] ->
        (msa_emb [N_clust, N_res, C_m], pair_emb [N_res, N_res, C_z])."""
        F_.check_cuda(tf, ri, msa)
        if _needs_grad(self, tf, msa):
            return self._train(tf, ri, msa)
        if tf.dim() != 2 or msa.dim() != 3 or ri.dim() != 1:
            raise RuntimeError("InputEmbedder: expected tf [r, tf_dim], ri [r], msa [s, r, msa_dim] without batch "
                               "dimensions, got %s / %s / %s" % (tuple(tf.shape), tuple(ri.shape), tuple(msa.shape)))
        dt, dev = self.linear_relpos.weight.dtype, tf.device
        if self.c_z not in (64, 128, 256):
            raise RuntimeError("InputEmbedder: unsupported pair width %d" % self.c_z)
        ktf, kmsa, wi, bi, wj, bj, wm, bm, table, brel = self._pk(dt, dev)
        r, s = tf.shape[0], msa.shape[0]
        tfp = _pad_cols(tf.to(dt), ktf).contiguous()
        row = F_.linear(tfp, wi, bi, self.c_z)
        col = F_.linear(tfp, wj, bj, self.c_z)
        pair_emb = torch.empty(r, r, self.c_z, dtype=dt, device=dev)
        _lib.pair_embed(pair_emb, None, None, None, table, brel, row, col, mode=_lib.FFK_EMBED_RELPOS,
                        pos=ri.to(torch.float32).contiguous(), r=r, C=self.c_z, nb=self.no_bins)
        x = torch.cat([msa.to(dt), tf.to(dt).unsqueeze(0).expand(s, -1, -1)], -1)
        x = _pad_cols(x, kmsa).reshape(s * r, kmsa).contiguous()
        msa_emb = F_.linear(x, wm, bm, self.c_m).view(s, r, self.c_m)
        return msa_emb, pair_emb


class RecyclingEmbedder(nn.Module, _PackMixin):
    """Embeds the output of an iteration of the model for recycling: Algorithm 32."""

    def __init__(self, c_m: int, c_z: int, min_bin: float, max_bin: float, no_bins: int, inf: float = 1e8, **kwargs):
        super(RecyclingEmbedder, self).__init__()
        self.c_m = c_m
        self.c_z = c_z
        self.min_bin = min_bin
        self.max_bin = max_bin
        self.no_bins = no_bins
        self.inf = inf
        self.linear = Linear(self.no_bins, self.c_z)
        self.layer_norm_m = LayerNorm(self.c_m)
        self.layer_norm_z = LayerNorm(self.c_z)

    def _train(self, m, z, x):
        """embedders.py:207-232, operator by operator (open bin intervals on the squared distances, in fp32; the
        coordinates receive no gradient: the one-hot is piecewise constant)."""
        x = x.detach().to(torch.float32)
        sq = torch.linspace(self.min_bin, self.max_bin, self.no_bins, dtype=torch.float32, device=x.device) ** 2
        upper = torch.cat([sq[1:], sq.new_tensor([self.inf])], dim=-1)
        d = torch.sum((x[..., None, :] - x[..., None, :, :]) ** 2, dim=-1, keepdim=True)
        d = ((d > sq) * (d < upper)).to(z.dtype)
        return self.layer_norm_m(m), self.linear(d) + self.layer_norm_z(z)

    def forward(self, m: torch.Tensor, z: torch.Tensor, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """m [N_res, C_m] (first MSA row), z [N_res, N_res, C_z], x [N_res, 3] predicted C_beta coordinates ->
        (m_update, z_update).  As in the reference, z is overwritten when a chunk size is set
        (ops.py:1137-1143) and left untouched otherwise."""
        F_.check_cuda(m, z, x)
        if _needs_grad(self, m, z, x):
            return self._train(m, z, x)
        if z.dim() != 3 or z.shape[0] != z.shape[1] or x.shape != (z.shape[0], 3):
            raise RuntimeError("RecyclingEmbedder: expected z [r, r, c_z] and x [r, 3], got %s / %s"
                               % (tuple(z.shape), tuple(x.shape)))
        dt, dev = z.dtype, z.device
        if self.c_z not in (64, 128, 256):
            raise RuntimeError("RecyclingEmbedder: unsupported pair width %d" % self.c_z)
        table, bias, gam, bet, edges = self._packed(
            ("re", dt, dev), [self.linear.weight, self.linear.bias, self.layer_norm_z.weight, self.layer_norm_z.bias],
            lambda: (self.linear.weight.detach().t().to(dt).contiguous(), self.linear.bias.detach().to(dt).contiguous(),
                     self.layer_norm_z.weight.detach().to(dt).contiguous(),
                     self.layer_norm_z.bias.detach().to(dt).contiguous(),
                     torch.linspace(self.min_bin, self.max_bin, self.no_bins, dtype=torch.float32, device=dev) ** 2))
        m_update = self.layer_norm_m(m)
        zc = z if z.is_contiguous() else z.contiguous()
        out = zc if (_ops.CHUNK_SIZE is not None and zc is z) else torch.empty_like(zc)
        _lib.pair_embed(out, zc, gam, bet, table, bias, None, None, mode=_lib.FFK_EMBED_DISTOGRAM,
                        pos=x.to(torch.float32).contiguous(), edges=edges, inf=float(self.inf), r=z.shape[0],
                        C=self.c_z, nb=self.no_bins, ln_eps=self.layer_norm_z.eps)
        return m_update, out


class TemplateAngleEmbedder(nn.Module):
    """Embeds the "template_angle_feat" feature: Algorithm 2, line 7 (fastnn/embedders.py:257-297)."""

    def __init__(self, c_in: int, c_out: int, **kwargs):
        super(TemplateAngleEmbedder, self).__init__()
        self.c_out = c_out
        self.c_in = c_in
        self.linear_1 = Linear(self.c_in, self.c_out, initializer="relu")
        self.relu = nn.ReLU()
        self.linear_2 = Linear(self.c_out, self.c_out, initializer="relu")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x [*, N_templ, N_res, c_in] -> [*, N_templ, N_res, c_out]; the relu runs in the first launch's epilogue."""
        return self.linear_2(self.linear_1(x, act=_lib.FFK_ACT_RELU))


class TemplatePairEmbedder(nn.Module):
    """Embeds "template_pair_feat" features: Algorithm 2, line 9 (fastnn/embedders.py:300-341)."""

    def __init__(self, c_in: int, c_out: int, **kwargs):
        super(TemplatePairEmbedder, self).__init__()
        self.c_in = c_in
        self.c_out = c_out
        self.linear = Linear(self.c_in, self.c_out, initializer="relu")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.linear(x)


class ExtraMSAEmbedder(nn.Module):
    """Embeds unclustered MSA sequences: Algorithm 2, line 15 (fastnn/embedders.py:344-372)."""

    def __init__(self, c_in: int, c_out: int, **kwargs):
        super(ExtraMSAEmbedder, self).__init__()
        self.c_in = c_in
        self.c_out = c_out
        self.linear = Linear(self.c_in, self.c_out)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x [*, N_extra_seq, N_res, c_in] -> [*, N_extra_seq, N_res, c_out]."""
        return self.linear(x)
