"""Plain-PyTorch fp32 CPU restatement of the reference Evoformer (oracle).

TEST INFRASTRUCTURE ONLY - never imported by the product package.

Every class restates one module of the reference's ``fastfold.model.nn``
package and keeps its attribute / parameter names (the "nn layout"), so that a
state dict or a weight-injection routine written for the reference applies to
these modules unchanged.  Nothing here is chunked, checkpointed or scripted:
it is the mathematics of the eval-mode forward pass only (dropout = identity).

Pinning (what each part is checked against, see tests/test_oracle.py):
  * Attention, LayerNorm, Linear, softmax      library routines / float64 brute force
  * tri-mul / OPM contractions                 einsum forms + triple-loop brute force
  * composition of a block (Evoformer,
    extra-MSA, template pair stack)            golden vectors written by importing the
                                               reference's fastfold.model.nn in the
                                               build container (tests/golden/)
  * global attention                           float64 loops over the published formula
  * template point-wise attention              golden vectors from the reference's module and
                                               float64 loops over positions / heads / templates
  * input / recycling embedders                float64 loops (a Linear on a one-hot vector is a
                                               column pick); no golden vectors: the reference's
                                               nn/embedders.py needs dm-tree, absent here
  * identity at default init, permutation
    equivariance, masked-key invariance        mathematical invariants
"""
import math
from typing import List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F


# --------------------------------------------------------------------------
# primitives  (reference: fastfold/model/nn/primitives.py:102-237,291-419)
# --------------------------------------------------------------------------
def _trunc_normal_(w: torch.Tensor, scale: float) -> None:
    # fan-in variance scaling with a [-2,2] sigma truncated normal
    # (reference: primitives.py:45-61; 0.8796... = std of that truncation)
    fan_in = w.shape[1]
    std = math.sqrt(scale / max(1, fan_in)) / 0.87962566103423978
    nn.init.trunc_normal_(w, mean=0.0, std=std, a=-2.0 * std, b=2.0 * std)


class Linear(nn.Linear):
    """nn.Linear with the AlphaFold initialisers (primitives.py:102-167)."""

    def __init__(self, in_dim: int, out_dim: int, bias: bool = True, init: str = "default"):
        super().__init__(in_dim, out_dim, bias=bias)
        with torch.no_grad():
            if bias:
                self.bias.zero_()
            if init == "default":
                _trunc_normal_(self.weight, 1.0)
            elif init == "relu":
                _trunc_normal_(self.weight, 2.0)
            elif init == "glorot":
                nn.init.xavier_uniform_(self.weight, gain=1.0)
            elif init == "gating":
                self.weight.zero_()
                if bias:
                    self.bias.fill_(1.0)
            elif init == "normal":
                nn.init.kaiming_normal_(self.weight, nonlinearity="linear")
            elif init == "final":
                self.weight.zero_()
            else:
                raise ValueError("Invalid init string.")


class LayerNorm(nn.Module):
    """LayerNorm over the last dim, biased variance, eps 1e-5 (primitives.py:170-190)."""

    def __init__(self, c_in: int, eps: float = 1e-5):
        super().__init__()
        self.c_in = (c_in,)
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(c_in))
        self.bias = nn.Parameter(torch.zeros(c_in))

    def forward(self, x):
        return F.layer_norm(x, self.c_in, self.weight, self.bias, self.eps)


class Attention(nn.Module):
    """Gated multi-head attention with additive biases (primitives.py:291-419,205-237).

    q = W_q x / sqrt(c_hidden), k = W_k x, v = W_v x, heads are the slow index of the
    feature axis (feature = h * c_hidden + j); a = softmax(q k^T + sum(biases));
    o = (a v) * sigmoid(W_g x + b_g); out = W_o o + b_o.
    """

    def __init__(self, c_q: int, c_k: int, c_v: int, c_hidden: int, no_heads: int, gating: bool = True):
        super().__init__()
        self.c_q, self.c_k, self.c_v = c_q, c_k, c_v
        self.c_hidden, self.no_heads, self.gating = c_hidden, no_heads, gating
        hc = c_hidden * no_heads
        self.linear_q = Linear(c_q, hc, bias=False, init="glorot")
        self.linear_k = Linear(c_k, hc, bias=False, init="glorot")
        self.linear_v = Linear(c_v, hc, bias=False, init="glorot")
        self.linear_o = Linear(hc, c_q, init="final")
        self.linear_g = Linear(c_q, hc, init="gating") if gating else None

    def forward(self, q_x: torch.Tensor, kv_x: torch.Tensor,
                biases: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
        H, D = self.no_heads, self.c_hidden
        q = self.linear_q(q_x).view(q_x.shape[:-1] + (H, D)) / math.sqrt(D)
        k = self.linear_k(kv_x).view(kv_x.shape[:-1] + (H, D))
        v = self.linear_v(kv_x).view(kv_x.shape[:-1] + (H, D))
        # [*, H, Q, K]
        a = torch.einsum("...qhd,...khd->...hqk", q, k)
        for b in (biases or []):
            a = a + b
        a = torch.softmax(a, dim=-1)
        o = torch.einsum("...hqk,...khd->...qhd", a, v)
        if self.linear_g is not None:
            g = torch.sigmoid(self.linear_g(q_x)).view(q_x.shape[:-1] + (H, D))
            o = o * g
        return self.linear_o(o.reshape(o.shape[:-2] + (H * D,)))


# --------------------------------------------------------------------------
# MSA side  (reference: fastfold/model/nn/msa.py:36-223,255-319)
# --------------------------------------------------------------------------
class MSAAttention(nn.Module):
    """LayerNorm + gated MHA over the residue axis of every sequence, with the key
    mask as an additive -inf*(1-mask) bias and, optionally, a pair bias
    permute(W_z LN(z)) shared by all sequences (msa.py:98-137,208-221)."""

    def __init__(self, c_in, c_hidden, no_heads, pair_bias=False, c_z=None, inf=1e9):
        super().__init__()
        self.c_in, self.c_hidden, self.no_heads = c_in, c_hidden, no_heads
        self.pair_bias, self.c_z, self.inf = pair_bias, c_z, inf
        self.layer_norm_m = LayerNorm(c_in)
        self.layer_norm_z = LayerNorm(c_z) if pair_bias else None
        self.linear_z = Linear(c_z, no_heads, bias=False, init="normal") if pair_bias else None
        self.mha = Attention(c_in, c_in, c_in, c_hidden, no_heads)

    def forward(self, m, z=None, mask=None, chunk_size=None):
        m = self.layer_norm_m(m)
        if mask is None:
            mask = m.new_ones(m.shape[:-1])
        biases = [(self.inf * (mask - 1))[..., :, None, None, :]]
        if self.pair_bias and z is not None:
            b = self.linear_z(self.layer_norm_z(z))           # [*, r, r, H]
            biases.append(b.permute(*range(b.dim() - 3), -1, -3, -2).unsqueeze(-4))
        return self.mha(m, m, biases)


class MSARowAttentionWithPairBias(MSAAttention):
    def __init__(self, c_m, c_z, c_hidden, no_heads, inf=1e9):
        super().__init__(c_m, c_hidden, no_heads, pair_bias=True, c_z=c_z, inf=inf)


class MSAColumnAttention(nn.Module):
    """MSAAttention (no pair bias) applied along the sequence axis (msa.py:291-319)."""

    def __init__(self, c_m, c_hidden, no_heads, inf=1e9):
        super().__init__()
        self.c_m, self.c_hidden, self.no_heads, self.inf = c_m, c_hidden, no_heads, inf
        self._msa_att = MSAAttention(c_m, c_hidden, no_heads, pair_bias=False, inf=inf)

    def forward(self, m, mask=None, chunk_size=None):
        m = m.transpose(-2, -3)
        if mask is not None:
            mask = mask.transpose(-1, -2)
        return self._msa_att(m, mask=mask).transpose(-2, -3)


class MSATransition(nn.Module):
    """W_2 relu(W_1 LN(m)) * mask (evoformer.py:43-118)."""

    def __init__(self, c_m, n):
        super().__init__()
        self.c_m, self.n = c_m, n
        self.layer_norm = LayerNorm(c_m)
        self.linear_1 = Linear(c_m, n * c_m, init="relu")
        self.linear_2 = Linear(n * c_m, c_m, init="final")

    def forward(self, m, mask=None, chunk_size=None):
        if mask is None:
            mask = m.new_ones(m.shape[:-1])
        x = self.layer_norm(m)
        return self.linear_2(F.relu(self.linear_1(x))) * mask.unsqueeze(-1)


# --------------------------------------------------------------------------
# outer product mean  (reference: fastfold/model/nn/outer_product_mean.py:26-129)
# --------------------------------------------------------------------------
class OuterProductMean(nn.Module):
    def __init__(self, c_m, c_z, c_hidden, eps=1e-3):
        super().__init__()
        self.c_m, self.c_z, self.c_hidden, self.eps = c_m, c_z, c_hidden, eps
        self.layer_norm = nn.LayerNorm(c_m)
        self.linear_1 = Linear(c_m, c_hidden)
        self.linear_2 = Linear(c_m, c_hidden)
        self.linear_out = Linear(c_hidden ** 2, c_z, init="final")

    def forward(self, m, mask=None, chunk_size=None):
        if mask is None:
            mask = m.new_ones(m.shape[:-1])
        x = self.layer_norm(m)
        mk = mask.unsqueeze(-1)
        a = self.linear_1(x) * mk                              # [*, s, r, c]
        b = self.linear_2(x) * mk
        outer = torch.einsum("...sic,...sje->...ijce", a, b)   # [*, r, r, c, c]
        outer = self.linear_out(outer.reshape(outer.shape[:-2] + (-1,)))
        norm = torch.einsum("...sic,...sjc->...ijc", mk, mk)   # [*, r, r, 1]
        return outer / (self.eps + norm)                       # bias is divided too (:127)


# --------------------------------------------------------------------------
# triangle multiplicative update
# (reference: fastfold/model/nn/triangular_multiplicative_update.py:36-152, un-fused branch)
# --------------------------------------------------------------------------
class TriangleMultiplicativeUpdate(nn.Module):
    def __init__(self, c_z, c_hidden, _outgoing=True):
        super().__init__()
        self.c_z, self.c_hidden, self._outgoing = c_z, c_hidden, _outgoing
        self.linear_a_p = Linear(c_z, c_hidden)
        self.linear_a_g = Linear(c_z, c_hidden, init="gating")
        self.linear_b_p = Linear(c_z, c_hidden)
        self.linear_b_g = Linear(c_z, c_hidden, init="gating")
        self.linear_g = Linear(c_z, c_z, init="gating")
        self.linear_z = Linear(c_hidden, c_z, init="final")
        self.layer_norm_in = LayerNorm(c_z)
        self.layer_norm_out = LayerNorm(c_hidden)

    def forward(self, z, mask=None):
        if mask is None:
            mask = z.new_ones(z.shape[:-1])
        mk = mask.unsqueeze(-1)
        x = self.layer_norm_in(z)
        a = self.linear_a_p(x) * torch.sigmoid(self.linear_a_g(x)) * mk
        b = self.linear_b_p(x) * torch.sigmoid(self.linear_b_g(x)) * mk
        if self._outgoing:
            p = torch.einsum("...ikc,...jkc->...ijc", a, b)    # :116-125
        else:
            p = torch.einsum("...kic,...kjc->...ijc", a, b)    # :141-150
        p = self.linear_z(self.layer_norm_out(p))
        return p * torch.sigmoid(self.linear_g(x))


class TriangleMultiplicationOutgoing(TriangleMultiplicativeUpdate):
    def __init__(self, c_z, c_hidden):
        super().__init__(c_z, c_hidden, _outgoing=True)


class TriangleMultiplicationIncoming(TriangleMultiplicativeUpdate):
    def __init__(self, c_z, c_hidden):
        super().__init__(c_z, c_hidden, _outgoing=False)


# --------------------------------------------------------------------------
# triangle attention  (reference: fastfold/model/nn/triangular_attention.py:31-139)
# --------------------------------------------------------------------------
class TriangleAttention(nn.Module):
    def __init__(self, c_in, c_hidden, no_heads, starting, inf=1e9):
        super().__init__()
        self.c_in, self.c_hidden, self.no_heads = c_in, c_hidden, no_heads
        self.starting, self.inf = starting, inf
        self.layer_norm = LayerNorm(c_in)
        self.linear = Linear(c_in, no_heads, bias=False, init="normal")
        self.mha = Attention(c_in, c_in, c_in, c_hidden, no_heads)

    def forward(self, x, mask=None, chunk_size=None):
        if mask is None:
            mask = x.new_ones(x.shape[:-1])
        if not self.starting:
            x = x.transpose(-2, -3)
            mask = mask.transpose(-1, -2)
        x = self.layer_norm(x)
        mask_bias = (self.inf * (mask - 1))[..., :, None, None, :]
        tb = self.linear(x)                                    # [*, I, J, H]
        tb = tb.permute(*range(tb.dim() - 3), -1, -3, -2).unsqueeze(-4)
        x = self.mha(x, x, [mask_bias, tb])
        if not self.starting:
            x = x.transpose(-2, -3)
        return x


class TriangleAttentionStartingNode(TriangleAttention):
    def __init__(self, c_in, c_hidden, no_heads, inf=1e9):
        super().__init__(c_in, c_hidden, no_heads, starting=True, inf=inf)


class TriangleAttentionEndingNode(TriangleAttention):
    def __init__(self, c_in, c_hidden, no_heads, inf=1e9):
        super().__init__(c_in, c_hidden, no_heads, starting=False, inf=inf)


class PairTransition(nn.Module):
    """W_2 relu(W_1 LN(z)) * mask (pair_transition.py:24-99)."""

    def __init__(self, c_z, n):
        super().__init__()
        self.c_z, self.n = c_z, n
        self.layer_norm = LayerNorm(c_z)
        self.linear_1 = Linear(c_z, n * c_z, init="relu")
        self.linear_2 = Linear(n * c_z, c_z, init="final")

    def forward(self, z, mask=None, chunk_size=None):
        if mask is None:
            mask = z.new_ones(z.shape[:-1])
        x = self.layer_norm(z)
        return self.linear_2(F.relu(self.linear_1(x))) * mask.unsqueeze(-1)


# --------------------------------------------------------------------------
# block and stack  (reference: fastfold/model/nn/evoformer.py:121-290,394-535)
# --------------------------------------------------------------------------
class EvoformerBlockCore(nn.Module):
    def __init__(self, c_m, c_z, c_hidden_opm, c_hidden_mul, c_hidden_pair_att,
                 no_heads_msa, no_heads_pair, transition_n, pair_dropout, inf, eps,
                 is_multimer=False):
        super().__init__()
        self.is_multimer = is_multimer
        self.msa_transition = MSATransition(c_m, transition_n)
        self.outer_product_mean = OuterProductMean(c_m, c_z, c_hidden_opm)
        self.tri_mul_out = TriangleMultiplicationOutgoing(c_z, c_hidden_mul)
        self.tri_mul_in = TriangleMultiplicationIncoming(c_z, c_hidden_mul)
        self.tri_att_start = TriangleAttentionStartingNode(c_z, c_hidden_pair_att, no_heads_pair, inf=inf)
        self.tri_att_end = TriangleAttentionEndingNode(c_z, c_hidden_pair_att, no_heads_pair, inf=inf)
        self.pair_transition = PairTransition(c_z, transition_n)

    def forward(self, m, z, msa_mask, pair_mask, chunk_size=None, _mask_trans=True):
        # order and residual placement: evoformer.py:193-212 (OPM reads the updated m)
        m = m + self.msa_transition(m, mask=msa_mask if _mask_trans else None)
        z = z + self.outer_product_mean(m, mask=msa_mask)
        z = z + self.tri_mul_out(z, mask=pair_mask)
        z = z + self.tri_mul_in(z, mask=pair_mask)
        z = z + self.tri_att_start(z, mask=pair_mask)
        z = z + self.tri_att_end(z, mask=pair_mask)
        z = z + self.pair_transition(z, mask=pair_mask if _mask_trans else None)
        return m, z


class EvoformerBlock(nn.Module):
    def __init__(self, c_m, c_z, c_hidden_msa_att, c_hidden_opm, c_hidden_mul,
                 c_hidden_pair_att, no_heads_msa, no_heads_pair, transition_n,
                 msa_dropout, pair_dropout, inf, eps, is_multimer=False):
        super().__init__()
        self.msa_att_row = MSARowAttentionWithPairBias(c_m, c_z, c_hidden_msa_att, no_heads_msa, inf=inf)
        self.msa_att_col = MSAColumnAttention(c_m, c_hidden_msa_att, no_heads_msa, inf=inf)
        self.core = EvoformerBlockCore(c_m, c_z, c_hidden_opm, c_hidden_mul, c_hidden_pair_att,
                                       no_heads_msa, no_heads_pair, transition_n, pair_dropout,
                                       inf, eps)
        self.is_multimer = is_multimer

    def forward(self, m, z, msa_mask, pair_mask, chunk_size=None, _mask_trans=True):
        # evoformer.py:277-288
        m = m + self.msa_att_row(m, z=z, mask=msa_mask)
        m = m + self.msa_att_col(m, mask=msa_mask)
        return self.core(m, z, msa_mask=msa_mask, pair_mask=pair_mask, _mask_trans=_mask_trans)


class EvoformerStack(nn.Module):
    """no_blocks blocks, then s = Linear(c_m -> c_s)(m[0]) (evoformer.py:394-535)."""

    def __init__(self, c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128,
                 c_hidden_pair_att=32, c_s=384, no_heads_msa=8, no_heads_pair=4, no_blocks=48,
                 transition_n=4, msa_dropout=0.15, pair_dropout=0.25, blocks_per_ckpt=1,
                 inf=1e9, eps=1e-8, clear_cache_between_blocks=False, is_multimer=False, **kwargs):
        super().__init__()
        self.blocks_per_ckpt = blocks_per_ckpt
        self.clear_cache_between_blocks = clear_cache_between_blocks
        self.blocks = nn.ModuleList([
            EvoformerBlock(c_m, c_z, c_hidden_msa_att, c_hidden_opm, c_hidden_mul, c_hidden_pair_att,
                           no_heads_msa, no_heads_pair, transition_n, msa_dropout, pair_dropout,
                           inf, eps, is_multimer)
            for _ in range(no_blocks)])
        self.linear = Linear(c_m, c_s)

    def forward(self, m, z, msa_mask, pair_mask, chunk_size=None, _mask_trans=True
                ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        for b in self.blocks:
            m, z = b(m, z, msa_mask=msa_mask, pair_mask=pair_mask, _mask_trans=_mask_trans)
        s = self.linear(m[..., 0, :, :])
        return m, z, s


# --------------------------------------------------------------------------
# extra-MSA stack  (reference: fastfold/model/nn/primitives.py:422-504,
# fastfold/model/nn/msa.py:322-392, fastfold/model/nn/evoformer.py:293-389,538-633)
# --------------------------------------------------------------------------
class GlobalAttention(nn.Module):
    """One query per column (the masked mean over the sequences), one key / value head shared
    by all query heads (primitives.py:452-504):
      q = W_q (sum_s mask x / (sum_s mask + eps)) / sqrt(c), k = W_k x, v = W_v x  (c wide),
      a[h, s] = softmax_s(q[h] . k[s] + inf * (mask[s] - 1)), o[h] = sum_s a[h, s] v[s],
      out[s] = W_o (sigmoid(W_g x[s] + b_g) * o) + b_o."""

    def __init__(self, c_in, c_hidden, no_heads, inf, eps):
        super().__init__()
        self.c_in, self.c_hidden, self.no_heads, self.inf, self.eps = c_in, c_hidden, no_heads, inf, eps
        self.linear_q = Linear(c_in, c_hidden * no_heads, bias=False, init="glorot")
        self.linear_k = Linear(c_in, c_hidden, bias=False, init="glorot")
        self.linear_v = Linear(c_in, c_hidden, bias=False, init="glorot")
        self.linear_g = Linear(c_in, c_hidden * no_heads, init="gating")
        self.linear_o = Linear(c_hidden * no_heads, c_in, init="final")

    def forward(self, m, mask):
        H, D = self.no_heads, self.c_hidden
        q = (m * mask.unsqueeze(-1)).sum(-2) / (mask.sum(-1)[..., None] + self.eps)     # [*, r, c_in]
        q = (self.linear_q(q) * D ** -0.5).view(q.shape[:-1] + (H, D))                  # [*, r, H, D]
        k, v = self.linear_k(m), self.linear_v(m)                                        # [*, r, s, D]
        a = torch.einsum("...hd,...sd->...hs", q, k) + (self.inf * (mask - 1))[..., :, None, :]
        a = torch.softmax(a, dim=-1)
        o = torch.einsum("...hs,...sd->...hd", a, v)                                     # [*, r, H, D]
        g = torch.sigmoid(self.linear_g(m)).view(m.shape[:-1] + (H, D))                  # [*, r, s, H, D]
        o = o.unsqueeze(-3) * g
        return self.linear_o(o.reshape(o.shape[:-2] + (H * D,)))


class MSAColumnGlobalAttention(nn.Module):
    """LayerNorm + GlobalAttention along the sequence axis of every residue column (msa.py:361-392)."""

    def __init__(self, c_in, c_hidden, no_heads, inf=1e9, eps=1e-10):
        super().__init__()
        self.layer_norm_m = nn.LayerNorm(c_in)
        self.global_attention = GlobalAttention(c_in, c_hidden, no_heads, inf, eps)

    def forward(self, m, mask=None, chunk_size=None):
        if mask is None:
            mask = m.new_ones(m.shape[:-1])
        m = self.layer_norm_m(m.transpose(-2, -3))
        return self.global_attention(m, mask.transpose(-1, -2)).transpose(-2, -3)


class ExtraMSABlock(nn.Module):
    """Evoformer block whose column attention is the global one (evoformer.py:354-389).  The
    reference calls the core without ``_mask_trans``, i.e. with masked transitions; the argument
    is exposed here so that a caller can also get the un-masked variant."""

    def __init__(self, c_m, c_z, c_hidden_msa_att, c_hidden_opm, c_hidden_mul, c_hidden_pair_att,
                 no_heads_msa, no_heads_pair, transition_n, msa_dropout, pair_dropout, inf, eps,
                 ckpt=False, is_multimer=False):
        super().__init__()
        self.ckpt = ckpt
        self.msa_att_row = MSARowAttentionWithPairBias(c_m, c_z, c_hidden_msa_att, no_heads_msa, inf=inf)
        self.msa_att_col = MSAColumnGlobalAttention(c_m, c_hidden_msa_att, no_heads_msa, inf=inf, eps=eps)
        self.core = EvoformerBlockCore(c_m, c_z, c_hidden_opm, c_hidden_mul, c_hidden_pair_att,
                                       no_heads_msa, no_heads_pair, transition_n, pair_dropout, inf, eps)
        self.is_multimer = is_multimer

    def forward(self, m, z, msa_mask, pair_mask, chunk_size=None, _mask_trans=True):
        m = m + self.msa_att_row(m, z=z, mask=msa_mask)
        m = m + self.msa_att_col(m, mask=msa_mask)
        return self.core(m, z, msa_mask=msa_mask, pair_mask=pair_mask, _mask_trans=_mask_trans)


class ExtraMSAStack(nn.Module):
    """no_blocks extra-MSA blocks; only the pair representation is returned (evoformer.py:587-633)."""

    def __init__(self, c_m=64, c_z=128, c_hidden_msa_att=8, c_hidden_opm=32, c_hidden_mul=128,
                 c_hidden_pair_att=32, no_heads_msa=8, no_heads_pair=4, no_blocks=4, transition_n=4,
                 msa_dropout=0.15, pair_dropout=0.25, inf=1e9, eps=1e-10, ckpt=False,
                 clear_cache_between_blocks=False, is_multimer=False, **kwargs):
        super().__init__()
        self.clear_cache_between_blocks = clear_cache_between_blocks
        self.blocks = nn.ModuleList([
            ExtraMSABlock(c_m, c_z, c_hidden_msa_att, c_hidden_opm, c_hidden_mul, c_hidden_pair_att,
                          no_heads_msa, no_heads_pair, transition_n, msa_dropout, pair_dropout, inf, eps,
                          ckpt, is_multimer)
            for _ in range(no_blocks)])

    def forward(self, m, z, chunk_size=None, msa_mask=None, pair_mask=None, _mask_trans=True):
        for b in self.blocks:
            m, z = b(m, z, msa_mask, pair_mask, chunk_size=chunk_size, _mask_trans=_mask_trans)
        return z


# --------------------------------------------------------------------------
# template pair stack  (reference: fastfold/model/nn/template.py:139-363)
# --------------------------------------------------------------------------
class TemplatePairStackBlock(nn.Module):
    """Per template: tri-att start, tri-att end, tri-mul out, tri-mul in, pair transition, each added
    to its input (template.py:205-242; dropout is the identity in eval mode)."""

    def __init__(self, c_t, c_hidden_tri_att, c_hidden_tri_mul, no_heads, pair_transition_n, dropout_rate,
                 inf, is_multimer=False, **kwargs):
        super().__init__()
        self.tri_att_start = TriangleAttentionStartingNode(c_t, c_hidden_tri_att, no_heads, inf=inf)
        self.tri_att_end = TriangleAttentionEndingNode(c_t, c_hidden_tri_att, no_heads, inf=inf)
        self.tri_mul_out = TriangleMultiplicationOutgoing(c_t, c_hidden_tri_mul)
        self.tri_mul_in = TriangleMultiplicationIncoming(c_t, c_hidden_tri_mul)
        self.pair_transition = PairTransition(c_t, pair_transition_n)

    def forward(self, z, mask, chunk_size=None, _mask_trans=True):
        outs = []
        for single, single_mask in zip(torch.unbind(z, dim=-4), torch.unbind(mask, dim=-3)):
            single, single_mask = single.unsqueeze(-4), single_mask.unsqueeze(-3)
            single = single + self.tri_att_start(single, mask=single_mask)
            single = single + self.tri_att_end(single, mask=single_mask)
            single = single + self.tri_mul_out(single, mask=single_mask)
            single = single + self.tri_mul_in(single, mask=single_mask)
            single = single + self.pair_transition(single, mask=single_mask if _mask_trans else None)
            outs.append(single)
        return torch.cat(outs, dim=-4)


class TemplatePairStack(nn.Module):
    """no_blocks blocks, then a LayerNorm (template.py:326-363)."""

    def __init__(self, c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_blocks=2, no_heads=4,
                 pair_transition_n=2, dropout_rate=0.25, blocks_per_ckpt=None, inf=1e9, **kwargs):
        super().__init__()
        self.blocks_per_ckpt = blocks_per_ckpt
        self.blocks = nn.ModuleList([
            TemplatePairStackBlock(c_t, c_hidden_tri_att, c_hidden_tri_mul, no_heads, pair_transition_n,
                                   dropout_rate, inf) for _ in range(no_blocks)])
        self.layer_norm = LayerNorm(c_t)

    def forward(self, t, mask, chunk_size=None, _mask_trans=True):
        if mask.shape[-3] == 1:
            mask = mask.expand(*mask.shape[:-3], t.shape[-4], *mask.shape[-2:])
        for b in self.blocks:
            t = b(t, mask, _mask_trans=_mask_trans)
        return self.layer_norm(t)


class TemplatePointwiseAttention(nn.Module):
    """Algorithm 17 (nn/template.py:45-133): every pair position attends over the templates' embeddings at
    that position.  q = W_q z[i, j], keys / values from t[n, i, j], additive bias inf * (template_mask - 1)
    over the template axis, no gating.  The caller zeroes the update when no template is valid
    (nn/embedders.py:316); the fastnn module does that inside (fastnn/template.py:117-119)."""

    def __init__(self, c_t=64, c_z=128, c_hidden=16, no_heads=4, inf=1e5, **kwargs):
        super().__init__()
        self.c_t, self.c_z, self.c_hidden, self.no_heads, self.inf = c_t, c_z, c_hidden, no_heads, inf
        self.mha = Attention(c_z, c_t, c_t, c_hidden, no_heads, gating=False)

    def forward(self, t, z, template_mask=None, chunk_size=None):
        """t [N_templ, N_res, N_res, C_t], z [N_res, N_res, C_z], template_mask [N_templ] -> [N_res, N_res, C_z]."""
        if template_mask is None:
            template_mask = t.new_ones(t.shape[:-3])
        bias = self.inf * (template_mask[..., None, None, None, None, :] - 1)     # [1, 1, 1, 1, N_templ]
        q_x = z.unsqueeze(-2)                                                    # [r, r, 1, C_z]
        kv_x = t.permute(1, 2, 0, 3)                                             # [r, r, N_templ, C_t]
        return self.mha(q_x, kv_x, biases=[bias]).squeeze(-2)


# --------------------------------------------------------------------------
# input and recycling embedders  (reference: fastfold/model/nn/embedders.py:35-232,
# one_hot: fastfold/utils/tensor_utils.py:63-67)
# --------------------------------------------------------------------------
def one_hot_nearest(x, v_bins):
    """One-hot of the bin centre nearest to x (first one on a tie)."""
    diffs = x[..., None] - v_bins.view(((1,) * x.dim()) + (len(v_bins),))
    am = torch.argmin(torch.abs(diffs), dim=-1)
    return F.one_hot(am, num_classes=len(v_bins)).float()


class InputEmbedder(nn.Module):
    """Algorithms 3 and 4 (embedders.py:99-135): pair_emb[i, j] = W_i tf[i] + W_j tf[j] + W_rel
    onehot(clip(ri[i] - ri[j], +-k)), msa_emb[s, i] = W_msa msa[s, i] + W_tf tf[i] (biases included)."""

    def __init__(self, tf_dim, msa_dim, c_z, c_m, relpos_k, **kwargs):
        super().__init__()
        self.tf_dim, self.msa_dim, self.c_z, self.c_m = tf_dim, msa_dim, c_z, c_m
        self.linear_tf_z_i = Linear(tf_dim, c_z)
        self.linear_tf_z_j = Linear(tf_dim, c_z)
        self.linear_tf_m = Linear(tf_dim, c_m)
        self.linear_msa_m = Linear(msa_dim, c_m)
        self.relpos_k = relpos_k
        self.no_bins = 2 * relpos_k + 1
        self.linear_relpos = Linear(self.no_bins, c_z)

    def relpos(self, ri):
        d = ri[..., None] - ri[..., None, :]
        boundaries = torch.arange(start=-self.relpos_k, end=self.relpos_k + 1, device=d.device)
        return self.linear_relpos(one_hot_nearest(d, boundaries).type(ri.dtype))

    def forward(self, tf, ri, msa):
        tf_emb_i = self.linear_tf_z_i(tf)
        tf_emb_j = self.linear_tf_z_j(tf)
        pair_emb = tf_emb_i[..., None, :] + tf_emb_j[..., None, :, :]
        pair_emb = pair_emb + self.relpos(ri.type(pair_emb.dtype))
        tf_m = self.linear_tf_m(tf).unsqueeze(-3)
        msa_emb = self.linear_msa_m(msa) + tf_m
        return msa_emb, pair_emb


class RecyclingEmbedder(nn.Module):
    """Algorithm 32 (embedders.py:183-232): m_update = LN(m); z_update = LN(z) + W onehot(bin of
    |x_i - x_j|^2 among the squared bin edges, open intervals: a distance on an edge or below the first
    one falls in no bin) + b."""

    def __init__(self, c_m, c_z, min_bin, max_bin, no_bins, inf=1e8, **kwargs):
        super().__init__()
        self.c_m, self.c_z, self.min_bin, self.max_bin, self.no_bins, self.inf = c_m, c_z, min_bin, max_bin, no_bins, inf
        self.linear = Linear(no_bins, c_z)
        self.layer_norm_m = LayerNorm(c_m)
        self.layer_norm_z = LayerNorm(c_z)

    def forward(self, m, z, x):
        bins = torch.linspace(self.min_bin, self.max_bin, self.no_bins, dtype=x.dtype, device=x.device)
        m_update = self.layer_norm_m(m)
        squared_bins = bins ** 2
        upper = torch.cat([squared_bins[1:], squared_bins.new_tensor([self.inf])], dim=-1)
        d = torch.sum((x[..., None, :] - x[..., None, :, :]) ** 2, dim=-1, keepdims=True)
        d = ((d > squared_bins) * (d < upper)).type(x.dtype)
        return m_update, self.linear(d) + self.layer_norm_z(z)


class OracleModel(nn.Module):
    """Minimal stand-in for the whole-model object the injection routine receives:
    it only has the ``evoformer`` attribute (reference call site: hub/alphafold.py:92-95)."""

    def __init__(self, extra_msa_kwargs=None, **stack_kwargs):
        super().__init__()
        self.evoformer = EvoformerStack(**stack_kwargs)
        if extra_msa_kwargs is not None:
            self.extra_msa_stack = ExtraMSAStack(**extra_msa_kwargs)
