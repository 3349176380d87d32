"""Evoformer building blocks with the reference's class names, constructor signatures,
parameter names and call signatures (fastfold/model/fastnn/ops.py), each forward being a
short sequence of HIP kernel launches (see ``_fused.py``) instead of PyTorch ops.

Differences that do not change results: there is no distributed code (DAP size 1: the
reference's gather/scatter calls are identities) and chunking (``set_chunk_size``) lowers
the scratch-memory budget of the launches: attention logits and the fused transition / outer-product
intermediates are never materialised, and what is (attention operand tiles, the hidden activations and
outer products of the unfused paths) is produced a bounded slab of rows at a time.
"""
import math
import os

import torch
import torch.nn as nn

from fastfold_amd import _lib
from fastfold_amd.model.fastnn.kernel import LayerNorm
from . import _fused as F_
from .initializer import glorot_uniform_af
from .kernel import layouts

CHUNK_SIZE = None
DEBUG = False


def set_chunk_size(chunk_size):
    """Process-global chunk knob (reference: ops.py:31-37)."""
    global CHUNK_SIZE
    CHUNK_SIZE = chunk_size


def get_chunk_size():
    global CHUNK_SIZE
    return CHUNK_SIZE


def _budget():
    return F_._WS_BUDGET_DEFAULT if CHUNK_SIZE is None else F_._WS_BUDGET_CHUNKED


class _PackMixin:
    """Caches kernel-ready copies of the parameters, keyed by dtype/device and rebuilt when a source parameter is
    modified in place (its ``_version`` changes), replaced or moved, when the module is cast / moved (``_apply``) and
    when a state dict is loaded.  A write through ``param.data`` (``p.data.copy_(w)``) changes none of these: call
    ``invalidate_packed()`` on the module (or any parent, via ``module.apply``) after such a write."""

    def invalidate_packed(self):
        self.__dict__.pop("_pack_cache", None)

    def _apply(self, fn, *args, **kwargs):
        self.invalidate_packed()
        return super()._apply(fn, *args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        self.invalidate_packed()
        return super()._load_from_state_dict(*args, **kwargs)

    def _packed(self, key, params, build):
        cache = self.__dict__.setdefault("_pack_cache", {})
        ver = tuple((p.data_ptr(), p._version, p.dtype) for p in params)
        ent = cache.get(key)
        if ent is None or ent[0] != ver:
            with torch.no_grad():
                ent = (ver, build())
            cache[key] = ent
        return ent[1]


def _no_grad_guard(module, *tensors):
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise NotImplementedError(
            "%s: the HIP path implements the forward pass only; run it under torch.no_grad()"
            % type(module).__name__)


_WARNED_EVAL_GRAD = False


def _needs_grad(module, *tensors):
    """True when autograd has to see this call: gradients are enabled and an input or a parameter of ``module``
    requires one.  Such calls take the differentiable composition (``_train`` methods); everything else takes the
    fused forward-only launches.  A module in ``eval()`` mode whose parameters still require gradients, called
    outside ``torch.no_grad()`` with inputs that need none, is almost always an inference call that forgot the
    ``no_grad``: it is honoured (autograd semantics), but a warning is raised once, because the differentiable
    composition is several times slower and carries the plain bf16 residual stream."""
    global _WARNED_EVAL_GRAD
    if not torch.is_grad_enabled():
        return False
    if any(t is not None and t.requires_grad for t in tensors):
        return True
    if any(p.requires_grad for p in module.parameters()):
        if not module.training and not _WARNED_EVAL_GRAD:
            _WARNED_EVAL_GRAD = True
            import warnings
            warnings.warn("fastfold_amd: %s is in eval() mode but was called with gradients enabled and parameters that "
                          "require them: taking the differentiable (slower, plain-residual) path.  Wrap inference calls in "
                          "torch.no_grad() to run the fused kernels." % type(module).__name__, RuntimeWarning, stacklevel=3)
        return True
    return False


_WGRAD_SPLIT_ROWS = 4096


def _storage_span(t):
    """(first byte, one past the last byte) that a view addresses inside its storage."""
    if t.numel() == 0:
        return (0, 0)
    last = t.storage_offset() + sum((n - 1) * st for n, st in zip(t.shape, t.stride()))
    return (t.storage_offset() * t.element_size(), (last + 1) * t.element_size())


def _check_library_gemm_operands(a, b, who):
    """Host-side guard in front of every *library* batched GEMM of the differentiable path: each operand view must lie
    inside its allocation, and the two operands must not be views of one allocation (two GPU memory faults at
    128 x 1024^3, bf16, were reported from inside the library's batched NT GEMM when its operands were the two halves
    of one buffer; the callers' views were in bounds).  Raises instead of launching."""
    for t in (a, b):
        lo, hi = _storage_span(t)
        if hi > t.untyped_storage().nbytes():
            raise RuntimeError("%s: an operand view addresses %d bytes of a %d-byte allocation"
                               % (who, hi, t.untyped_storage().nbytes()))
    if a.numel() and b.numel() and a.untyped_storage().data_ptr() == b.untyped_storage().data_ptr():
        raise RuntimeError("%s: both operands of a library batched GEMM are views of one allocation" % who)


def _weight_grad(dy2, x2):
    """dy2^T . x2 for [M, N] and [M, K] activations with M in the hundreds of thousands: one GEMM whose whole
    parallelism is its N x K output (a few hundred tiles reducing over a million rows each) runs at a few per cent
    of the matrix pipe, so the rows are cut into slabs that a batched GEMM reduces side by side; the slab results
    are added in fp32."""
    M = dy2.shape[0]
    S = 1
    while M % (2 * S) == 0 and M // (2 * S) >= _WGRAD_SPLIT_ROWS:
        S *= 2
    if S == 1 or dy2.dtype == torch.float32:
        return dy2.t() @ x2
    a = dy2.reshape(S, M // S, -1).transpose(1, 2)
    b = x2.reshape(S, M // S, -1)
    if a.untyped_storage().data_ptr() == b.untyped_storage().data_ptr():
        b = b.clone()                      # e.g. dy2 and x2 sliced from one tensor: give the library two allocations
    _check_library_gemm_operands(a, b, "_weight_grad")
    part = torch.bmm(a, b)
    return part.sum(0, dtype=torch.float32).to(dy2.dtype)


def _padded_copy(x):
    """[c, m, k] view (any strides) -> a freshly allocated contiguous [c, m, kpad] tensor, the last axis zero-padded
    to the GEMM kernels' 16-byte K step."""
    kpad = F_.round_up(x.shape[-1], F_.vec_of(x.dtype))
    out = (torch.zeros if kpad != x.shape[-1] else torch.empty)(x.shape[0], x.shape[1], kpad, dtype=x.dtype,
                                                                 device=x.device)
    out[..., :x.shape[-1]].copy_(x)
    return out


def _chan_major(t, perm):
    """[1, a, b, c] -> [c, x, kpad] with (c, x, k) the last three axes in the order ``perm`` names
    (permute_final_dims indices), in an allocation of its own."""
    return _padded_copy(permute_final_dims(t, perm)[0])


def _cm_alloc(c, r, dtype, device):
    """[c, r, kpad] with the last axis padded to the GEMM kernels' 16-byte K step; zeroed where padding exists."""
    kpad = F_.round_up(r, F_.vec_of(dtype))
    return (torch.zeros if kpad != r else torch.empty)(c, r, kpad, dtype=dtype, device=device)


def _transpose_cm(x, r):
    """[c, r, kpad] channel-major -> [c, r, kpad] with the two row indices exchanged: out[c, k, j] = x[c, j, k]."""
    c, _, kpad = x.shape
    out = _cm_alloc(c, r, x.dtype, x.device)
    _lib.transpose_batched(out, x, B=c, X=r, Y=r, in_bs=x.stride(0), in_xs=x.stride(1), out_bs=r * kpad, out_ys=kpad)
    return out


class _ToChanMajorFn(torch.autograd.Function):
    """lr [1, r, r, 2c] (channels contiguous) -> (L, R), each [c, r, kpad] channel-major in an allocation of its own:
    L[ch, i, k] = lr[0, i, k, ch] (outgoing) or lr[0, k, i, ch] (incoming), R the same from channels c .. 2c - 1
    (the permute_final_dims of fastnn/ops.py:400-403, 529-532).  One transposition launch per operand, forward and
    backward; the backward pass writes both halves of the gradient of ``lr`` in place (no concatenation)."""

    @staticmethod
    def forward(ctx, lr, incoming):
        _, r, r2, c2 = lr.shape
        if r != r2 or lr.stride(3) != 1 or c2 % 2:
            raise RuntimeError("_ToChanMajorFn: expected [1, r, r, 2c] with contiguous channels, got %s strides %s"
                               % (tuple(lr.shape), lr.stride()))
        c = c2 // 2
        s_i, s_k = (lr.stride(2), lr.stride(1)) if incoming else (lr.stride(1), lr.stride(2))
        outs = []
        for side in range(2):
            out = _cm_alloc(c, r, lr.dtype, lr.device)
            _lib.transpose_batched(out, lr, B=r, X=r, Y=c, in_bs=s_i, in_xs=s_k, out_bs=out.stride(1),
                                   out_ys=out.stride(0), in_off=side * c)
            outs.append(out)
        ctx.incoming, ctx.r, ctx.c = incoming, r, c
        return outs[0], outs[1]

    @staticmethod
    def backward(ctx, dL, dR):
        r, c = ctx.r, ctx.c
        ref = dL if dL is not None else dR
        g = torch.empty(1, r, r, 2 * c, dtype=ref.dtype, device=ref.device)
        s_i, s_k = (g.stride(2), g.stride(1)) if ctx.incoming else (g.stride(1), g.stride(2))
        for side, d in enumerate((dL, dR)):
            if d is None:
                g[..., side * c:(side + 1) * c].zero_()
                continue
            d = d.contiguous()
            # g[0, i, k, side c + ch] = d[ch, i, k]: per i the [ch, k] matrix transposed
            _lib.transpose_batched(g, d, B=r, X=c, Y=r, in_bs=d.stride(1), in_xs=d.stride(0), out_bs=s_i, out_ys=s_k,
                                   out_off=side * c)
        return g, None


class _FromChanMajorFn(torch.autograd.Function):
    """p [c, r, npad] channel-major -> [1, r, r, c] contiguous (the permute_final_dims(p, (1, 2, 0)) of
    fastnn/ops.py:404, :533), one transposition launch each way."""

    @staticmethod
    def forward(ctx, p, r):
        c = p.shape[0]
        p = p.contiguous()
        out = torch.empty(1, r, r, c, dtype=p.dtype, device=p.device)
        _lib.transpose_batched(out, p, B=r, X=c, Y=r, in_bs=p.stride(1), in_xs=p.stride(0), out_bs=r * c, out_ys=c)
        ctx.r, ctx.c, ctx.npad = r, c, p.shape[2]
        return out

    @staticmethod
    def backward(ctx, g):
        r, c = ctx.r, ctx.c
        g = g.contiguous()
        dp = _cm_alloc(c, r, g.dtype, g.device)
        _lib.transpose_batched(dp, g, B=r, X=r, Y=c, in_bs=r * c, in_xs=c, out_bs=dp.stride(1), out_ys=dp.stride(0))
        return dp, None


def _bgemm_cm(a, b, n_valid):
    """out[c, i, j] = sum_k a[c, i, k] b[c, j, k] for j < n_valid (rows of b past n_valid are padding) through
    ``ffk_bgemm_nt`` (the library's own batched NT GEMM, the kernel the fused path's contraction runs on); the
    output's last axis is padded like the operands' and the padding zero."""
    c, M, K = a.shape
    N = b.shape[1]
    npad = F_.round_up(n_valid, F_.vec_of(a.dtype))
    out = (torch.zeros if npad != n_valid else torch.empty)(c, M, npad, dtype=a.dtype, device=a.device)
    _lib.bgemm_nt(a, b, out, M=M, N=n_valid, K=K, lda=K, ldb=K, batch=c, a_bs=M * K, b_bs=N * K, o_bs=M * npad,
                  s_i=npad)
    return out


class _TriContractFn(torch.autograd.Function):
    """p[c, i, j] = sum_k L[c, i, k] R[c, j, k], forward and both backward products on ``ffk_bgemm_nt``
    (reference: the permuted ``torch.matmul`` of fastnn/ops.py:400-403,529-532).  L, R: separately allocated
    [c, r, kpad] tensors (``_chan_major``); returns [c, r, kpad] with zero padding columns."""

    @staticmethod
    def forward(ctx, L, R, r):
        ctx.save_for_backward(L, R)
        ctx.r = r
        return _bgemm_cm(L, R, r)

    @staticmethod
    def backward(ctx, dp):
        L, R = ctx.saved_tensors
        r = ctx.r
        dp = dp.contiguous()
        dL = dR = None
        if ctx.needs_input_grad[0]:      # dL[c, i, k] = sum_j dp[c, i, j] R[c, j, k]: K runs over j
            dL = _bgemm_cm(dp, _transpose_cm(R, r), r)
        if ctx.needs_input_grad[1]:      # dR[c, j, k] = sum_i dp[c, i, j] L[c, i, k]: K runs over i
            dR = _bgemm_cm(_transpose_cm(dp, r), _transpose_cm(L, r), r)
        return dL, dR, None


class _LinearFn(torch.autograd.Function):
    """y = x W^T + b through the library GEMM, with the weight gradient computed by ``_weight_grad``."""

    @staticmethod
    def forward(ctx, x, w, b):
        ctx.save_for_backward(x, w)
        return torch.nn.functional.linear(x, w, b)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1])
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = (dy2 @ w).view(x.shape)
        if ctx.needs_input_grad[1]:
            dw = _weight_grad(dy2, x.reshape(-1, x.shape[-1]))
        if ctx.needs_input_grad[2]:
            db = dy2.sum(0)
        return dx, dw, db


def _check_tail(xtail, x):
    """The int8 tail of ``x`` as an extended residual stream (see include/ffk.h): same shape, bf16 stream only."""
    if xtail is None:
        return None
    if x.dtype != torch.bfloat16 or xtail.dtype != torch.int8 or xtail.shape != x.shape or not xtail.is_contiguous() \
            or xtail.device != x.device:
        raise RuntimeError("residual tail must be a contiguous int8 tensor of the bf16 stream's shape %s on its device"
                           % (tuple(x.shape),))
    return xtail


def _ln_pair(ln, dtype):
    return (ln.weight.detach().to(dtype).contiguous(), ln.bias.detach().to(dtype).contiguous())


def _mask_like(mask, x):
    if mask.dtype == x.dtype and mask.is_contiguous():
        return mask
    # a converted copy is itself derived from the mask only: one per stack, and a stable key for what follows
    return F_._mask_derived(mask, ("cast", x.dtype), lambda: mask.to(dtype=x.dtype).contiguous())


class _SharedAxisDropout(nn.Module):
    """Dropout whose keep / drop decision is drawn once per slice and shared along one axis of a
    [b, i, j, c] tensor (reference: ops.py:45-68): the decision tensor has extent 1 on ``_shared_axis``."""
    _shared_axis = 1

    def __init__(self, p):
        super().__init__()
        self.p = p
        self.dropout = nn.Dropout(p=p)

    def forward(self, x):
        keep = self.dropout(torch.ones_like(x.narrow(self._shared_axis, 0, 1)))
        return x * keep


class DropoutRowwise(_SharedAxisDropout):
    """One decision per (b, j, c), shared by all rows i."""
    _shared_axis = 1


class DropoutColumnwise(_SharedAxisDropout):
    """One decision per (b, i, c), shared by all columns j."""
    _shared_axis = 2


class Linear(nn.Linear, _PackMixin):
    """nn.Linear with the reference's initialisers (ops.py:229-256): 'linear' = Glorot gain 1,
    'relu' = gain 2, 'zeros' = zero weight; any other string (the reference's call sites pass
    'zero') keeps nn.Linear's default init.  The forward is an MFMA GEMM launch."""

    def __init__(self, feature_in: int, feature_out: int, initializer: str = 'linear', use_bias: bool = True,
                 bias_init: float = 0.):
        super(Linear, self).__init__(feature_in, feature_out, bias=use_bias)
        self.use_bias = use_bias
        if initializer == 'linear':
            glorot_uniform_af(self.weight, gain=1.0)
        elif initializer == 'relu':
            glorot_uniform_af(self.weight, gain=2.0)
        elif initializer == 'zeros':
            nn.init.zeros_(self.weight)
        if self.use_bias:
            with torch.no_grad():
                self.bias.fill_(bias_init)

    def _kpad(self):
        # ragged input widths (feature embedders: 22, 25, 49, 57, 88 ...) are zero-padded to the kernels' K step
        return self.in_features if self.in_features % 32 == 0 else F_.round_up(self.in_features, 32)

    def _pk(self, dtype, device):
        params = [self.weight] + ([self.bias] if self.use_bias else [])
        kp = self._kpad()
        return self._packed(("lin", dtype, device), params, lambda: (
            F_.pack_rows([torch.nn.functional.pad(self.weight.detach(), (0, kp - self.in_features))], dtype, device),
            F_.pack_vec([self.bias], dtype, device) if self.use_bias else None))

    def forward(self, input, act=_lib.FFK_ACT_NONE):
        F_.check_cuda(input)
        if _needs_grad(self, input):
            y = _LinearFn.apply(input, self.weight.to(input.dtype),
                                self.bias.to(input.dtype) if self.use_bias else None)
            if act == _lib.FFK_ACT_RELU:
                return torch.relu(y)
            return torch.sigmoid(y) if act == _lib.FFK_ACT_SIGMOID else y
        w, b = self._pk(input.dtype, input.device)
        x2 = input.reshape(-1, self.in_features)
        kp = self._kpad()
        if kp != self.in_features:
            x2 = torch.nn.functional.pad(x2, (0, kp - self.in_features))
        out = F_.linear(x2.contiguous(), w, b, self.out_features, act=act)
        return out.view(*input.shape[:-1], self.out_features)


class Transition(nn.Module, _PackMixin):
    """src + W2 relu(W1 LN(src) + b1) + b2 (ops.py:71-82); no mask, as in the reference."""

    def __init__(self, d, n=4):
        super(Transition, self).__init__()
        self.norm = LayerNorm(d)
        self.linear1 = Linear(d, n * d, initializer='relu')
        self.linear2 = Linear(n * d, d, initializer='zeros')

    def _run(self, src, out, xtail=None):
        F_.check_cuda(src)
        _no_grad_guard(self, src)
        dt, dev = src.dtype, src.device
        d = src.shape[-1]
        hidden = self.linear1.out_features
        if not F_.fits_fused(d, dt) or hidden % 128 != 0:
            raise RuntimeError("Transition: unsupported width %d" % d)
        w1, b1, w2, b2 = self._packed(("tr", dt, dev), [self.linear1.weight, self.linear1.bias,
                                                       self.linear2.weight, self.linear2.bias], lambda: (
            F_.pack_rows([self.linear1.weight], dt, dev), F_.pack_vec([self.linear1.bias], dt, dev),
            self.linear2.weight.detach().to(dt).contiguous(), self.linear2.bias.detach().to(dt).contiguous()))
        x = src.view(-1, d)
        F_.transition(x, out.view(-1, d), ln=_ln_pair(self.norm, dt), w1_pk=w1, b1_pk=b1, w2=w2, b2=b2,
                      hidden=hidden, budget=_budget(), xtail=_check_tail(xtail, src))
        return out

    def _train(self, src):
        """ops.py:79-82, operator by operator."""
        x = self.norm(src)
        return src + self.linear2(torch.relu(self.linear1(x)))

    def forward(self, src):
        if _needs_grad(self, src):
            return self._train(src)
        src = src.contiguous()
        return self._run(src, torch.empty_like(src))


class ChunkTransition(Transition):
    """Same computation (ops.py:85-123); rows are always streamed in bounded chunks."""

    def inplace(self, src):
        src[0] = src[0].contiguous()
        self._run(src[0], src[0])
        return src


class OutProductMean(nn.Module, _PackMixin):
    """Outer-product-mean update of the pair representation (ops.py:126-227)."""

    def __init__(self, n_feat=64, n_feat_out=128, n_feat_proj=32):
        super(OutProductMean, self).__init__()
        self.layernormM = LayerNorm(n_feat)
        self.linear_a = Linear(n_feat, n_feat_proj)
        self.linear_b = Linear(n_feat, n_feat_proj)
        self.o_linear = Linear(n_feat_proj * n_feat_proj, n_feat_out, initializer='zero', use_bias=True)
        self.n_feat_proj = n_feat_proj

    def _run(self, M, M_mask, Z_raw, out, xtail=None):
        F_.check_cuda(M, M_mask, Z_raw)
        _no_grad_guard(self, M, Z_raw)
        if self.n_feat_proj != 32:
            raise RuntimeError("OutProductMean: the kernel path needs n_feat_proj == 32")
        dt, dev = M.dtype, M.device
        if M.dim() == 4:
            if M.shape[0] != 1:
                raise RuntimeError("OutProductMean: leading batch dimension must be 1")
            M, M_mask = M[0], M_mask[0]
        s, r, C = M.shape
        Cz = Z_raw.shape[-1]
        if not F_.fits_fused(C, dt):
            raise RuntimeError("OutProductMean: unsupported MSA width %d" % C)
        wab, bab, wo, bo, wo_ed = self._packed(("opm", dt, dev), [self.linear_a.weight, self.linear_a.bias,
                                                          self.linear_b.weight, self.linear_b.bias,
                                                          self.o_linear.weight, self.o_linear.bias], lambda: (
            F_.pack_rows([self.linear_a.weight, self.linear_b.weight], dt, dev),
            F_.pack_vec([self.linear_a.bias, self.linear_b.bias], dt, dev),
            self.o_linear.weight.detach().to(dt).contiguous(), self.o_linear.bias.detach().to(dt).contiguous(),
            # the fused kernel contracts over (e, d) instead of (d, e)
            self.o_linear.weight.detach().to(dt).view(-1, 32, 32).transpose(1, 2).reshape(-1, 1024).contiguous()))
        F_.outer_product_mean(M.contiguous(), _mask_like(M_mask, M), Z_raw, out, s=s, r=r, C=C, Cz=Cz,
                              ln=_ln_pair(self.layernormM, dt), wab_pk=wab, bab_pk=bab, wo=wo, bo=bo, wo_ed=wo_ed,
                              budget=_budget(), xtail=_check_tail(xtail, Z_raw))
        return out

    def _train(self, M, M_mask, Z_raw):
        """ops.py:141-173 (the un-chunked branch); the normaliser is kept in fp32."""
        M = self.layernormM(M)
        mask = M_mask.unsqueeze(-1).to(M.dtype)
        left = mask * self.linear_a(M)
        right = mask * self.linear_b(M)
        norm = torch.einsum('bsid,bsjd->bijd', mask.float(), mask.float()) + 1e-3
        out = torch.einsum('bsid,bsje->bijde', left, right).flatten(-2)
        out = self.o_linear(out)
        return (out.float() / norm).to(Z_raw.dtype) + Z_raw

    def forward(self, M, M_mask, Z_raw):
        if _needs_grad(self, M, Z_raw):
            return self._train(M, M_mask, Z_raw)
        Z_raw = Z_raw.contiguous()
        return self._run(M, M_mask, Z_raw, torch.empty_like(Z_raw))

    def inplace(self, M, M_mask, Z_raw):
        Z_raw[0] = Z_raw[0].contiguous()
        self._run(M, M_mask, Z_raw[0], Z_raw[0])
        return Z_raw


def _pad_heads(w, n_head, c, dim):
    """Index h * c + d along ``dim`` -> h * 32 + d, new entries zero (a head narrower than the kernels'
    32 channels contributes nothing through its padding: zero q / k / v channels and zero o_linear columns)."""
    if c == 32:
        return w
    w = w.detach().unflatten(dim, (n_head, c))
    pad = [0, 0] * (w.dim() - dim - 2) + [0, 32 - c]
    return torch.nn.functional.pad(w, pad).flatten(dim, dim + 1)


class SelfAttention(nn.Module, _PackMixin):
    """Multi-head self attention over [batch_size1, batch_size2, len, dim] tensors with gating
    (ops.py:259-363).  Head dimension ``c`` at most 32 and ``n_head`` a multiple of 4."""

    def __init__(self, qkv_dim, c, n_head, out_dim, gating=True, last_bias_fuse=False):
        super(SelfAttention, self).__init__()
        self.qkv_dim = qkv_dim
        self.c = c
        self.n_head = n_head
        self.out_dim = out_dim
        self.gating = gating
        self.last_bias_fuse = last_bias_fuse
        self.scaling = self.c**(-0.5)
        self.to_qkv = Linear(qkv_dim, 3 * n_head * c, initializer='linear', use_bias=False)
        if gating:
            self.gating_bias = nn.parameter.Parameter(data=torch.ones((n_head * c,)))
            self.gating_linear = Linear(qkv_dim, n_head * c, initializer='zero', use_bias=False)
        self.o_linear = Linear(n_head * c, out_dim, initializer='zero', use_bias=(not last_bias_fuse))

    def _check(self, dtype):
        if self.c > 32 or self.n_head % 4 != 0 or not self.gating:
            raise RuntimeError("SelfAttention: the kernel path needs head dim <= 32, n_head % 4 == 0 and gating=True")
        if not F_.fits_fused(self.qkv_dim, dtype):
            raise RuntimeError("SelfAttention: unsupported input width %d" % self.qkv_dim)

    def packed(self, dtype, device, extra_rows=None, extra_params=()):
        """(w_pk [q;k;v;gate(;extra)], gating_bias_pk, wo_pk)."""
        key = ("att", dtype, device, extra_rows is not None)
        params = [self.to_qkv.weight, self.gating_linear.weight, self.gating_bias, self.o_linear.weight]
        params += list(extra_params)

        def build():
            H, c = self.n_head, self.c
            mats = [_pad_heads(self.to_qkv.weight.detach().unflatten(0, (3, H * c)), H, c, 1).flatten(0, 1),
                    _pad_heads(self.gating_linear.weight, H, c, 0)]
            w = F_.pack_rows(mats, dtype, device)
            if extra_rows is not None:
                hc = H * 32
                extra = F_.pack_rows([extra_rows()], dtype, device)
                w = torch.cat([w, extra], 0).contiguous()
                # the same without the gate block ([q; k; v; extra]): the projection launch of an attention whose gate
                # is computed in the output stage finds the extra (pair-bias) rows right behind v
                w.without_gate = torch.cat([w[:3 * hc], extra], 0).contiguous()
            return (w, F_.pack_vec([_pad_heads(self.gating_bias, H, c, 0)], dtype, device),
                    F_.pack_rows([_pad_heads(self.o_linear.weight, H, c, 1)], dtype, device))
        return self._packed(key, params, build)

    def _train(self, in_data, mask, nonbatched_bias=None):
        """ops.py:289-331 with the logits / softmax / weighted average of :310-322 inside the attention-core kernels
        (forward and backward recompute the logits tile by tile; they are never stored)."""
        from .kernel import bias_sigmod_ele, fused_attention_core
        bias = None
        if nonbatched_bias is not None:
            bias = nonbatched_bias[0]
            if not (isinstance(nonbatched_bias[-1], int) and nonbatched_bias[-1] == -1):
                bias = bias.permute(0, 3, 1, 2)                 # 'b q k h -> b h q k'
            bias = bias.contiguous()
        qkv = self.to_qkv(in_data).chunk(3, dim=-1)
        # [b1, b2, h, n, d] views of the projection's output: the operator re-tiles them as they lie
        q, k, v = (t.unflatten(-1, (self.n_head, self.c)).transpose(-2, -3) for t in qkv)
        if mask is not None:
            mask = mask.to(in_data.dtype).contiguous()
        weighted_avg = fused_attention_core(q, k, v, mask, bias)          # [b1, b2, n, h * d]
        if self.gating:
            weighted_avg = bias_sigmod_ele(self.gating_linear(in_data), self.gating_bias, weighted_avg)
        return self.o_linear(weighted_avg)

    def forward(self, in_data, mask, nonbatched_bias=None):
        """
        :param in_data: [batch_size1, batch_size2, len_qkv, qkv_dim]
        :param mask: None or [batch_size1, batch_size2, len_kv]
        :param nonbatched_bias: None, or (b [batch_size1, len_q, len_kv, n_head], work), or
                                (bias [batch_size1, n_head, len_q, len_kv], -1)
        """
        F_.check_cuda(in_data, mask)
        if _needs_grad(self, in_data, None if nonbatched_bias is None else nonbatched_bias[0]):
            return self._train(in_data, mask, nonbatched_bias)
        dt, dev = in_data.dtype, in_data.device
        self._check(dt)
        if in_data.dim() != 4 or in_data.shape[0] != 1:
            raise RuntimeError("SelfAttention: expected [1, B2, N, C] input, got %s" % (tuple(in_data.shape),))
        _, B2, N, C = in_data.shape
        x = in_data.contiguous()
        bias_t = None
        if nonbatched_bias is not None:
            b = nonbatched_bias[0]
            if not (isinstance(nonbatched_bias[-1], int) and nonbatched_bias[-1] == -1):
                b = b.permute(0, 3, 1, 2)                       # 'b q k h -> b h q k'
            bias_t = layouts.tile_bias(b[0].float() * _lib.LOG2E).to(dt)
        if mask is None:
            mk, sb, sn = None, 0, 1
        else:
            mk, sb, sn = _mask_like(mask, x)[0], N, 1
        w_pk, gb_pk, wo_pk = self.packed(dt, dev)
        ob = None
        if self.o_linear.use_bias:
            ob = self._packed(("ob", dt, dev), [self.o_linear.bias], lambda: F_.pack_vec([self.o_linear.bias], dt, dev))
        out = torch.empty(1, B2, N, self.out_dim, dtype=dt, device=dev)
        F_.attention(x, out, None, B2=B2, N=N, C=C, H=self.n_head, a_map=(B2 * N, 0, C), ln=None, w_pk=w_pk,
                     gate_bias_pk=gb_pk, wo_pk=wo_pk, out_bias_pk=ob, c_out=self.out_dim, mask=mk, mask_sb=sb,
                     mask_sn=sn, bias_t=bias_t, head_dim=self.c, budget=_budget(), o_map=(B2 * N, 0, self.out_dim))
        return out


class GlobalAttention(nn.Module, _PackMixin):
    """Global attention over [batch_size1, batch_size2, len, dim] tensors (ops.py:1148-1236): one query
    per (batch_size1, batch_size2) entry - the masked mean over ``len`` - and a single key / value head."""

    def __init__(self, qkv_dim, c, n_head, out_dim):
        super(GlobalAttention, self).__init__()
        self.qkv_dim = qkv_dim
        self.c = c
        self.n_head = n_head
        self.out_dim = out_dim
        self.scaling = self.c ** (-0.5)
        self.eps = 1e-10
        self.inf = 1e9
        self.to_q = Linear(qkv_dim, c * self.n_head, use_bias=False)
        self.to_kv = Linear(qkv_dim, 2 * c, initializer="linear", use_bias=False)
        self.gating_bias = nn.parameter.Parameter(data=torch.ones((n_head * c,)))
        self.gating_linear = Linear(qkv_dim, n_head * c, initializer="zero", use_bias=False)
        self.o_linear = Linear(n_head * c, out_dim, initializer="zero")

    def _pk(self, dt, dev):
        ps = [self.to_q.weight, self.to_kv.weight, self.gating_linear.weight, self.gating_bias,
              self.o_linear.weight, self.o_linear.bias]
        return self._packed(("ga", dt, dev), ps, lambda: (
            self.to_q.weight.detach().to(dt).contiguous(),
            self.to_kv.weight.detach()[:self.c].to(dt).contiguous(),
            self.to_kv.weight.detach()[self.c:].to(dt).contiguous(),
            F_.pack_rows([self.gating_linear.weight], dt, dev), F_.pack_vec([self.gating_bias], dt, dev),
            F_.pack_rows([self.o_linear.weight], dt, dev), F_.pack_vec([self.o_linear.bias], dt, dev)))

    def _run(self, x, out, resid, *, S, R, x_ss, x_sr, out_ss, out_sr, ln, mask, mask_ss, mask_sr):
        """Rows (s, j), s < S along the attended axis, j < R columns; see ``_fused.global_attention``."""
        dt, dev = x.dtype, x.device
        wq, wk, wv, wg, gb, wo, ob = self._pk(dt, dev)
        return F_.global_attention(x, out, resid, S=S, R=R, C=self.qkv_dim, H=self.n_head, D=self.c, x_ss=x_ss,
                                   x_sr=x_sr, out_ss=out_ss, out_sr=out_sr, ln=ln, wq=wq, wk=wk, wv=wv, wg_pk=wg,
                                   gb_pk=gb, wo_pk=wo, ob_pk=ob, c_out=self.out_dim, mask=mask, mask_ss=mask_ss,
                                   mask_sr=mask_sr, eps=self.eps, budget=_budget())

    def _train(self, m, mask):
        """ops.py:1174-1197, operator by operator (the un-chunked branch)."""
        from .kernel import bias_sigmod_ele, fused_softmax
        mask = mask.to(m.dtype)
        q = torch.sum(m * mask.unsqueeze(-1), dim=-2) / (torch.sum(mask, dim=-1)[..., None] + self.eps)
        q = self.to_q(q * self.scaling)
        q = q.view(q.shape[:-1] + (self.n_head, -1))                        # [1, R, H, c]
        k, v = self.to_kv(m).chunk(2, dim=-1)                               # [1, R, S, c]
        logits = torch.matmul(q, k.transpose(-1, -2))                       # [1, R, H, S]
        weights = fused_softmax(logits.unsqueeze(-2), mask.contiguous()).squeeze(-2)
        weighted_avg = torch.matmul(weights, v).flatten(-2)                 # [1, R, H * c]
        gate_values = self.gating_linear(m)
        weighted_avg = bias_sigmod_ele(gate_values, self.gating_bias, weighted_avg.unsqueeze(-2).expand_as(gate_values))
        return self.o_linear(weighted_avg)

    def forward(self, m, mask):
        """m [1, batch_size2, len, qkv_dim] (already normalised), mask [1, batch_size2, len] ->
        [1, batch_size2, len, out_dim]."""
        F_.check_cuda(m, mask)
        if _needs_grad(self, m):
            return self._train(m, mask)
        if m.dim() != 4 or m.shape[0] != 1 or m.shape[-1] != self.qkv_dim:
            raise RuntimeError("GlobalAttention: expected [1, B2, N, %d] input, got %s" % (self.qkv_dim, tuple(m.shape)))
        _, R, S, C = m.shape
        if m.stride(-1) != 1 or m.stride(1) % 8 or m.stride(2) % 8:
            m = m.contiguous()
        mk = mask.to(m.dtype)[0]
        out = torch.empty(1, R, S, self.out_dim, dtype=m.dtype, device=m.device)
        self._run(m, out, None, S=S, R=R, x_ss=m.stride(2), x_sr=m.stride(1), out_ss=self.out_dim,
                  out_sr=S * self.out_dim, ln=None, mask=mk, mask_ss=mk.stride(1), mask_sr=mk.stride(0))
        return out


class ChunkMSAColumnGlobalAttention(nn.Module):
    """M_raw + GlobalAttention(LayerNorm(M_raw) along the sequence axis) (ops.py:992-1043)."""

    def __init__(self, d_node, c=8, n_head=8):
        super(ChunkMSAColumnGlobalAttention, self).__init__()
        self.d_node = d_node
        self.c = c
        self.n_head = n_head
        self.layernormM = LayerNorm(d_node)
        self.global_attention = GlobalAttention(qkv_dim=d_node, c=c, n_head=n_head, out_dim=d_node)

    def _run(self, M_raw, M_mask, out):
        F_.check_cuda(M_raw, M_mask)
        _no_grad_guard(self, M_raw)
        if M_raw.dim() != 4 or M_raw.shape[0] != 1:
            raise RuntimeError("ChunkMSAColumnGlobalAttention: expected [1, s, r, C], got %s" % (tuple(M_raw.shape),))
        _, s, r, C = M_raw.shape
        mask = _mask_like(M_mask, M_raw)[0]               # [s, r]
        self.global_attention._run(M_raw, out, M_raw, S=s, R=r, x_ss=r * C, x_sr=C, out_ss=r * C, out_sr=C,
                                   ln=_ln_pair(self.layernormM, M_raw.dtype), mask=mask, mask_ss=r, mask_sr=1)
        return out

    def _train(self, M_raw, M_mask):
        """ops.py:1005-1010, operator by operator."""
        m = self.layernormM(M_raw.transpose(-2, -3))
        m = self.global_attention._train(m, M_mask.transpose(-1, -2))
        return M_raw + m.transpose(-2, -3)

    def forward(self, M_raw, M_mask):
        if _needs_grad(self, M_raw):
            return self._train(M_raw, M_mask)
        M_raw = M_raw.contiguous()
        return self._run(M_raw, M_mask, torch.empty_like(M_raw))

    def inplace(self, M_raw, M_mask):
        M_raw[0] = M_raw[0].contiguous()
        self._run(M_raw[0], M_mask, M_raw[0])
        return M_raw


def permute_final_dims(tensor, inds):
    """Permutes the last ``len(inds)`` axes of ``tensor`` by ``inds`` (reference: ops.py:366-369)."""
    n = len(inds)
    lead = tensor.dim() - n
    return tensor.permute(*range(lead), *(lead + i for i in inds))


class _TriangleMultiplication(nn.Module, _PackMixin):
    _incoming = False

    def __init__(self, d_pair, p_drop, c=128):
        super().__init__()
        self.d_pair = d_pair
        self.c = c
        self.layernorm1 = LayerNorm(d_pair)
        self.left_right_projection = Linear(d_pair, 2 * c)
        self.left_right_gate = Linear(d_pair, 2 * c, initializer='zeros', bias_init=1.)
        self.output_gate = Linear(d_pair, d_pair, initializer='zeros', bias_init=1.)
        self.layernorm2 = LayerNorm(c)
        self.output_projection = Linear(d_pair, d_pair, initializer='zeros', use_bias=False)
        self.output_bias = nn.parameter.Parameter(data=torch.zeros((d_pair,)), requires_grad=True)
        self.p_drop = p_drop

    def _run(self, Z_raw, Z_mask, out, xtail=None, drop=None):
        """``drop``: None or the [1, 1, r, C] dropout multipliers of a training-mode call (drawn by the caller)."""
        F_.check_cuda(Z_raw, Z_mask)
        _no_grad_guard(self, Z_raw)
        dt, dev = Z_raw.dtype, Z_raw.device
        if Z_raw.dim() != 4 or Z_raw.shape[0] != 1 or Z_raw.shape[1] != Z_raw.shape[2]:
            raise RuntimeError("TriangleMultiplication: expected [1, r, r, C], got %s" % (tuple(Z_raw.shape),))
        r, C = Z_raw.shape[1], Z_raw.shape[3]
        if not F_.fits_fused(C, dt) or not F_.fits_fused(self.c, dt):
            raise RuntimeError("TriangleMultiplication: unsupported widths %d / %d" % (C, self.c))
        ps = [self.left_right_projection.weight, self.left_right_projection.bias, self.left_right_gate.weight,
              self.left_right_gate.bias, self.output_gate.weight, self.output_gate.bias,
              self.output_projection.weight, self.output_bias, self.layernorm2.weight, self.layernorm2.bias,
              self.layernorm1.weight, self.layernorm1.bias]

        def build():
            w, b, n_glu = F_.pack_trimul(self.left_right_projection.weight, self.left_right_projection.bias,
                                         self.left_right_gate.weight, self.left_right_gate.bias,
                                         self.output_gate.weight, self.output_gate.bias, self.c, dt, dev)
            dual = None
            if F_.trimul_gate_in_output_stage(dt, r, C, self.c):
                dual = F_.pack_trimul_out(self.output_projection.weight, self.output_bias, self.output_gate.weight,
                                          self.output_gate.bias, C, dt, dev,
                                          ln_p=(self.layernorm2.weight, self.layernorm2.bias),
                                          ln_z=(self.layernorm1.weight, self.layernorm1.bias))
            return (w, b, n_glu, F_.pack_rows([self.output_projection.weight], dt, dev),
                    F_.pack_vec([self.output_bias], dt, dev), dual)
        w, b, n_glu, wout, bout, dual = self._packed(("tm", dt, dev, r % 8 == 0), ps, build)
        F_.triangle_multiplication(Z_raw, out, r=r, C=C, c=self.c, incoming=self._incoming,
                                   ln1=_ln_pair(self.layernorm1, dt), w_pk=w, b_pk=b, n_glu=n_glu,
                                   ln2=_ln_pair(self.layernorm2, dt), wout_pk=wout, out_bias_pk=bout,
                                   mask=_mask_like(Z_mask, Z_raw), dual_pk=dual, xtail=_check_tail(xtail, Z_raw),
                                   drop=None if drop is None else drop.reshape(r, C).contiguous())
        return out

    def _train(self, Z_raw, Z_mask, drop=None):
        """triangle.py:41-75 / :97-131, operator by operator.  ``drop``: dropout multipliers drawn by the caller
        ([1, 1, r, C]); None = drawn here in training mode."""
        from .kernel import bias_ele_dropout_residual
        Z = self.layernorm1(Z_raw)
        lr = Z_mask.unsqueeze(-1).to(Z.dtype) * self.left_right_projection(Z)
        lr = lr * torch.sigmoid(self.left_right_gate(Z))
        g = torch.sigmoid(self.output_gate(Z))
        # channel-major operands [c, i, k] / [c, j, k] in two allocations of their own (incoming: L[c, i, k] =
        # left[k, i, c]), the contraction and its two backward products on the library's own batched GEMM kernel, the
        # re-orderings on both sides on the library's transposition kernel
        r = Z_raw.shape[1]
        left, right = _ToChanMajorFn.apply(lr.contiguous(), self._incoming)
        p = _FromChanMajorFn.apply(_TriContractFn.apply(left, right, r), r)
        ab = self.output_projection(self.layernorm2(p))
        if drop is not None:
            return bias_ele_dropout_residual(ab, self.output_bias, g, drop, Z_raw, prob=0.0, training=False)
        dropout_mask = torch.ones_like(Z[:, 0:1, :, :])
        return bias_ele_dropout_residual(ab, self.output_bias, g, dropout_mask, Z_raw, prob=self.p_drop,
                                         training=self.training)

    def forward(self, Z_raw, Z_mask):
        if _needs_grad(self, Z_raw):
            return self._train(Z_raw, Z_mask)
        Z_raw = Z_raw.contiguous()
        return self._run(Z_raw, Z_mask, torch.empty_like(Z_raw))

    def inplace(self, Z_raw, Z_mask):
        Z_raw[0] = Z_raw[0].contiguous()
        self._run(Z_raw[0], Z_mask, Z_raw[0])
        return Z_raw


class AsyncChunkTriangleMultiplicationOutgoing(_TriangleMultiplication):
    """Algorithm 11 (ops.py:372-498): p[i,j] = sum_k a[i,k] b[j,k]."""
    _incoming = False


class AsyncChunkTriangleMultiplicationIncoming(_TriangleMultiplication):
    """Algorithm 12 (ops.py:501-630): p[i,j] = sum_k a[k,i] b[k,j]."""
    _incoming = True


class _TriangleAttention(nn.Module, _PackMixin):
    _ending = False

    def __init__(self, d_pair, p_drop, c=32, n_head=4):
        super().__init__()
        self.d_pair = d_pair
        self.c = c
        self.n_head = n_head
        self.p_drop = p_drop
        self.layernorm1 = LayerNorm(d_pair)
        self.linear_b = Linear(d_pair, n_head, initializer='linear', use_bias=False)
        self.attention = SelfAttention(qkv_dim=d_pair, c=c, n_head=n_head, out_dim=d_pair, gating=True,
                                       last_bias_fuse=True)
        self.out_bias = nn.parameter.Parameter(data=torch.zeros((d_pair,)), requires_grad=True)

    def _run(self, Z_raw, Z_mask, out, xtail=None, drop=None):
        """``drop``: None or the dropout multipliers of a training-mode call, [1, 1, r, C] (starting node) or
        [1, r, 1, C] (ending node)."""
        F_.check_cuda(Z_raw, Z_mask)
        _no_grad_guard(self, Z_raw)
        dt, dev = Z_raw.dtype, Z_raw.device
        self.attention._check(dt)
        if Z_raw.dim() != 4 or Z_raw.shape[0] != 1 or Z_raw.shape[1] != Z_raw.shape[2]:
            raise RuntimeError("TriangleAttention: expected [1, r, r, C], got %s" % (tuple(Z_raw.shape),))
        r, C = Z_raw.shape[1], Z_raw.shape[3]
        w_pk, gb_pk, wo_pk = self.attention.packed(dt, dev, extra_rows=lambda: self.linear_b.weight,
                                                  extra_params=[self.linear_b.weight])
        ob = self._packed(("ob", dt, dev), [self.out_bias], lambda: F_.pack_vec([self.out_bias], dt, dev))
        pbs = self._packed(("pbs", dt, dev), [self.linear_b.weight, self.layernorm1.weight, self.layernorm1.bias],
                           lambda: F_.PairBiasScratch(C, dev))
        mask = _mask_like(Z_mask, Z_raw)[0]
        if self._ending:    # logical row (j, i) reads z[i, j]; keys run along i
            a_map, sb, sn = (r, C, r * C), 1, r
        else:
            a_map, sb, sn = (r * r, 0, C), r, 1
        F_.attention(Z_raw, out, Z_raw, B2=r, N=r, C=C, H=self.n_head, a_map=a_map,
                     ln=_ln_pair(self.layernorm1, dt), w_pk=w_pk, gate_bias_pk=gb_pk, wo_pk=wo_pk, out_bias_pk=ob,
                     c_out=C, mask=mask, mask_sb=sb, mask_sn=sn, bias_t=None, bias_in_launch=True, pb_scratch=pbs,
                     head_dim=self.c, budget=_budget(), xtail=_check_tail(xtail, Z_raw),
                     drop=None if drop is None else drop.reshape(r, C).contiguous())     # logical row m: key index m % r
        return out

    def _train(self, Z_raw, Z_mask, drop=None):
        """triangle.py:156-173 (starting node) / :202-222 (ending node: the same on the transposed pair tensor, with
        the dropout mask shared along the other axis)."""
        from .kernel import bias_dropout_add
        Z = Z_raw.transpose(-2, -3) if self._ending else Z_raw
        mask = Z_mask.transpose(-1, -2) if self._ending else Z_mask
        Z = self.layernorm1(Z)
        b = self.linear_b(Z)
        Z = self.attention(Z, mask, (b, None))
        if self._ending:
            Z = Z.transpose(-2, -3)
            dropout_mask = torch.ones_like(Z[:, :, 0:1, :])
        else:
            dropout_mask = torch.ones_like(Z[:, 0:1, :, :])
        if drop is not None:
            return bias_dropout_add(Z, self.out_bias, drop, Z_raw, prob=0.0, training=False)
        return bias_dropout_add(Z, self.out_bias, dropout_mask, Z_raw, prob=self.p_drop, training=self.training)

    def forward(self, Z_raw, Z_mask):
        if _needs_grad(self, Z_raw):
            return self._train(Z_raw, Z_mask)
        Z_raw = Z_raw.contiguous()
        return self._run(Z_raw, Z_mask, torch.empty_like(Z_raw))

    def inplace(self, Z_raw, Z_mask):
        Z_raw[0] = Z_raw[0].contiguous()
        self._run(Z_raw[0], Z_mask, Z_raw[0])
        return Z_raw


class ChunkTriangleAttentionStartingNode(_TriangleAttention):
    """Algorithm 13 (ops.py:633-748): attention along each row of the pair representation."""
    _ending = False


class ChunkTriangleAttentionEndingNode(_TriangleAttention):
    """Algorithm 14 (ops.py:869-989): attention along each column."""
    _ending = True


def __getattr__(name):
    # the reference keeps these classes in this module; here they live in modules that import this one
    if name == "ChunkMSARowAttentionWithPairBias":
        from .msa import ChunkMSARowAttentionWithPairBias
        return ChunkMSARowAttentionWithPairBias
    if name in ("InputEmbedder", "RecyclingEmbedder", "TemplateAngleEmbedder", "TemplatePairEmbedder",
                "ExtraMSAEmbedder"):      # ops.py:1046-1145,1238-1334; embedders.py:257-372
        from . import embedders
        return getattr(embedders, name)
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
