"""Launch sequences of the HIP kernels for each Evoformer sub-module (single GPU, DAP size 1).

These functions take plain tensors plus weights already packed for the kernels and issue
C-ABI calls only; torch is used for buffer allocation and for re-packing weights (once per
weight version).  Row-addressing conventions are those of ``ffk_fused_linear``: logical row
``m = hi * inner + lo`` lives at ``hi * s_o + lo * s_i``.
"""
import contextlib
import math
import os

import torch

from fastfold_amd import _lib
from fastfold_amd._lib import (FFK_ACT_NONE, FFK_ACT_RELU, FFK_ACT_SIGMOID, FFK_TILE_ACC, FFK_TILE_BIAS, FFK_TILE_QK,
                               FFK_TILE_STRIDED, FFK_TILE_V, LOG2E, make_tile)

_WS_BUDGET_DEFAULT = 6 << 30     # bytes of scratch one sub-module may hold at a time
_WS_BUDGET_CHUNKED = 1 << 30     # when the user asked for chunking (set_chunk_size)


def es_of(dtype):
    return 4 if dtype == torch.float32 else 2


def vec_of(dtype):
    return 16 // es_of(dtype)


def round_up(x, m):
    return (x + m - 1) // m * m


def alloc(shape, dtype, device, zero=False):
    return (torch.zeros if zero else torch.empty)(shape, dtype=dtype, device=device)


def pack_rows(mats, dtype, device):
    """cat([n_i, K]) zero-padded to a multiple of 128 rows, in the kernel dtype."""
    w = torch.cat([m.detach().to(device=device, dtype=dtype) for m in mats], 0)
    n, npad = w.shape[0], round_up(w.shape[0], 128)
    if npad != n:
        w = torch.cat([w, w.new_zeros(npad - n, w.shape[1])], 0)
    return w.contiguous()


def pack_vec(vecs, dtype, device, total=None):
    v = torch.cat([x.detach().to(device=device, dtype=dtype).reshape(-1) for x in vecs], 0)
    total = round_up(v.numel(), 128) if total is None else total
    if total != v.numel():
        v = torch.cat([v, v.new_zeros(total - v.numel())], 0)
    return v.contiguous()


def check_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("fastfold_amd: the Evoformer modules run on the GPU only "
                               "(got a %s tensor); there is no CPU fallback" % t.device)


def check_nonempty(who, *ts):
    """The kernels take at least one sequence and one residue; an empty tensor is an error of the caller."""
    for t in ts:
        if t is not None and t.numel() == 0:
            raise RuntimeError("%s: empty input tensor of shape %s" % (who, tuple(t.shape)))


# ---- values derived from a mask only (key bias + tile flags of an attention, the normaliser of the outer
# product mean) are the same in every block of a stack: inside `mask_cache()` they are computed once ----
_MASK_CACHE = None


@contextlib.contextmanager
def mask_cache():
    """While active, launches whose result depends only on a mask tensor are done once per distinct
    (storage, view geometry, version) and reused.  Entries keep their mask alive, so its memory cannot be
    handed to another tensor while the entry exists; the cache dies with the context."""
    global _MASK_CACHE
    prev, _MASK_CACHE = _MASK_CACHE, []
    try:
        yield
    finally:
        _MASK_CACHE = prev


def _mask_derived(mask, what, build):
    if _MASK_CACHE is None:
        return build()
    key = (what, mask.data_ptr(), mask._version, tuple(mask.shape), tuple(mask.stride()), mask.dtype)
    for k, _, v in _MASK_CACHE:
        if k == key:
            return v
    v = build()
    if len(_MASK_CACHE) < 32:          # a stack needs about ten; bounded whatever the caller does
        _MASK_CACHE.append((key, mask, v))
    return v


class PairBiasScratch:
    """Device scratch of ffk_pair_bias together with the fact that it already holds the weight operand
    (built by the first call from the projection weights and the LayerNorm parameters); modules keep one
    per packed weight set, so that later calls skip the preparation kernel."""

    def __init__(self, C, device):
        self.buf = torch.empty(16 * C + 16, dtype=torch.float32, device=device)
        self.ready = False


def _pair_bias_launch(bias_t, x, ln, w, scratch, **kw):
    if scratch is None:
        scratch = PairBiasScratch(x.shape[-1], x.device)
    _lib.pair_bias(bias_t, x, ln[0], ln[1], None if scratch.ready else w, scratch.buf, **kw)
    scratch.ready = True


def fits_fused(K, dtype):
    return K <= 256 and K % 32 == 0


# ------------------------------------------------------------------------- linear ----
def linear(x2, w_pk, b_pk, N, *, act=FFK_ACT_NONE, out=None, resid=None, ln=None):
    """out[M, N] = act(LN(x2)[M, K] @ W^T + b) (+ resid).  ``w_pk`` is [>=N (padded to 128), K]."""
    M, K = x2.shape
    dt, dev = x2.dtype, x2.device
    es = es_of(dt)
    if out is None:
        out = torch.empty(M, N, dtype=dt, device=dev)
    if M == 0:
        return out
    if fits_fused(K, dt) and N % vec_of(dt) == 0:
        nt = (N + 127) // 128
        for t0 in range(0, nt, _lib.FFK_MAX_TILES):
            tiles = []
            for t in range(t0, min(nt, t0 + _lib.FFK_MAX_TILES)):
                tiles.append(make_tile(out.data_ptr() + t * 128 * es,
                                       bias=None if b_pk is None else b_pk.data_ptr() + t * 128 * es,
                                       resid=None if resid is None else resid.data_ptr() + t * 128 * es,
                                       inner=M, s_i=N, act=act, ncols=min(128, N - t * 128)))
            _lib.fused_linear(x2, w_pk, tiles, M=M, K=K, ln=ln, w_row_off=t0 * 128)
    else:
        if ln is not None:
            raise RuntimeError("linear: LayerNorm prologue needs K <= 256")
        if K % vec_of(dt) != 0:
            raise RuntimeError("linear: in_features=%d must be a multiple of %d for %s" % (K, vec_of(dt), dt))
        _lib.bgemm_nt(x2, w_pk, out, M=M, N=N, K=K, lda=K, ldb=K, bias=b_pk, resid=resid, act=act)
    return out


# --------------------------------------------------------------------- transition ----
def xtail_ptr(xtail, off=0):
    """Address of element ``off`` of an int8 residual tail (None stays None)."""
    return None if xtail is None else xtail.data_ptr() + off


# False: every transition runs as projection + GEMM with the hidden activation in HBM (tests compare the two)
_FUSED_TRANSITION = True


def transition(x, out, *, ln, w1_pk, b1_pk, w2, b2, hidden, budget, xtail=None):
    """out = x + W2 relu(W1 LN(x) + b1) + b2 over rows of x [M, C]; out may alias x.  ``xtail`` (here and in the
    other sub-modules): int8 tensor of x's shape holding the tail bytes of x / out as an extended residual stream."""
    M, C = x.shape
    dt, dev = x.dtype, x.device
    es = es_of(dt)
    if dt == torch.bfloat16 and C in (128, 256) and hidden == 4 * C and ln is not None and _FUSED_TRANSITION:
        # both layers in one kernel, hidden activation kept on chip
        _lib.transition_fused(out, x, ln[0], ln[1], w1_pk, b1_pk, w2, b2, M=M, C=C, hidden=hidden, xtail=xtail)
        return out
    rows = max(128, min(M, (budget // (hidden * es)) // 128 * 128))
    hid = torch.empty(min(rows, M), hidden, dtype=dt, device=dev)
    nt = hidden // 128
    for r0 in range(0, M, rows):
        n = min(rows, M - r0)
        per = 4 if (dt == torch.bfloat16 and C == 256) else _lib.FFK_MAX_TILES
        for t0 in range(0, nt, per):
            tiles = [make_tile(hid.data_ptr() + t * 128 * es, bias=b1_pk.data_ptr() + t * 128 * es, inner=n,
                               s_i=hidden, act=FFK_ACT_RELU)
                     for t in range(t0, min(nt, t0 + per))]
            _lib.fused_linear(x, w1_pk, tiles, M=n, K=C, ln=ln, a_off=r0 * C, w_row_off=t0 * 128)
        _lib.bgemm_nt(hid, w2, out.data_ptr() + r0 * C * es, M=n, N=C, K=hidden, lda=hidden, ldb=hidden, bias=b2,
                      resid=x.data_ptr() + r0 * C * es, dtype=dt, xtail=xtail_ptr(xtail, r0 * C))
    return out


# ---------------------------------------------------------------------- attention ----
def attention(x, out, resid, *, B2, N, C, H, a_map, ln, w_pk, gate_bias_pk, wo_pk, out_bias_pk, c_out,
              mask, mask_sb, mask_sn, bias_t=None, bias_in_launch=False, pb_scratch=None, head_dim=32, budget=None, o_map=None, xtail=None,
              drop=None):
    """Gated multi-head attention over N tokens for each of B2 batch rows.  The kernels work on 32-wide
    heads; a narrower head (``head_dim`` < 32) arrives zero-padded to 32 channels in ``w_pk`` / ``wo_pk``,
    which changes neither the scores nor the used output channels - only the score scale is its own.

    x holds the C-channel rows addressed by ``a_map = (inner, s_o, s_i)`` with ``inner`` either B2 * N (plain
    row-major) or N (one batch row per outer step); w_pk is the packed [q; k; v; gate(; bias)] weight.  The
    attention update is projected by wo_pk and written as ``out = resid + update + out_bias`` with the same row
    addressing, or with ``o_map`` if the output rows have another width (``resid=None``: no residual).  With ``bias_in_launch`` the last N-tile of w_pk produces the
    [H, N, N] additive bias into ``bias_t`` from the same normalised rows.

    ``budget`` (bytes) bounds the operand buffers (q, k, v, gate and the head outputs: 5 * H * ceil(N / 32) KB
    elements per batch row): the batch rows are then processed in slabs - projection, core, output projection per
    slab.  Batch rows are independent and a slab's outputs overwrite only the rows it read, so this also holds
    when ``out`` aliases ``x``; the additive bias, which reads all of x, is computed before the first slab.

    ``drop``: None, or a [period, c_out] tensor of dropout multipliers (0 or 1 / (1 - p)) that scales the update of logical
    row m by its row ``m % period`` before the residual is added (the shared-axis dropout of the training mode:
    ``bias_dropout_add`` with a mask drawn by the caller).
    """
    dt, dev = x.dtype, x.device
    es = es_of(dt)
    HC = H * 32
    if HC % 128 != 0:
        raise RuntimeError("attention: n_head * 32 must be a multiple of 128 (got %d heads)" % H)
    M = B2 * N
    NT = (N + 31) // 32
    zero = (N % 32) != 0
    a_inner, a_so, a_si = a_map
    o_inner, o_so, o_si = a_map if o_map is None else o_map
    if a_inner not in (M, N) or o_inner != a_inner:
        raise RuntimeError("attention: row maps with inner=%d / %d fit neither B2 * N nor N" % (a_inner, o_inner))
    per_row = 5 * H * NT * 1024 * es
    slab = B2 if budget is None else min(B2, max(2, (budget // per_row) // 2 * 2))
    q_t = alloc((slab, H, NT, 1024), dt, dev, zero)
    k_t = alloc((slab, H, NT, 1024), dt, dev, zero)
    v_t = alloc((slab, H, NT, 1024), dt, dev, zero)
    # With bf16, 128 input channels and whole key tiles the projection runs on the weights-stationary
    # kernel, which writes q, k and the gate in accumulator order straight from its registers.
    acc_order = dt == torch.bfloat16 and C in (64, 128, 256) and N % 32 == 0
    qk_kind = FFK_TILE_ACC if acc_order else FFK_TILE_QK
    # Where the update goes back into the tensor the gate is computed from (every attention of the Evoformer block),
    # the gate is not a tensor at all: the output stage computes sigmoid(Wg LN(x) + bg) from the rows of x it reads as
    # residual anyway and multiplies the heads' outputs by it on their way into the output projection
    # (ffk_gated_out_fused).  The projection launch then writes q, k, v only and the core reads no gate.
    # Measured at N_seq = 128, same box: on the triangle attentions at N_res = 1024 the projection and the core each get
    # ~ 3 % faster and the output stage as much slower - 1.1 GB less memory traffic per block at the same block time; at
    # N_res = 256 a block gains 1.4 % (0.631 vs 0.640 ms) since the output stage runs three workgroups per CU (with two
    # it lost 1.3 %); on the MSA attentions (256 channels, two workgroups per CU) it loses slightly at both sizes.
    # Shorter rows were not measured and keep the gate tensor.  The choice depends on the row length and the width only, never on the number of
    # batch rows: a subset of the batch rows must give the bits of the full call.
    gate_in_out = (_GATE_IN_OUT_STAGE and drop is None and N >= _GATE_IN_OUT_MIN_N and C in _GATE_IN_OUT_WIDTHS and acc_order
                   and ln is not None and HC == C and c_out == C and resid is not None and o_map is None
                   and resid.data_ptr() == x.data_ptr() and a_so % 16 == 0 and a_si % 16 == 0)
    gate = None
    if not gate_in_out:
        gate = torch.empty((slab, H, NT, 1024) if acc_order else (slab * N, HC), dtype=dt, device=dev)
    o = torch.empty(slab * N, HC, dtype=dt, device=dev)
    tpg = HC // 128
    qscale = LOG2E / math.sqrt(float(head_dim))
    tkw = dict(inner=N, s_o=H * NT * 1024, s_h=NT * 1024)
    bias_tile = None
    # rows of a bias buffer the caller leaves to this function (bias_in_launch with bias_t None) end in one unused tile
    # when the projection launch writes them: with 2^n key tiles per row every query-tile row would start in the same
    # memory channel (-2 % per triangle-attention launch at N = 1024, measured three times on one box)
    will_ride = (bias_in_launch and acc_order and C == 128 and H <= 4 and slab >= B2 and _PAIR_BIAS_RIDES
                 and (not gate_in_out or hasattr(w_pk, "without_gate")))
    bias_padded = will_ride and _BIAS_ROW_PAD and bias_t is None
    if bias_in_launch:
        ntp = NT + (1 if bias_padded else 0)
        if bias_t is None:
            bias_t = alloc((H, NT, ntp, 1024), dt, dev, zero=(N % 32) != 0)
        bias_tile = make_tile(bias_t, kind=FFK_TILE_BIAS, inner=N, s_o=ntp * 1024, s_h=NT * ntp * 1024, ncols=H,
                              scale=LOG2E)
    # With 128 input channels, at most four heads and all rows in one slab the bias rides on the projection launch:
    # the weights-stationary kernel computes its four dot products per row (small MFMAs) from the rows it
    # has in LDS anyway (one read of x less than a pass of its own; -0.05 ms per triangle attention at N = 1024).
    rides = will_ride
    # Otherwise the skinny bias projection has its own pass over x.  It goes first: x was written by the launch before
    # this call and is still (partly) cache-resident, and the bias pass writes little, so the projection after
    # it finds x as warm as before - the other way round the projection's output (four times the size of x)
    # has pushed x out by the time the bias pass reads it (measured: -0.65 % block time at N = 1024).
    if rides:
        pass
    elif bias_tile is not None and acc_order and C in (64, 128):
        _pair_bias_launch(bias_t, x, ln, w_pk[4 * tpg * 128:], pb_scratch, N=N, C=C, H=H, a_inner=a_inner,
                          a_so=a_so, a_si=a_si, scale=LOG2E)
        bias_tile = None
    if bias_tile is not None and not rides and (acc_order or slab < B2):     # its own launch over all rows, before x changes
        _lib.fused_linear(x, w_pk, [bias_tile], M=M, K=C, a_inner=a_inner, a_so=a_so, a_si=a_si, ln=ln,
                          w_row_off=4 * tpg * 128)
        bias_tile = None
    def key_bias():
        kb = torch.empty(B2, NT * 32, dtype=torch.float32, device=dev)
        flags = torch.empty(B2, NT, dtype=torch.int32, device=dev)
        _lib.key_bias(kb, flags, mask, B=B2, N=N, mask_sb=mask_sb, mask_sn=mask_sn)
        return kb, flags
    kb, flags = _mask_derived(mask, ("key_bias", B2, N, mask_sb, mask_sn), key_bias) if mask is not None else key_bias()
    for b0 in range(0, B2, slab):
        nb = min(slab, B2 - b0)
        Ms = nb * N
        # rows b0 * N ... of the map: a shifted base, and an inner extent that still covers the slab
        off, inner = (b0 * N * a_si, Ms) if a_inner == M else (b0 * a_so, N)
        o_off = b0 * N * o_si if a_inner == M else b0 * o_so
        tiles = []
        for buf, kind, scale in ((q_t, qk_kind, qscale), (k_t, qk_kind, 1.0), (v_t, FFK_TILE_V, 1.0)):
            for t in range(tpg):
                tiles.append(make_tile(buf.data_ptr() + t * 4 * NT * 1024 * es, kind=kind, scale=scale, **tkw))
        for t in range(0 if gate_in_out else tpg):
            if acc_order:
                tiles.append(make_tile(gate.data_ptr() + t * 4 * NT * 1024 * es, kind=FFK_TILE_ACC,
                                       bias=gate_bias_pk.data_ptr() + t * 128 * es, act=FFK_ACT_SIGMOID, **tkw))
            else:
                tiles.append(make_tile(gate.data_ptr() + t * 128 * es, bias=gate_bias_pk.data_ptr() + t * 128 * es,
                                       inner=Ms, s_i=HC, act=FFK_ACT_SIGMOID))
        if bias_tile is not None:      # single slab: the bias rides on the projection launch
            tiles.append(bias_tile)
        # the weights-stationary kernel holds at most 16 (K = 256) or 24 (K = 128) 32-channel units per launch
        per = (3 if gate_in_out else 4) if (acc_order and C == 256) else len(tiles)
        for t0 in range(0, len(tiles), per):
            # a bias tile riding behind q, k, v (no gate tiles) takes its weight rows from the gate-less packing
            wp = w_pk.without_gate if (gate_in_out and bias_tile is not None) else w_pk
            _lib.fused_linear(x, wp, tiles[t0:t0 + per], M=Ms, K=C, a_inner=inner, a_so=a_so, a_si=a_si, ln=ln,
                              w_row_off=t0 * 128, a_off=off)
        _lib.attention_fwd(o, q_t, k_t, v_t, bias_t, kb[b0:b0 + nb], flags[b0:b0 + nb], gate, B2=nb, H=H, Nq=N, Nk=N,
                           gate_tiled=acc_order, bias_padded=bias_padded,
                           half_k=head_dim <= (16 if acc_order else 8))
        if gate_in_out:
            # packed rows of w_pk: q, k, v, gate blocks of HC rows each; o holds the slab's rows in logical order
            _lib.gated_out_fused(out.data_ptr() + o_off * es, x.data_ptr() + off * es, ln[0], ln[1],
                                 w_pk.data_ptr() + 3 * HC * C * es, gate_bias_pk, o, wo_pk, out_bias_pk, M=Ms, C=C,
                                 inner=inner, s_o=a_so, s_i=a_si,
                                 xtail=None if xtail is None else xtail.data_ptr() + o_off)
            continue
        tiles = []
        for t in range((c_out + 127) // 128):
            tiles.append(make_tile(out.data_ptr() + (o_off + t * 128) * es,
                                   bias=None if out_bias_pk is None else out_bias_pk.data_ptr() + t * 128 * es,
                                   resid=None if resid is None else resid.data_ptr() + (o_off + t * 128) * es,
                                   xtail=xtail_ptr(xtail, o_off + t * 128),
                                   gate=None if drop is None else drop.data_ptr() + t * 128 * es,
                                   gate_ld=0 if drop is None else c_out, gate_rows=0 if drop is None else drop.shape[0],
                                   inner=inner, s_o=o_so, s_i=o_si, ncols=min(128, c_out - t * 128)))
        _lib.fused_linear(o, wo_pk, tiles, M=Ms, K=HC)
    return out


def pair_bias(z, *, r, C, H, ln, wb_pk, pb_scratch=None):
    """bias_t[h][q/32][k/32][tile] = log2e * (LN(z)[q, k, :] . Wb[h, :]) in score-accumulator tiles."""
    NT = (r + 31) // 32
    bias_t = alloc((H, NT, NT, 1024), z.dtype, z.device, zero=(r % 32) != 0)
    if z.dtype == torch.bfloat16 and C in (64, 128) and H <= 8:
        _pair_bias_launch(bias_t, z, ln, wb_pk, pb_scratch, N=r, C=C, H=H, a_inner=r * r, a_so=0, a_si=C, scale=LOG2E)
        return bias_t
    tile = make_tile(bias_t, kind=FFK_TILE_BIAS, inner=r, s_o=NT * 1024, s_h=NT * NT * 1024, ncols=H, scale=LOG2E)
    _lib.fused_linear(z, wb_pk, [tile], M=r * r, K=C, ln=ln)
    return bias_t


# ----------------------------------------------------------- triangle multiplication ----
def pack_trimul(proj_w, proj_b, gate_w, gate_b, og_w, og_b, c, dtype, device):
    """[left GLU tiles | right GLU tiles | output-gate tiles]; a GLU tile packs 64 channels as
    [p c0..c0+31 | g c0..c0+31 | p c0+32..c0+63 | g c0+32..c0+63]."""
    if c % 64 != 0:
        raise RuntimeError("triangle multiplication: hidden width must be a multiple of 64, got %d" % c)
    ws, bs = [], []
    for side in range(2):
        for t in range(c // 64):
            for q in range(2):
                sl = slice(side * c + t * 64 + q * 32, side * c + t * 64 + q * 32 + 32)
                ws += [proj_w[sl], gate_w[sl]]
                bs += [proj_b[sl], gate_b[sl]]
    n_glu = 2 * (c // 64)
    w = pack_rows(ws, dtype, device)
    b = pack_vec(bs, dtype, device)
    wg = pack_rows([og_w], dtype, device)
    bg = pack_vec([og_b], dtype, device)
    return torch.cat([w, wg], 0).contiguous(), torch.cat([b, bg], 0).contiguous(), n_glu


def pack_trimul_out(out_w, out_b, og_w, og_b, C, dtype, device, ln_p, ln_z):
    """Output stage with the gate computed in the same launch: GLU tiles of 64 channels,
    [Wout c0..c0+31 | Wog c0..c0+31 | Wout c0+32..c0+63 | Wog c0+32..c0+63] (biases alike), with both
    LayerNorms folded in: ``ln_p = (gamma, beta)`` of the contraction result into the value rows, ``ln_z`` of the
    pair tensor into the gate rows (W' = W * gamma rounded to the kernel dtype, b' = W beta + b).  Returns
    (weights, biases, fp32 row sums of W' in the same packed order)."""
    def fold(w, b, ln):
        w, b = w.detach().float(), b.detach().float()
        gam, bet = ln[0].detach().float(), ln[1].detach().float()
        wf = (w * gam[None, :]).to(dtype).float()
        return wf, w @ bet + b, wf.sum(1)
    out_w, out_b, out_rs = fold(out_w, out_b, ln_p)
    og_w, og_b, og_rs = fold(og_w, og_b, ln_z)
    ws, bs, cs = [], [], []
    for t in range(C // 64):
        for q in range(2):
            sl = slice(t * 64 + q * 32, t * 64 + q * 32 + 32)
            ws += [out_w[sl], og_w[sl]]
            bs += [out_b[sl], og_b[sl]]
            cs += [out_rs[sl], og_rs[sl]]
    return pack_rows(ws, dtype, device), pack_vec(bs, dtype, device), pack_vec(cs, torch.float32, device)


def trimul_gate_in_output_stage(dtype, r, C, c):
    """The output gate sigmoid(Wg LN(z) + bg) can be computed inside the output stage (second operand
    of the projection kernel) instead of being written by the first stage and read back."""
    return dtype == torch.bfloat16 and C == 128 and c == 128 and r % 8 == 0


# Elements between the channel planes of the triangle multiplication's operands and of its contraction result, beyond the
# r * kpad the data needs.  With planes exactly 2 MB apart (N_res = 1024, bf16) the 32 lanes of a channel-major store of
# the projection kernel - one channel each - all land in the same memory channel; 128 bytes of padding spread them
# (block 6.97 -> 6.885 ms in a same-box A/B at N_res = 1024; 64, 192 and 1088 elements measure the same).
_TRIMUL_CHAN_PAD = 64
_PAIR_BIAS_RIDES = True      # see attention(): switch for same-box comparisons
_BIAS_ROW_PAD = True         # see attention(): switch for same-box comparisons
_GATE_IN_OUT_STAGE = True    # see attention(): False keeps the gate a tensor (written by the projection, read by the core)
_GATE_IN_OUT_MIN_N = 256         # shortest attended axis for which the gate moves into the output stage
_GATE_IN_OUT_WIDTHS = (128,)     # ... and the channel widths (the kernel is built for 128 and 256)


def triangle_multiplication(z, out, *, r, C, c, incoming, ln1, w_pk, b_pk, n_glu, ln2, wout_pk, out_bias_pk, mask,
                            dual_pk=None, xtail=None, drop=None):
    """out = z + sigmoid(Wg LN(z) + bg) * (Wout LN2(p) + b_out),  p[i,j,:] = sum_k a[i,k,:] b[j,k,:]
    (outgoing) or sum_k a[k,i,:] b[k,j,:] (incoming), a/b the masked gated projections.
    ``dual_pk`` = (weights, biases) of pack_trimul_out: the gate is then computed in the output stage.
    ``drop``: None, or [r, C] dropout multipliers shared by all rows i (the update of (i, j) is scaled by drop[j]): the
    gate tensor is multiplied by it, so the output stage is the one with a gate tensor."""
    dt, dev = z.dtype, z.device
    es = es_of(dt)
    M = r * r
    kpad = round_up(r, vec_of(dt))
    zero = kpad != r
    # channel planes of the operands and of the contraction result are cs elements apart (_TRIMUL_CHAN_PAD beyond r * kpad)
    cs = r * kpad + _TRIMUL_CHAN_PAD
    lr = alloc((2, c, cs), dt, dev, zero)
    dual = dual_pk is not None and drop is None and trimul_gate_in_output_stage(dt, r, C, c)
    g = None if dual else torch.empty(M, C, dtype=dt, device=dev)
    tiles = []
    if incoming:      # logical row (a, b) reads z[b, a]
        a_map, m_so, m_si = (r, C, r * C), 1, r
    else:
        a_map, m_so, m_si = (M, 0, C), r, 1
    for side in range(2):
        for t in range(c // 64):
            ti = side * (c // 64) + t
            tiles.append(make_tile(lr.data_ptr() + (side * c + t * 64) * cs * es,
                                   bias=b_pk.data_ptr() + ti * 128 * es, glu=1, ncols=64, inner=r, s_o=kpad, s_i=1,
                                   s_h=32 * cs, s_d=cs, rowmask=mask, m_so=m_so, m_si=m_si))
    for t in range((C + 127) // 128 if not dual else 0):
        kw = dict(inner=r, s_o=C, s_i=r * C) if incoming else dict(inner=M, s_i=C)
        tiles.append(make_tile(g.data_ptr() + t * 128 * es, bias=b_pk.data_ptr() + (n_glu + t) * 128 * es,
                               act=FFK_ACT_SIGMOID, ncols=min(128, C - t * 128), **kw))
    _lib.fused_linear(z, w_pk, tiles, M=M, K=C, a_inner=a_map[0], a_so=a_map[1], a_si=a_map[2], ln=ln1)
    if drop is not None:
        g.view(r, r, C).mul_(drop[None])
    p = torch.empty(c, cs, dtype=dt, device=dev)
    _lib.bgemm_nt(lr[0], lr[1], p, M=r, N=r, K=kpad, lda=kpad, ldb=kpad, batch=c, a_bs=cs, b_bs=cs,
                  o_bs=cs, s_i=kpad)
    del lr
    if dual:
        wd, bd, rowsums = dual_pk
        tiles = [make_tile(out.data_ptr() + t * 64 * es, bias=bd.data_ptr() + t * 128 * es, glu=1, ncols=64,
                           resid=z.data_ptr() + t * 64 * es, xtail=xtail_ptr(xtail, t * 64), inner=M, s_i=C)
                 for t in range(C // 64)]
        # both LayerNorms (of p and of z) are folded into the packed weights: no normalisation pass over either
        _lib.fused_linear(p, wd, tiles, M=M, K=c, a_inner=r, a_so=kpad, a_si=1, a_chanmajor=True, a_cs=cs,
                          ln_rowsums=rowsums, a2=z, a2_inner=M, a2_si=C)
        return out
    tiles = []
    for t in range((C + 127) // 128):
        tiles.append(make_tile(out.data_ptr() + t * 128 * es, bias=out_bias_pk.data_ptr() + t * 128 * es,
                               gate=g.data_ptr() + t * 128 * es, gate_ld=C, resid=z.data_ptr() + t * 128 * es,
                               xtail=xtail_ptr(xtail, t * 128), inner=M, s_i=C, ncols=min(128, C - t * 128)))
    _lib.fused_linear(p, wout_pk, tiles, M=M, K=c, a_inner=r, a_so=kpad, a_si=1, a_chanmajor=True, a_cs=cs,
                      ln=ln2)
    return out


# ------------------------------------------------------------------ outer product mean ----
def outer_product_mean(m, mask, z, out, *, s, r, C, Cz, ln, wab_pk, bab_pk, wo, bo, budget, eps=1e-3, wo_ed=None,
                       xtail=None):
    """out = z + (Wo vec(sum_s a[s,i,:] (x) b[s,j,:]) + bo) / (sum_s mask[s,i] mask[s,j] + eps),
    a, b the masked 32-channel projections of LN(m).  m is [s, r, C] rows, mask [s, r]."""
    dt, dev = m.dtype, m.device
    es = es_of(dt)
    spad = round_up(s, vec_of(dt))
    ab = alloc((2, r * 32, spad), dt, dev, zero=spad != s)
    tile = make_tile(ab, bias=bab_pk, ncols=64, inner=s, s_o=32 * spad, s_i=1, s_h=r * 32 * spad, s_d=spad,
                     rowmask=mask, m_so=1, m_si=r)
    # logical row (i, s') reads m[s', i]
    _lib.fused_linear(m, wab_pk, [tile], M=s * r, K=C, a_inner=s, a_so=C, a_si=r * C, ln=ln)
    def normaliser():
        mt = torch.zeros(r, spad, dtype=dt, device=dev)
        mt[:, :s] = mask.t()
        nrm = torch.empty(r, r, dtype=torch.float32, device=dev)
        _lib.bgemm_nt(mt, mt, nrm, M=r, N=r, K=spad, lda=spad, ldb=spad, out_f32=True)
        return nrm
    nrm = _mask_derived(mask, ("opm_norm", s, r, spad), normaliser)
    if wo_ed is not None and dt == torch.bfloat16 and Cz == 128 and r % 32 == 0 and spad in (64, 128):
        # fused core: the [r, r, 1024] outer product never leaves the chip
        _lib.opm_fused(out, z, ab[0], ab[1], wo_ed, bo, nrm, r=r, spad=spad, eps=eps, xtail=xtail)
        return out
    ci = max(1, min(r, budget // (r * 1024 * es)))
    O = torch.empty(ci * r, 1024, dtype=dt, device=dev)
    for i0 in range(0, r, ci):
        n = min(ci, r - i0)
        _lib.bgemm_nt(ab.data_ptr() + i0 * 32 * spad * es, ab[1], O, M=32 * n, N=32 * r, K=spad, lda=spad, ldb=spad,
                      inner=32, s_o=r * 1024, s_i=32, s_h=1024, s_d=1, dtype=dt)
        _lib.bgemm_nt(O, wo, out.data_ptr() + i0 * r * Cz * es, M=n * r, N=Cz, K=1024, lda=1024, ldb=1024, bias=bo,
                      rowdiv=nrm.data_ptr() + i0 * r * 4, div_eps=eps, resid=z.data_ptr() + i0 * r * Cz * es, dtype=dt,
                      xtail=xtail_ptr(xtail, i0 * r * Cz))
    return out


# --------------------------------------------------------------- global attention ----
def global_attention(x, out, resid, *, S, R, C, H, D, x_ss, x_sr, out_ss, out_sr, ln, wq, wk, wv, wg_pk, gb_pk,
                     wo_pk, ob_pk, c_out, mask, mask_ss, mask_sr, eps, budget):
    """Global column attention (one mean query per column j, shared key / value head):
    out[s, j] = (resid[s, j] +) Wo (sigmoid(Wg LN(x[s, j]) + bg) * o[j]) + bo, o from
    ``ffk_global_attention_core``.  Row (s, j) of x is at ``s * x_ss + j * x_sr`` (elements), of out /
    resid at ``s * out_ss + j * out_sr``; ``ln = None`` takes x as already normalised."""
    dt, dev = x.dtype, x.device
    es = es_of(dt)
    HD = H * D
    if not fits_fused(C, dt) or not fits_fused(HD, dt) or HD > 128 or c_out % vec_of(dt) != 0:
        raise RuntimeError("global_attention: unsupported widths C=%d, H*D=%d, out=%d" % (C, HD, c_out))
    o = torch.empty(R, HD, dtype=dt, device=dev)
    _lib.global_attention_core(o, x, mask, None if ln is None else ln[0], None if ln is None else ln[1], wq, wk, wv,
                               S=S, R=R, C=C, H=H, D=D, m_ss=x_ss, m_sr=x_sr, mask_ss=mask_ss, mask_sr=mask_sr,
                               scaling=D ** -0.5, eps=eps)
    # gate and output projection, a bounded number of sequences at a time
    sc = max(1, min(S, budget // max(1, R * HD * es)))
    tmp = torch.empty(sc * R, HD, dtype=dt, device=dev)
    for s0 in range(0, S, sc):
        n = min(sc, S - s0)
        M = n * R
        gate_tile = make_tile(tmp, bias=gb_pk, inner=M, s_i=HD, act=FFK_ACT_SIGMOID, ncols=HD, gate=o, gate_ld=HD,
                              gate_rows=R)
        _lib.fused_linear(x, wg_pk, [gate_tile], M=M, K=C, a_inner=R, a_so=x_ss, a_si=x_sr, ln=ln, a_off=s0 * x_ss)
        tiles = []
        for t in range((c_out + 127) // 128):
            tiles.append(make_tile(out.data_ptr() + (s0 * out_ss + t * 128) * es,
                                   bias=None if ob_pk is None else ob_pk.data_ptr() + t * 128 * es,
                                   resid=None if resid is None else resid.data_ptr() + (s0 * out_ss + t * 128) * es,
                                   inner=R, s_o=out_ss, s_i=out_sr, ncols=min(128, c_out - t * 128)))
        _lib.fused_linear(tmp, wo_pk, tiles, M=M, K=HD)
    return out
