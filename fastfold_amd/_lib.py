"""ctypes binding of libffk.so, the C-ABI kernel library (include/ffk.h).

The library is loaded from ``fastfold_amd/csrc/libffk.so`` (built in-tree by
``python -m fastfold_amd.csrc.build``).  There is no fallback: every op raises
``RuntimeError`` if the library is missing or a call returns a non-zero status.
Tensors cross the boundary as ``data_ptr()`` integers plus explicit shapes; the
launch stream is torch's current HIP stream.
"""
import ctypes
import os
from ctypes import c_int, c_int64, c_float, c_void_p, c_char_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libffk.so")

FFK_F32, FFK_BF16, FFK_F16 = 0, 1, 2
_DTYPE_TAG = {torch.float32: FFK_F32, torch.bfloat16: FFK_BF16, torch.float16: FFK_F16}

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float

# name -> argtypes; every entry of include/ffk.h that returns an int status
SIGNATURES = {
    "ffk_softmax_fwd": [_P, _P, _P, _P, _L, _L, _L, _L, _L, _I, _P],
    "ffk_softmax_bwd": [_P, _P, _P, _L, _L, _I, _P],
    "ffk_layernorm_fwd": [_P, _P, _P, _P, _P, _P, _L, _L, _F, _I, _P],
    "ffk_layernorm_bwd": [_P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _P],
    "ffk_bias_sigmoid_mul": [_P, _P, _P, _P, _L, _L, _I, _P],
    "ffk_bias_dropout_add": [_P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _L, _I, _P],
    "ffk_bias_ele_dropout_res": [_P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _L, _I, _P],
    "ffk_stream_copy": [_P, _P, _L, _P],
}

_lib = None


def load(path: str = None):
    """Loads libffk.so (once) and declares the prototypes."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise RuntimeError(
            "fastfold_amd: %s not found - build it with `python -m fastfold_amd.csrc.build` "
            "(there is no CPU or PyTorch fallback)" % p)
    lib = ctypes.CDLL(p)
    lib.ffk_version.restype = c_int
    lib.ffk_version.argtypes = []
    lib.ffk_last_error_string.restype = c_char_p
    lib.ffk_last_error_string.argtypes = []
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = argtypes
    _lib = lib
    return lib


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def dtype_tag(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_TAG[dtype]
    except KeyError:
        raise RuntimeError("fastfold_amd: unsupported dtype %s" % dtype)


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def ptr(t):
    """Device address of a tensor (None -> NULL; an address given as an int is passed through)."""
    return None if t is None else (t if isinstance(t, int) else t.data_ptr())


def check_device(*tensors):
    """The reference's CHECK_INPUT: every tensor on the GPU and contiguous
    (fastfold/model/fastnn/kernel/cuda_native/csrc/softmax_cuda_kernel.cu:12-16)."""
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("fastfold_amd: tensor must be a CUDA/HIP tensor (got %s)" % t.device)
        if not t.is_contiguous():
            raise RuntimeError("fastfold_amd: tensor must be contiguous")


# Optional per-launch timing: name -> list of (start_event, end_event, args).  Events are recorded
# on torch's current stream, which is the stream every kernel is launched on.
_TIMED = {}


def time_kernel(name, enable=True):
    """Starts (or stops) recording HIP events around every launch of entry point ``name``;
    returns the list the records go to: tuples (start_event, end_event, args)."""
    if enable:
        _TIMED[name] = []
        return _TIMED[name]
    return _TIMED.pop(name, None)


def call(name: str, *args):
    """Calls an entry point; raises RuntimeError with the library's message on failure."""
    lib = load()
    rec = _TIMED.get(name)
    if rec is not None:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        rc = getattr(lib, name)(*args)
        e1.record()
        rec.append((e0, e1, args))
    else:
        rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.ffk_last_error_string()
        raise RuntimeError("%s failed (status %d): %s" % (name, rc, msg.decode() if msg else "?"))


# ------------------------------------------------------------------ fused linear ----
FFK_TILE_STRIDED, FFK_TILE_QK, FFK_TILE_V, FFK_TILE_BIAS, FFK_TILE_ACC = 0, 1, 2, 3, 4
FFK_ACT_NONE, FFK_ACT_RELU, FFK_ACT_SIGMOID = 0, 1, 2
FFK_MAX_TILES = 10
LOG2E = 1.4426950408889634


class Tile(ctypes.Structure):
    """Mirror of ``ffk_tile`` (include/ffk.h)."""
    _fields_ = [
        ("out", c_void_p), ("bias", c_void_p), ("resid", c_void_p), ("gate", c_void_p), ("rowmask", c_void_p),
        ("s_o", c_int64), ("s_i", c_int64), ("s_h", c_int64), ("s_d", c_int64),
        ("gate_ld", c_int64), ("m_so", c_int64), ("m_si", c_int64),
        ("inner", c_int), ("kind", c_int), ("act", c_int), ("ncols", c_int), ("glu", c_int),
        ("scale", c_float), ("gate_rows", c_int), ("reserved", c_int),
        ("xtail", c_void_p),
    ]


class LinearDesc(ctypes.Structure):
    """Mirror of ``ffk_linear_desc`` (include/ffk.h)."""
    _fields_ = [
        ("a", c_void_p), ("a_so", c_int64), ("a_si", c_int64), ("a_cs", c_int64),
        ("a_inner", c_int), ("a_chanmajor", c_int),
        ("ln_gamma", c_void_p), ("ln_beta", c_void_p), ("ln_eps", c_float), ("dtype", c_int),
        ("w", c_void_p),
        ("M", c_int), ("K", c_int), ("n_tiles", c_int), ("ln_folded", c_int),
        ("a2", c_void_p), ("ln2_gamma", c_void_p), ("ln2_beta", c_void_p),
        ("a2_so", c_int64), ("a2_si", c_int64), ("a2_inner", c_int), ("variant", c_int),
        ("tiles", Tile * FFK_MAX_TILES),
    ]


SIGNATURES["ffk_fused_linear"] = [ctypes.POINTER(LinearDesc), _P]


def make_tile(out, *, kind=FFK_TILE_STRIDED, bias=None, resid=None, gate=None, gate_ld=0, rowmask=None,
              m_so=0, m_si=0, s_o=0, s_i=0, s_h=32, s_d=1, inner=1, act=FFK_ACT_NONE, ncols=128, glu=0,
              scale=1.0, gate_rows=0, xtail=None):
    """Builds one epilogue descriptor; tensors may be passed directly (their data_ptr is taken).  ``xtail`` is the
    int8 tail tensor (or its address) of ``resid`` / ``out`` as an extended residual stream."""
    def p(t):
        return None if t is None else (t if isinstance(t, int) else t.data_ptr())
    t = Tile()
    t.out, t.bias, t.resid, t.gate, t.rowmask = p(out), p(bias), p(resid), p(gate), p(rowmask)
    t.s_o, t.s_i, t.s_h, t.s_d = s_o, s_i, s_h, s_d
    t.gate_ld, t.m_so, t.m_si = gate_ld, m_so, m_si
    t.inner, t.kind, t.act, t.ncols, t.glu, t.scale = inner, kind, act, ncols, glu, scale
    t.gate_rows = gate_rows
    t.xtail = p(xtail)
    return t


def fused_linear(a, w, tiles, *, M, K, a_inner=None, a_so=0, a_si=None, a_chanmajor=False, a_cs=0,
                 ln=None, eps=1e-5, a_off=0, w_row_off=0, a2=None, ln2=None, a2_inner=None, a2_so=0, a2_si=None,
                 ln_rowsums=None, staged=False):
    """Launches ``ffk_fused_linear``.  ``a`` / ``w`` are tensors (``w`` packed [>= n_tiles*128, K]);
    ``ln`` is ``(gamma, beta)`` or None; ``a_off`` (elements) / ``w_row_off`` (rows) offset the bases.
    ``a2`` is the second operand the gate halves of GLU tiles are computed from; it goes with ``ln_rowsums``
    (fp32 [n_tiles * 128]) instead of ``ln``: both LayerNorms folded into ``w`` and the tile biases
    (``ln_folded`` in include/ffk.h).  ``ln2`` is accepted for symmetry and ignored."""
    d = LinearDesc()
    d.a = a.data_ptr() + a_off * a.element_size()
    d.a_inner = M if a_inner is None else a_inner
    d.a_so = a_so
    d.a_si = K if a_si is None else a_si
    d.a_cs = a_cs
    d.a_chanmajor = 1 if a_chanmajor else 0
    if ln is not None:
        d.ln_gamma, d.ln_beta = ln[0].data_ptr(), ln[1].data_ptr()
    if ln_rowsums is not None:
        if ln is not None or ln_rowsums.dtype != torch.float32 or ln_rowsums.numel() < 128 * len(tiles):
            raise RuntimeError("fused_linear: ln_rowsums must be fp32 [n_tiles * 128] and excludes ln")
        d.ln_gamma, d.ln_folded = ln_rowsums.data_ptr(), 1
    d.ln_eps = eps
    d.dtype = dtype_tag(a.dtype)
    d.w = w.data_ptr() + w_row_off * K * w.element_size()
    d.M, d.K, d.n_tiles = M, K, len(tiles)
    d.variant = 1 if staged else 0      # FFK_LINEAR_STAGED: the LDS-staged kernels even where the weights-stationary one applies
    if a2 is not None:
        if ln_rowsums is None:
            raise RuntimeError("fused_linear: a second operand needs folded LayerNorms (ln_rowsums)")
        d.a2 = a2.data_ptr()
        d.a2_inner = M if a2_inner is None else a2_inner
        d.a2_so = a2_so
        d.a2_si = K if a2_si is None else a2_si
    if len(tiles) > FFK_MAX_TILES:
        raise RuntimeError("fused_linear: at most %d N-tiles per launch" % FFK_MAX_TILES)
    if w.shape[0] < w_row_off + 128 * len(tiles) or w.shape[1] != K or w.dtype != a.dtype:
        raise RuntimeError("fused_linear: packed weight must be [%d, %d] %s, got %s %s"
                           % (128 * len(tiles), K, a.dtype, tuple(w.shape), w.dtype))
    for i, t in enumerate(tiles):
        d.tiles[i] = t
    call("ffk_fused_linear", ctypes.byref(d), stream_ptr())


# ------------------------------------------------------------------ batched GEMM ----
class BgemmDesc(ctypes.Structure):
    """Mirror of ``ffk_bgemm_desc`` (include/ffk.h)."""
    _fields_ = [
        ("a", c_void_p), ("b", c_void_p), ("out", c_void_p), ("bias", c_void_p), ("resid", c_void_p),
        ("rowdiv", c_void_p), ("xtail", c_void_p),
        ("lda", c_int64), ("ldb", c_int64), ("a_bs", c_int64), ("b_bs", c_int64), ("o_bs", c_int64),
        ("s_o", c_int64), ("s_i", c_int64), ("s_h", c_int64), ("s_d", c_int64),
        ("inner", c_int), ("M", c_int), ("N", c_int), ("K", c_int), ("batch", c_int),
        ("dtype", c_int), ("act", c_int), ("out_f32", c_int),
        ("scale", c_float), ("div_eps", c_float),
    ]


SIGNATURES["ffk_bgemm_nt"] = [ctypes.POINTER(BgemmDesc), _P]
SIGNATURES["ffk_attention_fwd"] = [_P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _I, _I, _P]
SIGNATURES["ffk_key_bias"] = [_P, _P, _P, _L, _L, _L, _L, _I, _P]


def bgemm_nt(a, b, out, *, M, N, K, lda, ldb, batch=1, a_bs=0, b_bs=0, o_bs=0, inner=None, s_o=0, s_i=None,
             s_h=32, s_d=1, bias=None, resid=None, rowdiv=None, div_eps=0.0, act=FFK_ACT_NONE, scale=1.0,
             out_f32=False, dtype=None, xtail=None):
    """Launches ``ffk_bgemm_nt``; default output addressing is row-major [M, N] (``s_i`` = N).  ``xtail``: int8 tail
    of ``resid`` / ``out`` as an extended residual stream."""
    def p(t):
        return None if t is None else (t if isinstance(t, int) else t.data_ptr())
    d = BgemmDesc()
    d.a, d.b, d.out, d.bias, d.resid, d.rowdiv = p(a), p(b), p(out), p(bias), p(resid), p(rowdiv)
    d.xtail = p(xtail)
    d.lda, d.ldb, d.a_bs, d.b_bs, d.o_bs = lda, ldb, a_bs, b_bs, o_bs
    d.inner = M if inner is None else inner
    d.s_o, d.s_i, d.s_h, d.s_d = s_o, (N if s_i is None else s_i), s_h, s_d
    d.M, d.N, d.K, d.batch = M, N, K, batch
    d.dtype = dtype_tag(a.dtype if dtype is None else dtype)
    d.act, d.out_f32, d.scale, d.div_eps = act, 1 if out_f32 else 0, scale, div_eps
    call("ffk_bgemm_nt", ctypes.byref(d), stream_ptr())


FFK_ATT_GATE_TILED = 1
FFK_ATT_BIAS_PADDED = 2
FFK_ATT_HALF_K = 4


def attention_fwd(out, q_t, k_t, v_t, bias_t, keybias, tileflags, gate, *, B2, H, Nq, Nk, D=32, gate_tiled=False,
                  bias_padded=False, half_k=False):
    call("ffk_attention_fwd", ptr(out), ptr(q_t), ptr(k_t), ptr(v_t), ptr(bias_t), ptr(keybias), ptr(tileflags),
         ptr(gate),
         B2, H, Nq, Nk, D, (FFK_ATT_GATE_TILED if gate_tiled else 0) | (FFK_ATT_BIAS_PADDED if bias_padded else 0)
         | (FFK_ATT_HALF_K if half_k else 0),
         dtype_tag(q_t.dtype), stream_ptr())


SIGNATURES["ffk_attention_bwd"] = [_P] * 16 + [_L, _L, _L, _L, _L, _F, _F, _I, _P]


def attention_bwd(dq, dk, dv, dbias, lse, dsum, q_qk, q_acc, k_qk, k_acc, v_qk, bias_t, keybias, do_qk, do_acc,
                  o_qk, *, B2, H, Nq, Nk, dq_scale, dk_scale, D=32):
    call("ffk_attention_bwd", ptr(dq), ptr(dk), ptr(dv), ptr(dbias), ptr(lse), ptr(dsum), ptr(q_qk), ptr(q_acc), ptr(k_qk),
         ptr(k_acc), ptr(v_qk), ptr(bias_t), ptr(keybias), ptr(do_qk), ptr(do_acc), ptr(o_qk), B2, H, Nq, Nk, D,
         dq_scale, dk_scale, dtype_tag(q_qk.dtype), stream_ptr())


SIGNATURES["ffk_tile_pack"] = [_P, _P, _L, _L, _L, _L, _L, _L, _L, _F, _I, _I, _P]
SIGNATURES["ffk_transpose_batched"] = [_P, _P, _L, _L, _L, _L, _L, _L, _L, _I, _P]


def transpose_batched(out, inp, *, B, X, Y, in_bs, in_xs, out_bs, out_ys, out_off=0, in_off=0):
    """out[b][y][x] = in[b][x][y] with element strides (see include/ffk.h); ``out_off`` / ``in_off``: element offsets
    added to the tensors' data pointers."""
    if not (out.is_cuda and inp.is_cuda) or out.device != inp.device:
        raise RuntimeError("fastfold_amd: tensors must be CUDA/HIP tensors on one device (got %s / %s)" % (out.device, inp.device))
    if out.dtype != inp.dtype:
        raise RuntimeError("transpose_batched: dtype mismatch %s / %s" % (out.dtype, inp.dtype))
    es = inp.element_size()
    call("ffk_transpose_batched", out.data_ptr() + out_off * es, inp.data_ptr() + in_off * es, B, X, Y, in_bs, in_xs,
         out_bs, out_ys, dtype_tag(inp.dtype), stream_ptr())


def tile_pack(x, kind, scale=1.0):
    """[B2, H, N, D] (any strides over the first three dims, channels contiguous) -> operand tiles of the attention
    kernels in ``kind`` order (``FFK_TILE_QK`` / ``FFK_TILE_V``), times ``scale``: [B2, H, ceil(N/32), 1024] for
    D <= 32 (channels past D zero), [D/32, B2, H, ceil(N/32), 1024] - one block per 32-channel part of the head - for
    D = 64 or 128."""
    import torch
    if x.dim() != 4 or (x.shape[-1] > 32 and x.shape[-1] not in (64, 128)):
        raise RuntimeError("tile_pack: expected [B2, H, N, D] with D <= 32, 64 or 128, got %s" % (tuple(x.shape),))
    if x.stride(-1) != 1:
        x = x.contiguous()
    B2, H, N, D = x.shape
    parts = max(1, D // 32)
    out = torch.empty(parts, B2, H, (N + 31) // 32, 1024, dtype=x.dtype, device=x.device)
    if out.numel():
        for p in range(parts):
            call("ffk_tile_pack", ptr(out[p]), x.data_ptr() + p * 32 * x.element_size(), B2, H, N, min(D, 32),
                 x.stride(0), x.stride(1), x.stride(2), float(scale), kind, dtype_tag(x.dtype), stream_ptr())
    return out[0] if D <= 32 else out


SIGNATURES["ffk_pair_bias"] = [_P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _F, _F, _I, _P]


def pair_bias(bias_t, z, gamma, beta, w, scratch, *, N, C, H, a_inner, a_so, a_si, scale, eps=1e-5):
    call("ffk_pair_bias", ptr(bias_t), ptr(z), ptr(gamma), ptr(beta), ptr(w), ptr(scratch), N, C, H, a_inner, a_so, a_si,
         scale, eps, dtype_tag(z.dtype), stream_ptr())


SIGNATURES["ffk_pair_bias_static"] = [_P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _F, _F, _I, _P]


def pair_bias_static(bias_t, z, gamma, beta, w, *, N, C, H, a_inner, a_so, a_si, scale, eps=1e-5):
    """``ffk_pair_bias`` without a scratch tensor: the library's per-GPU static array holds the weight operand."""
    call("ffk_pair_bias_static", ptr(bias_t), ptr(z), ptr(gamma), ptr(beta), ptr(w), N, C, H, a_inner, a_so, a_si,
         scale, eps, dtype_tag(z.dtype), stream_ptr())


SIGNATURES["ffk_opm_fused"] = [_P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _F, _I, _P]


def opm_fused(out, resid, a_t, b_t, w2p, bias, norm, *, r, spad, eps, xtail=None):
    call("ffk_opm_fused", ptr(out), ptr(resid), ptr(xtail), ptr(a_t), ptr(b_t), ptr(w2p), ptr(bias), ptr(norm), r, spad,
         eps, dtype_tag(a_t.dtype), stream_ptr())


SIGNATURES["ffk_transition_fused"] = [_P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _L, _F, _I, _P]


def transition_fused(out, x, gamma, beta, w1, b1, w2, b2, *, M, C, hidden, eps=1e-5, xtail=None):
    call("ffk_transition_fused", ptr(out), ptr(x), ptr(xtail), ptr(gamma), ptr(beta), ptr(w1), ptr(b1), ptr(w2), ptr(b2), M, C,
         hidden, eps, dtype_tag(x.dtype), stream_ptr())


SIGNATURES["ffk_gated_out_fused"] = [_P] * 10 + [_L, _L, _L, _L, _L, _F, _I, _P]


def gated_out_fused(out, x, gamma, beta, wg, bg, o, wo, bo, *, M, C, inner, s_o, s_i, eps=1e-5, xtail=None):
    """out = x + Wo (sigmoid(Wg LN(x) + bg) * o) + bo over logical rows (see include/ffk.h)."""
    call("ffk_gated_out_fused", ptr(out), ptr(x), ptr(xtail), ptr(gamma), ptr(beta), ptr(wg), ptr(bg), ptr(o), ptr(wo), ptr(bo),
         M, C, inner, s_o, s_i, eps, dtype_tag(o.dtype), stream_ptr())


def key_bias(keybias, tileflags, mask, *, B, N, mask_sb=0, mask_sn=1):
    call("ffk_key_bias", ptr(keybias), ptr(tileflags), ptr(mask), B, N, mask_sb, mask_sn,
         dtype_tag(mask.dtype) if mask is not None else FFK_F32, stream_ptr())


SIGNATURES["ffk_global_attention_core"] = [_P, _P, _P, _P, _P, _F, _P, _P, _P, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                                           _F, _F, _I, _P]


def global_attention_core(o, m, mask, gamma, beta, wq, wk, wv, *, S, R, C, H, D, m_ss, m_sr, mask_ss, mask_sr,
                          scaling, eps, ln_eps=1e-5):
    call("ffk_global_attention_core", ptr(o), ptr(m), ptr(mask), ptr(gamma), ptr(beta), ln_eps, ptr(wq), ptr(wk),
         ptr(wv), S, R, C, H, D, m_ss, m_sr, mask_ss, mask_sr, scaling, eps, dtype_tag(m.dtype), stream_ptr())


FFK_EMBED_RELPOS, FFK_EMBED_DISTOGRAM = 0, 1
SIGNATURES["ffk_pair_embed"] = [_P, _P, _P, _P, _F, _P, _P, _P, _P, _I, _P, _P, _F, _L, _L, _L, _I, _P]


def pair_embed(out, z, gamma, beta, table, bias, row, col, *, mode, pos, edges=None, inf=1e8, r, C, nb, ln_eps=1e-5):
    call("ffk_pair_embed", ptr(out), ptr(z), ptr(gamma), ptr(beta), ln_eps, ptr(table), ptr(bias), ptr(row), ptr(col),
         mode, ptr(pos), ptr(edges), inf, r, C, nb, dtype_tag(out.dtype), stream_ptr())


SIGNATURES["ffk_pointwise_attention_core"] = [_P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _L, _I, _P]


def pointwise_attention_core(o, q, kv, bias, *, P, H, D, NT, kv_st, kv_sp, v_off, out_scale=None):
    """o[p, h] = softmax_t(q[p, h] . k[t, p, h] + bias[t]) v[t, p, h]; strides in elements (see include/ffk.h)."""
    check_device(o, q, kv, bias)
    if bias.dtype != torch.float32 or bias.numel() != NT:
        raise RuntimeError("pointwise_attention_core: bias must be fp32 [NT]")
    if out_scale is not None and (out_scale.dtype != torch.float32 or out_scale.numel() != 1 or not out_scale.is_cuda):
        raise RuntimeError("pointwise_attention_core: out_scale must be one fp32 value on the device")
    call("ffk_pointwise_attention_core", ptr(o), ptr(q), ptr(kv), ptr(bias), ptr(out_scale), P, H, D, NT, kv_st, kv_sp, v_off,
         dtype_tag(q.dtype), stream_ptr())
