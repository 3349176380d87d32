"""Torch-side (re)packing between plain tensors and the 32x32 operand tiles the attention
kernel consumes (see ``qk_tile_off`` / ``acc_tile_off`` in csrc/ffk_common.h).  On the hot
path these layouts are written directly by the projection kernel; the functions here serve
the stand-alone ``fused_attention_core`` op and the tests.
"""
import torch
import torch.nn.functional as F


def _pad_to(t, dim, mult):
    n = t.shape[dim]
    pad = (-n) % mult
    if pad == 0:
        return t
    spec = [0, 0] * (t.dim() - 1 - dim % t.dim()) + [0, pad]
    return F.pad(t, spec)


def n_tiles(n):
    return (n + 31) // 32


def tile_qk(x):
    """[B2, H, N, 32] -> [B2, H, NT, 2, 32, 16]   (element (n, d) at [n//32, d//16, n%32, d%16])."""
    B2, H, N, D = x.shape
    assert D == 32
    x = _pad_to(x, 2, 32)
    return x.view(B2, H, -1, 32, 2, 16).permute(0, 1, 2, 4, 3, 5).contiguous()


def untile_qk(t, N):
    B2, H, NT = t.shape[:3]
    return t.permute(0, 1, 2, 4, 3, 5).reshape(B2, H, NT * 32, 32)[:, :, :N]


def tile_rows_acc(x):
    """[B2, H, N, 32] -> [B2, H, NT, 2, 32, 4, 4]: FFK_TILE_ACC order, channel d = 8a + 4*half + b of
    token n at [n//32, half, n%32, a, b] (the lane that owns row n of a 32x32 accumulator holds its
    16 channels contiguously)."""
    B2, H, N, D = x.shape
    assert D == 32
    x = _pad_to(x, 2, 32)
    return x.view(B2, H, -1, 32, 4, 2, 4).permute(0, 1, 2, 5, 3, 4, 6).contiguous()


def untile_rows_acc(t, N):
    B2, H, NT = t.shape[:3]
    return t.permute(0, 1, 2, 4, 5, 3, 6).reshape(B2, H, NT * 32, 32)[:, :, :N]


def tile_acc(x):
    """[..., R, C32] with the row axis second to last (keys) and 32 columns ->
    [..., RT, 2, 32, 4, 4]: row = 8a + 4kg + b at [row//32, kg, col, a, b]."""
    lead = x.shape[:-2]
    assert x.shape[-1] == 32
    x = _pad_to(x, x.dim() - 2, 32)
    rt = x.shape[-2] // 32
    x = x.reshape(*lead, rt, 4, 2, 4, 32)                    # [rt, a, kg, b, col]
    nl = len(lead)
    return x.permute(*range(nl), nl, nl + 2, nl + 4, nl + 1, nl + 3).contiguous()   # [rt, kg, col, a, b]


def untile_acc(t, R):
    lead = t.shape[:-5]
    nl = len(lead)
    rt = t.shape[-5]
    x = t.permute(*range(nl), nl, nl + 3, nl + 1, nl + 4, nl + 2)  # [rt, a, kg, b, col]
    return x.reshape(*lead, rt * 32, 32)[..., :R, :]


def tile_v(v):
    """[B2, H, N, 32] -> [B2, H, NT, 2, 32, 4, 4]."""
    return tile_acc(v)


def untile_v(t, N):
    return untile_acc(t, N)


def tile_bias(b, scale=1.0):
    """[H, Nq, Nk] -> [H, QT, KT, 2, 32, 16]: element (k, q) of a tile at [q%32 // 16, k%32, q%16]
    (an MFMA operand with rows = keys and the tile's 32 queries as the reduction dim), times scale."""
    H, Nq, Nk = b.shape
    b = _pad_to(_pad_to(b, 1, 32), 2, 32) * scale
    qt, kt = b.shape[1] // 32, b.shape[2] // 32
    x = b.view(H, qt, 2, 16, kt, 32)                          # [h, qt, qhi, qlo, kt, k32]
    return x.permute(0, 1, 4, 2, 5, 3).contiguous()           # [h, qt, kt, qhi, k32, qlo]


def untile_bias(t, Nq, Nk):
    H, qt, kt = t.shape[:3]
    x = t.permute(0, 1, 3, 5, 2, 4)                           # [h, qt, qhi, qlo, kt, k32]
    return x.reshape(H, qt * 32, kt * 32)[:, :Nq, :Nk]
