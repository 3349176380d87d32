"""GPU parity of ffk_fused_linear (through the C ABI) against float64 numpy linear algebra
(oracle.ops_np): every prologue / epilogue / layout the Evoformer modules use."""
import numpy as np
import pytest
import torch

from oracle import ops_np

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}   # relative to max |ref|


def _np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def _pack(w, n_tiles):
    out = torch.zeros(n_tiles * 128, w.shape[1], dtype=w.dtype, device=w.device)
    out[: w.shape[0]] = w
    return out


def _rel(got, ref):
    return np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-6)


def _sig(x):
    return 1.0 / (1.0 + np.exp(-x))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,K,N", [(300, 128, 256), (129, 256, 200), (64, 64, 36), (1000, 256, 1024)])
def test_plain_bias_relu_rowmajor(dev, dtype, M, K, N):
    from fastfold_amd import _lib
    g = torch.Generator().manual_seed(M + K)
    a = torch.randn(M, K, generator=g).to(dev, dtype)
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(dev, dtype)
    b = torch.randn(N, generator=g).to(dev, dtype)
    nt = (N + 127) // 128
    wp, bp = _pack(w, nt), torch.zeros(nt * 128, dtype=dtype, device=dev)
    bp[:N] = b
    out = torch.full((M, N), 7.0, dtype=dtype, device=dev)
    tiles = [_lib.make_tile(out.data_ptr() + i * 128 * out.element_size(), bias=bp.data_ptr() + i * 128 * out.element_size(),
                            inner=M, s_i=N, act=_lib.FFK_ACT_RELU, ncols=min(128, N - i * 128)) for i in range(nt)]
    if N % (16 // out.element_size()) != 0:
        pytest.skip("row pitch not 16-byte aligned")
    _lib.fused_linear(a, wp, tiles, M=M, K=K)
    ref = np.maximum(ops_np.linear(_np(a), _np(w), _np(b)), 0)
    assert _rel(_np(out), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K", [128, 256])
def test_layernorm_prologue_resid_gate_inplace(dev, dtype, K):
    from fastfold_amd import _lib
    M, N = 333, 128
    g = torch.Generator().manual_seed(K)
    a = (torch.randn(M, K, generator=g) * 2 + 0.5).to(dev, dtype)
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(dev, dtype)
    b = torch.randn(N, generator=g).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(K, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(K, generator=g)).to(dev, dtype)
    gate = torch.rand(M, N, generator=g).to(dev, dtype)
    z = torch.randn(M, N, generator=g).to(dev, dtype)
    z0 = z.clone()
    tiles = [_lib.make_tile(z, bias=b, resid=z, gate=gate, gate_ld=N, inner=M, s_i=N)]
    _lib.fused_linear(a, _pack(w, 1), tiles, M=M, K=K, ln=(gam, bet))
    x = ops_np.layer_norm(_np(a), _np(gam), _np(bet))
    if dtype == torch.bfloat16:
        x = _np(torch.from_numpy(x).to(torch.bfloat16))       # the kernel rounds LN output to the operand dtype
    ref = _np(z0) + _np(gate) * ops_np.linear(x, _np(w), _np(b))
    assert _rel(_np(z), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_transposed_rows_in_and_out(dev, dtype):
    """A is z[I,J,C] traversed as (j, i); the update is written back to z[i, j]."""
    from fastfold_amd import _lib
    I, J, C = 21, 13, 128
    g = torch.Generator().manual_seed(3)
    z = torch.randn(I, J, C, generator=g).to(dev, dtype)
    w = (torch.randn(C, C, generator=g) / C ** 0.5).to(dev, dtype)
    z0 = z.clone()
    # logical row m = j * I + i  ->  z[i, j]
    tiles = [_lib.make_tile(z, resid=z, inner=I, s_o=C, s_i=J * C)]
    _lib.fused_linear(z0, _pack(w, 1), tiles, M=I * J, K=C, a_inner=I, a_so=C, a_si=J * C)
    ref = _np(z0) + ops_np.linear(_np(z0), _np(w))
    assert _rel(_np(z), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r", [24, 37])
def test_glu_rowmask_channel_major(dev, dtype, r):
    """Triangle-multiplication projection: (Wp x + bp) * sigmoid(Wg x + bg) * mask, stored [c][i][kpad]."""
    from fastfold_amd import _lib
    C, Ch = 128, 128
    kpad = (r + 7) // 8 * 8
    g = torch.Generator().manual_seed(r)
    z = torch.randn(r, r, C, generator=g).to(dev, dtype)
    wp = (torch.randn(Ch, C, generator=g) / C ** 0.5).to(dev, dtype)
    wg = (torch.randn(Ch, C, generator=g) / C ** 0.5).to(dev, dtype)
    bp, bg = torch.randn(Ch, generator=g).to(dev, dtype), torch.randn(Ch, generator=g).to(dev, dtype)
    mask = (torch.rand(r, r, generator=g) > 0.2).to(dev, dtype)
    # packed tiles: [p 0..31 | g 0..31 | p 32..63 | g 32..63] per 128 rows
    idx = []
    wcat, bcat = [], []
    for t in range(Ch // 64):
        for q in range(2):
            sl = slice(t * 64 + q * 32, t * 64 + q * 32 + 32)
            wcat += [wp[sl], wg[sl]]
            bcat += [bp[sl], bg[sl]]
    wpk, bpk = torch.cat(wcat).contiguous(), torch.cat(bcat).contiguous()
    for transposed in (False, True):
        out = torch.zeros(Ch, r, kpad, dtype=dtype, device=dev)
        es = out.element_size()
        tiles = []
        for t in range(Ch // 64):
            tiles.append(_lib.make_tile(out.data_ptr() + t * 64 * r * kpad * es, bias=bpk.data_ptr() + t * 128 * es,
                                        glu=1, ncols=64, inner=r, s_o=kpad, s_i=1, s_h=32 * r * kpad, s_d=r * kpad,
                                        rowmask=mask, m_so=(1 if transposed else r), m_si=(r if transposed else 1)))
        if transposed:   # logical row (a, b) reads z[b, a]
            _lib.fused_linear(z, wpk, tiles, M=r * r, K=C, a_inner=r, a_so=C, a_si=r * C)
        else:
            _lib.fused_linear(z, wpk, tiles, M=r * r, K=C)
        zz = _np(z).transpose(1, 0, 2) if transposed else _np(z)
        mm = _np(mask).T if transposed else _np(mask)
        ref = ops_np.linear(zz, _np(wp), _np(bp)) * _sig(ops_np.linear(zz, _np(wg), _np(bg))) * mm[..., None]
        got = _np(out)[:, :, :r].transpose(1, 2, 0)
        assert _rel(got, ref) < TOL[dtype]
        assert float(out[:, :, r:].abs().max()) == 0.0 if kpad > r else True


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B2,N,H", [(3, 70, 4), (2, 32, 8)])
def test_attention_operand_tiles(dev, dtype, B2, N, H):
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    C = H * 32
    K = 128
    g = torch.Generator().manual_seed(N)
    x = torch.randn(B2, N, K, generator=g).to(dev, dtype)
    wq, wk, wv = ((torch.randn(C, K, generator=g) / K ** 0.5).to(dev, dtype) for _ in range(3))
    NT = layouts.n_tiles(N)
    q = torch.zeros(B2, H, NT, 2, 32, 16, dtype=dtype, device=dev)
    k = torch.zeros_like(q)
    v = torch.zeros(B2, H, NT, 2, 32, 4, 4, dtype=dtype, device=dev)
    es = q.element_size()
    tiles, ws = [], []
    for buf, w, kind, scale in ((q, wq, _lib.FFK_TILE_QK, 0.25), (k, wk, _lib.FFK_TILE_QK, 1.0), (v, wv, _lib.FFK_TILE_V, 1.0)):
        for t in range(C // 128):
            tiles.append(_lib.make_tile(buf.data_ptr() + t * 4 * NT * 1024 * es, kind=kind, inner=N, s_o=H * NT * 1024,
                                        s_h=NT * 1024, scale=scale))
            ws.append(w[t * 128:(t + 1) * 128])
    _lib.fused_linear(x, torch.cat(ws).contiguous(), tiles, M=B2 * N, K=K)
    for buf, w, un, scale in ((q, wq, layouts.untile_qk, 0.25), (k, wk, layouts.untile_qk, 1.0), (v, wv, layouts.untile_v, 1.0)):
        ref = (ops_np.linear(_np(x), _np(w)) * scale).reshape(B2, N, H, 32).transpose(0, 2, 1, 3)
        assert _rel(_np(un(buf, N)), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r,H", [(45, 4), (64, 8)])
def test_bias_tiles(dev, dtype, r, H):
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    C = 128
    g = torch.Generator().manual_seed(r)
    z = torch.randn(r, r, C, generator=g).to(dev, dtype)
    wb = (torch.randn(H, C, generator=g) / C ** 0.5).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    T = layouts.n_tiles(r)
    for transposed in (False, True):
        bt = torch.zeros(H, T, T, 2, 32, 16, dtype=dtype, device=dev)
        tile = _lib.make_tile(bt, kind=_lib.FFK_TILE_BIAS, inner=r, s_o=T * 1024, s_h=T * T * 1024, ncols=H, scale=_lib.LOG2E)
        kw = dict(a_inner=r, a_so=C, a_si=r * C) if transposed else {}
        _lib.fused_linear(z, _pack(wb, 1), [tile], M=r * r, K=C, ln=(gam, bet), **kw)
        zz = _np(z).transpose(1, 0, 2) if transposed else _np(z)
        x = ops_np.layer_norm(zz, _np(gam), _np(bet))
        if dtype == torch.bfloat16:
            x = _np(torch.from_numpy(x).to(torch.bfloat16))
        ref = (ops_np.linear(x, _np(wb)) * _lib.LOG2E).transpose(2, 0, 1)       # [h, q, k]
        assert _rel(_np(layouts.untile_bias(bt, r, r)), ref) < TOL[dtype]


@pytest.mark.parametrize("r,H", [(45, 4), (64, 3), (33, 1)])
def test_bias_tile_rides_on_a_projection_launch(dev, r, H):
    """A trailing FFK_TILE_BIAS tile in a launch of the weights-stationary kernel (bf16, K = 128, <= 4 heads): computed
    on the vector pipe from the slab rows, no weight slot.  Checked against numpy, against the staged kernels on the
    same descriptor, in both traversal orders; the other tile of the launch is unaffected and the padding of ragged
    bias tiles stays zero."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    dtype, C = torch.bfloat16, 128
    g = torch.Generator().manual_seed(r * 7 + H)
    z = (torch.randn(r, r, C, generator=g) * 1.3 + 0.2).to(dev, dtype)
    w = (torch.randn(128, C, generator=g) / C ** 0.5).to(dev, dtype)
    wb = (torch.randn(H, C, generator=g) / C ** 0.5).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    wpk = torch.cat([_pack(w, 1), _pack(wb, 1)]).contiguous()
    T = layouts.n_tiles(r)
    for transposed in (False, True):
        res = []
        for staged in (False, True):
            y = torch.zeros(r * r, 128, dtype=dtype, device=dev)
            bt = torch.zeros(H, T, T, 2, 32, 16, dtype=dtype, device=dev)
            tiles = [_lib.make_tile(y, inner=r * r, s_i=128),
                     _lib.make_tile(bt, kind=_lib.FFK_TILE_BIAS, inner=r, s_o=T * 1024, s_h=T * T * 1024, ncols=H,
                                    scale=_lib.LOG2E)]
            kw = dict(a_inner=r, a_so=C, a_si=r * C) if transposed else {}
            _lib.fused_linear(z, wpk, tiles, M=r * r, K=C, ln=(gam, bet), staged=staged, **kw)
            res.append((y, bt))
        zz = _np(z).transpose(1, 0, 2) if transposed else _np(z)
        x = _np(torch.from_numpy(ops_np.layer_norm(zz, _np(gam), _np(bet))).to(dtype))
        ref = (ops_np.linear(x, _np(wb)) * _lib.LOG2E).transpose(2, 0, 1)       # [h, q, k]
        for y, bt in res:
            assert _rel(_np(layouts.untile_bias(bt, r, r)), ref) < 1e-2
            assert _rel(_np(y), ops_np.linear(x, _np(w)).reshape(r * r, 128)) < TOL[dtype]
            full = _np(layouts.untile_bias(bt, T * 32, T * 32))
            assert np.abs(full[:, r:, :]).max(initial=0.0) == 0.0 and np.abs(full[:, :, r:]).max(initial=0.0) == 0.0
        assert _rel(_np(res[0][1]), _np(res[1][1])) < 1e-2
        assert torch.equal(res[0][0], res[1][0]) or _rel(_np(res[0][0]), _np(res[1][0])) < 1e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,with_ln", [(128, True), (64, True), (64, False)])
@pytest.mark.parametrize("r", [40, 27, 104])
def test_channel_major_a_with_layernorm(dev, dtype, r, C, with_ln):
    """Triangle-multiplication output stage: A[(i,j), c] = P[c][i][jpad], at the Evoformer's 128 channels and the
    template stack's 64."""
    from fastfold_amd import _lib
    jpad = (r + 7) // 8 * 8
    g = torch.Generator().manual_seed(r + C)
    P = torch.randn(C, r, jpad, generator=g).to(dev, dtype)
    w = (torch.randn(C, C, generator=g) / C ** 0.5).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    b = torch.randn(C, generator=g).to(dev, dtype)
    gate = torch.rand(r * r, C, generator=g).to(dev, dtype)
    z = torch.randn(r, r, C, generator=g).to(dev, dtype)
    z0 = z.clone()
    tiles = [_lib.make_tile(z, bias=b, resid=z, gate=gate, gate_ld=C, inner=r * r, s_i=C, ncols=C)]
    _lib.fused_linear(P, _pack(w, 1), tiles, M=r * r, K=C, a_inner=r, a_so=jpad, a_si=1, a_chanmajor=True,
                      a_cs=r * jpad, ln=(gam, bet) if with_ln else None)
    x = _np(P)[:, :, :r].transpose(1, 2, 0)
    if with_ln:
        x = ops_np.layer_norm(x, _np(gam), _np(bet))
        if dtype == torch.bfloat16:
            x = _np(torch.from_numpy(x).to(torch.bfloat16))
    ref = _np(z0) + _np(gate).reshape(r, r, C) * ops_np.linear(x, _np(w), _np(b))
    assert _rel(_np(z), ref) < TOL[dtype]


def test_bad_descriptors_are_rejected(dev):
    from fastfold_amd import _lib
    a = torch.zeros(64, 100, device=dev)
    w = torch.zeros(128, 100, device=dev)
    out = torch.zeros(64, 128, device=dev)
    with pytest.raises(RuntimeError):
        _lib.fused_linear(a, w, [_lib.make_tile(out, inner=64, s_i=128)], M=64, K=100)     # K % 32
    a = torch.zeros(64, 128, device=dev)
    w = torch.zeros(128, 128, device=dev)
    with pytest.raises(RuntimeError):
        _lib.fused_linear(a, w, [_lib.make_tile(out, inner=0, s_i=128)], M=64, K=128)      # inner
    with pytest.raises(RuntimeError):
        _lib.fused_linear(a, w, [_lib.make_tile(out, inner=64, s_i=128, s_d=2, resid=out)], M=64, K=128)


def test_weights_stationary_many_slabs(dev):
    """bf16, K = 128, more slabs than workgroups (persistent loop, ragged last slab): q in accumulator
    order with a scale, k in q/k order, v, a sigmoid gate in accumulator order and a plain relu tile,
    all from one LayerNorm-ed pass over A."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    dtype = torch.bfloat16
    B2, N, H, K = 131, 288, 4, 128                      # M = 37728 rows = 294.75 slabs
    C = H * 32
    M = B2 * N
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(B2, N, K, generator=g) + 0.3).to(dev, dtype)
    ws_ = [(torch.randn(C, K, generator=g) / K ** 0.5).to(dev, dtype) for _ in range(5)]
    bias_g = torch.randn(C, generator=g).to(dev, dtype)
    bias_r = torch.randn(C, generator=g).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(K, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(K, generator=g)).to(dev, dtype)
    NT = layouts.n_tiles(N)
    q = torch.zeros(B2, H, NT, 2, 32, 4, 4, dtype=dtype, device=dev)
    k = torch.zeros(B2, H, NT, 2, 32, 16, dtype=dtype, device=dev)
    v = torch.zeros(B2, H, NT, 2, 32, 4, 4, dtype=dtype, device=dev)
    gt = torch.zeros(B2, H, NT, 2, 32, 4, 4, dtype=dtype, device=dev)
    plain = torch.zeros(M, C, dtype=dtype, device=dev)
    tk = dict(inner=N, s_o=H * NT * 1024, s_h=NT * 1024)
    tiles = [_lib.make_tile(q, kind=_lib.FFK_TILE_ACC, scale=0.25, **tk),
             _lib.make_tile(k, kind=_lib.FFK_TILE_QK, **tk),
             _lib.make_tile(v, kind=_lib.FFK_TILE_V, **tk),
             _lib.make_tile(gt, kind=_lib.FFK_TILE_ACC, bias=bias_g, act=_lib.FFK_ACT_SIGMOID, **tk),
             _lib.make_tile(plain, bias=bias_r, act=_lib.FFK_ACT_RELU, inner=M, s_i=C)]
    bias_all = torch.zeros(5 * 128, dtype=dtype, device=dev)
    bias_all[3 * 128:4 * 128] = bias_g
    bias_all[4 * 128:] = bias_r
    tiles[3].bias = bias_all.data_ptr() + 3 * 128 * 2
    tiles[4].bias = bias_all.data_ptr() + 4 * 128 * 2
    _lib.fused_linear(x, torch.cat(ws_).contiguous(), tiles, M=M, K=K, ln=(gam, bet))
    xn = _np(torch.from_numpy(ops_np.layer_norm(_np(x), _np(gam), _np(bet))).to(torch.bfloat16))
    lin = [ops_np.linear(xn, _np(w)) for w in ws_]
    heads = lambda y: y.reshape(B2, N, H, 32).transpose(0, 2, 1, 3)
    assert _rel(_np(layouts.untile_rows_acc(q, N)), heads(lin[0] * 0.25)) < TOL[dtype]
    assert _rel(_np(layouts.untile_qk(k, N)), heads(lin[1])) < TOL[dtype]
    assert _rel(_np(layouts.untile_v(v, N)), heads(lin[2])) < TOL[dtype]
    assert _rel(_np(layouts.untile_rows_acc(gt, N)), heads(_sig(lin[3] + _np(bias_g)))) < TOL[dtype]
    assert _rel(_np(plain).reshape(B2, N, C), np.maximum(lin[4] + _np(bias_r), 0)) < TOL[dtype]


def test_weights_stationary_matches_other_variant(dev):
    """GLU + row mask, channel-major store, both traversal orders, at a multi-slab size: the
    weights-stationary kernel and the LDS-staged kernel must agree to bf16 rounding."""
    from fastfold_amd import _lib
    dtype = torch.bfloat16
    r, C, Ch = 200, 128, 128
    g = torch.Generator().manual_seed(5)
    z = torch.randn(r, r, C, generator=g).to(dev, dtype)
    wpk = (torch.randn(2 * Ch + 128, C, generator=g) / C ** 0.5).to(dev, dtype)
    bpk = torch.randn(2 * Ch + 128, generator=g).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    mask = (torch.rand(r, r, generator=g) > 0.2).to(dev, dtype)
    outs = []
    for no_ws in (False, True):
        res = []
        for transposed in (False, True):
            out = torch.zeros(Ch, r, r, dtype=dtype, device=dev)
            gate = torch.zeros(r * r, C, dtype=dtype, device=dev)
            tiles = []
            for t in range(Ch // 64):
                tiles.append(_lib.make_tile(out.data_ptr() + t * 64 * r * r * 2, bias=bpk.data_ptr() + t * 128 * 2,
                                            glu=1, ncols=64, inner=r, s_o=r, s_i=1, s_h=32 * r * r, s_d=r * r,
                                            rowmask=mask, m_so=(1 if transposed else r), m_si=(r if transposed else 1)))
            kw = dict(inner=r, s_o=C, s_i=r * C) if transposed else dict(inner=r * r, s_i=C)
            tiles.append(_lib.make_tile(gate, bias=bpk.data_ptr() + 2 * 128 * 2, act=_lib.FFK_ACT_SIGMOID, **kw))
            akw = dict(a_inner=r, a_so=C, a_si=r * C) if transposed else {}
            _lib.fused_linear(z, wpk, tiles, M=r * r, K=C, ln=(gam, bet), staged=no_ws, **akw)
            res += [out, gate]
        outs.append(res)
    for a, b in zip(*outs):
        assert float(a.float().abs().max()) > 0.1
        assert _rel(_np(a), _np(b)) < 1e-2


@pytest.mark.parametrize("r,H,C", [(45, 4, 128), (64, 8, 128), (96, 4, 128), (45, 4, 64), (64, 4, 64)])
def test_pair_bias_kernel(dev, r, H, C):
    """ffk_pair_bias (bf16): LayerNorm + H-row projection written as attention bias tiles, in both
    traversal orders, against float64 numpy."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(r + H)
    z = (torch.randn(r, r, C, generator=g) * 1.5 + 0.4).to(dev, dtype)
    wb = (torch.randn(H, C, generator=g) / C ** 0.5).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    T = layouts.n_tiles(r)
    scratch = torch.empty(16 * C + 16, dtype=torch.float32, device=dev)
    for transposed in (False, True):
        bt = torch.zeros(H, T, T, 2, 32, 16, dtype=dtype, device=dev)
        kw = dict(a_inner=r, a_so=C, a_si=r * C) if transposed else dict(a_inner=r * r, a_so=0, a_si=C)
        _lib.pair_bias(bt, z, gam, bet, wb, scratch, N=r, C=C, H=H, scale=_lib.LOG2E, **kw)
        zz = _np(z).transpose(1, 0, 2) if transposed else _np(z)
        x = ops_np.layer_norm(zz, _np(gam), _np(bet))
        ref = (ops_np.linear(x, _np(wb)) * _lib.LOG2E).transpose(2, 0, 1)       # [h, q, k]
        assert _rel(_np(layouts.untile_bias(bt, r, r)), ref) < TOL[dtype]
        # a later call may reuse the weight operand the first one left in scratch (w = None)
        bt2 = torch.zeros_like(bt)
        _lib.pair_bias(bt2, z, None, None, None, scratch, N=r, C=C, H=H, scale=_lib.LOG2E, **kw)
        assert torch.equal(bt2, bt)
        # padding of ragged tiles is left untouched (zero)
        full = _np(layouts.untile_bias(bt, T * 32, T * 32))
        assert np.abs(full[:, r:, :]).max(initial=0.0) == 0.0 and np.abs(full[:, :, r:]).max(initial=0.0) == 0.0


@pytest.mark.parametrize("r,s", [(64, 128), (96, 64)])
def test_opm_fused_kernel(dev, r, s):
    """ffk_opm_fused against float64 numpy: out = resid + (sum_{d,e} (a_i^T b_j)[d,e] W[c,d,e] + bias) / (norm + eps)."""
    from fastfold_amd import _lib
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(r + s)
    a_t = (torch.randn(r * 32, s, generator=g) * 0.5).to(dev, dtype)       # row i*32 + d, K = sequences
    b_t = (torch.randn(r * 32, s, generator=g) * 0.5).to(dev, dtype)
    w = (torch.randn(128, 32, 32, generator=g) / 32).to(dev, dtype)         # [c, d, e] as in the reference weight
    bias = torch.randn(128, generator=g).to(dev, dtype)
    norm = (torch.rand(r, r, generator=g) * s + 1).to(dev)
    resid = torch.randn(r * r, 128, generator=g).to(dev, dtype)
    out = torch.empty_like(resid)
    w_ed = w.transpose(1, 2).reshape(128, 1024).contiguous()
    _lib.opm_fused(out, resid, a_t, b_t, w_ed, bias, norm, r=r, spad=s, eps=1e-3)
    A = _np(a_t).reshape(r, 32, s)
    B = _np(b_t).reshape(r, 32, s)
    O = np.einsum("ids,jes->ijde", A, B)
    O = _np(torch.from_numpy(O).to(torch.bfloat16))                         # the kernel rounds the outer product to bf16
    upd = (np.einsum("ijde,cde->ijc", O, _np(w)) + _np(bias)) / (_np(norm)[..., None] + 1e-3)
    got = _np(out).reshape(r, r, 128) - _np(resid).reshape(r, r, 128)
    assert _rel(got, upd) < TOL[dtype]
    # in place
    res2 = resid.clone()
    _lib.opm_fused(res2, res2, a_t, b_t, w_ed, bias, norm, r=r, spad=s, eps=1e-3)
    assert torch.equal(res2, out)
    with pytest.raises(RuntimeError):
        _lib.opm_fused(out, resid, a_t, b_t, w_ed, bias, norm, r=r + 8, spad=s, eps=1e-3)


@pytest.mark.parametrize("C", [128, 256])
@pytest.mark.parametrize("M", [256, 1000, 70000])
def test_transition_fused_kernel(dev, M, C):
    """ffk_transition_fused (pair width 128, MSA width 256) against float64 numpy, including a ragged last workgroup
    and in-place use."""
    from fastfold_amd import _lib
    dtype = torch.bfloat16
    Hd = 4 * C
    g = torch.Generator().manual_seed(M + C)
    x = (torch.randn(M, C, generator=g) * 1.5 + 0.2).to(dev, dtype)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dtype)
    w1 = (torch.randn(Hd, C, generator=g) / C ** 0.5).to(dev, dtype)
    b1 = torch.randn(Hd, generator=g).to(dev, dtype)
    w2 = (torch.randn(C, Hd, generator=g) / Hd ** 0.5).to(dev, dtype)
    b2 = torch.randn(C, generator=g).to(dev, dtype)
    out = torch.full_like(x, 7.0)
    _lib.transition_fused(out, x, gam, bet, w1, b1, w2, b2, M=M, C=C, hidden=Hd)
    xn = _np(torch.from_numpy(ops_np.layer_norm(_np(x), _np(gam), _np(bet))).to(torch.bfloat16))
    h = np.maximum(ops_np.linear(xn, _np(w1), _np(b1)), 0)
    h = _np(torch.from_numpy(h).to(torch.bfloat16))                         # hidden is rounded to bf16 on chip
    upd = ops_np.linear(h, _np(w2), _np(b2))
    assert _rel(_np(out) - _np(x), upd) < TOL[dtype]
    x2 = x.clone()
    _lib.transition_fused(x2, x2, gam, bet, w1, b1, w2, b2, M=M, C=C, hidden=Hd)
    assert torch.equal(x2, out)
    with pytest.raises(RuntimeError):
        _lib.transition_fused(out, x, gam, bet, w1, b1, w2, b2, M=M, C=64, hidden=256)
    with pytest.raises(RuntimeError):
        _lib.transition_fused(out, x, gam, bet, w1, b1, w2, b2, M=M, C=C, hidden=2 * C)


@pytest.mark.parametrize("r", [64, 104])
def test_fused_linear_second_operand(dev, r):
    """GLU tiles whose gate halves come from a second operand (the output stage of the triangle multiplication):
    out = resid + (W_p LN2(p) + b_p) * sigmoid(W_g LN1(z) + b_g), p channel-major, both LayerNorms folded into
    the packed weights (statistics taken from the operand fragments inside the kernel)."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn import _fused as F_
    dtype = torch.bfloat16
    C, M = 128, r * r
    g = torch.Generator().manual_seed(r)
    p_cm = (torch.randn(C, r, r, generator=g) * 2 + 0.3).to(dev, dtype)            # [c, i, j]
    z = (torch.randn(M, C, generator=g) * 1.5 - 0.2).to(dev, dtype)
    gam1, gam2 = ((1 + 0.1 * torch.randn(C, generator=g)).to(dev, dtype) for _ in range(2))
    bet1, bet2 = ((0.1 * torch.randn(C, generator=g)).to(dev, dtype) for _ in range(2))
    wp, wg = ((torch.randn(C, C, generator=g) / C ** 0.5).to(dev, dtype) for _ in range(2))
    bp, bg = (torch.randn(C, generator=g).to(dev, dtype) for _ in range(2))
    w_pk, b_pk, rowsums = F_.pack_trimul_out(wp, bp, wg, bg, C, dtype, dev, ln_p=(gam2, bet2), ln_z=(gam1, bet1))
    out = torch.empty(M, C, device=dev, dtype=dtype)
    tiles = [_lib.make_tile(out.data_ptr() + t * 64 * 2, bias=b_pk.data_ptr() + t * 128 * 2, glu=1, ncols=64,
                            resid=z.data_ptr() + t * 64 * 2, inner=M, s_i=C) for t in range(2)]
    kw = dict(M=M, K=C, a_inner=r, a_so=r, a_si=1, a_chanmajor=True, a_cs=r * r, ln_rowsums=rowsums, a2_inner=M, a2_si=C)
    _lib.fused_linear(p_cm, w_pk, tiles, a2=z, **kw)
    pn = ops_np.layer_norm(_np(p_cm).reshape(C, M).T, _np(gam2), _np(bet2))
    zn = ops_np.layer_norm(_np(z), _np(gam1), _np(bet1))
    upd = ops_np.linear(pn, _np(wp), _np(bp)) / (1 + np.exp(-ops_np.linear(zn, _np(wg), _np(bg))))
    assert _rel(_np(out) - _np(z), upd) < TOL[dtype]
    # in place on the second operand / residual
    z2 = z.clone()
    tiles = [_lib.make_tile(z2.data_ptr() + t * 64 * 2, bias=b_pk.data_ptr() + t * 128 * 2, glu=1, ncols=64,
                            resid=z2.data_ptr() + t * 64 * 2, inner=M, s_i=C) for t in range(2)]
    _lib.fused_linear(p_cm, w_pk, tiles, a2=z2, **kw)
    assert torch.equal(z2, out)
    # rows with a large common offset: the folded form subtracts mean * rowsum after the product
    p_off = (p_cm.float() + 40.0).to(dtype)
    out3 = torch.empty_like(out)
    tiles3 = [_lib.make_tile(out3.data_ptr() + t * 64 * 2, bias=b_pk.data_ptr() + t * 128 * 2, glu=1, ncols=64,
                             resid=z.data_ptr() + t * 64 * 2, inner=M, s_i=C) for t in range(2)]
    _lib.fused_linear(p_off, w_pk, tiles3, a2=z, **kw)
    pn = ops_np.layer_norm(_np(p_off).reshape(C, M).T, _np(gam2), _np(bet2))
    upd = ops_np.linear(pn, _np(wp), _np(bp)) / (1 + np.exp(-ops_np.linear(zn, _np(wg), _np(bg))))
    assert _rel(_np(out3) - _np(z), upd) < TOL[dtype]
    # a second operand without the shapes it is built for, or without folded LayerNorms, is refused, not ignored
    with pytest.raises(RuntimeError):
        _lib.fused_linear(z, w_pk, tiles, M=M, K=C, ln_rowsums=rowsums, a2=z, a2_inner=M, a2_si=C)
    with pytest.raises(RuntimeError):
        _lib.fused_linear(p_cm, w_pk, tiles, M=M, K=C, a_inner=r, a_so=r, a_si=1, a_chanmajor=True, a_cs=r * r,
                          ln=(gam2, bet2), a2=z, a2_inner=M, a2_si=C)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K,N,P", [(64, 64, 37), (128, 128, 16)])
def test_periodic_gate_rows(dev, dtype, K, N, P):
    """gate_rows = P: logical row m is multiplied by gate row m % P (one multiplier row per column of an
    [S, P] grid of rows, as the global column attention uses it)."""
    from fastfold_amd import _lib
    S = 9
    M = S * P
    g = torch.Generator().manual_seed(K + P)
    a = torch.randn(M, K, generator=g).to(dev, dtype)
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(dev, dtype)
    b = torch.randn(N, generator=g).to(dev, dtype)
    gate = torch.randn(P, N, generator=g).to(dev, dtype)
    out = torch.empty(M, N, dtype=dtype, device=dev)
    bp = torch.zeros(128, dtype=dtype, device=dev)
    bp[:N] = b
    tiles = [_lib.make_tile(out, bias=bp, gate=gate, gate_ld=N, gate_rows=P, inner=M, s_i=N, ncols=N,
                            act=_lib.FFK_ACT_SIGMOID)]
    _lib.fused_linear(a, _pack(w, 1), tiles, M=M, K=K)
    y = 1.0 / (1.0 + np.exp(-ops_np.linear(_np(a), _np(w), _np(b))))
    ref = y.reshape(S, P, N) * _np(gate)[None]
    assert _rel(_np(out).reshape(S, P, N), ref) < TOL[dtype]
