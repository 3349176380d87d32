"""GPU parity of the flash attention core and the batched NT GEMM (through the C ABI)
against the float64 numpy oracle."""
import math

import numpy as np
import pytest
import torch

from oracle import ops_np

pytestmark = pytest.mark.gpu

LOG2E = 1.4426950408889634


def _np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def _rel(got, ref):
    return np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-6)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("B2,H,N,use_bias,use_gate", [(3, 4, 70, True, True), (2, 8, 32, False, False),
                                                      (1, 4, 257, True, False), (5, 2, 129, False, True),
                                                      (2, 4, 300, True, True)])
def test_attention_core(dev, dtype, tol, B2, H, N, use_bias, use_gate):
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    g = torch.Generator().manual_seed(N + H)
    q, k, v = (torch.randn(1, B2, H, N, 32, generator=g).to(dev, dtype) for _ in range(3))
    bias = (2 * torch.randn(1, H, N, N, generator=g)).to(dev, dtype) if use_bias else None
    mask = (torch.rand(1, B2, N, generator=g) > 0.2).to(dev, dtype)
    mask[..., 1] = 1
    gate = torch.rand(B2 * N, H * 32, generator=g).to(dev, dtype) if use_gate else None
    scale = LOG2E / math.sqrt(32)
    qs = (q.float() * scale).to(dtype)       # what the projection epilogue would have written
    qt, kt, vt = layouts.tile_qk(qs[0]), layouts.tile_qk(k[0]), layouts.tile_v(v[0])
    bt = layouts.tile_bias((bias[0].float() * LOG2E).to(dtype)) if use_bias else None
    NT = layouts.n_tiles(N)
    kb = torch.empty(B2, NT * 32, dtype=torch.float32, device=dev)
    fl = torch.empty(B2, NT, dtype=torch.int32, device=dev)
    _lib.key_bias(kb, fl, mask[0], B=B2, N=N, mask_sb=N, mask_sn=1)
    assert float(kb[:, :N][mask[0] != 0].abs().max()) == 0.0 and float(kb[:, :N][mask[0] == 0].max()) < -1e9
    bad = torch.nn.functional.pad(mask[0].float(), (0, NT * 32 - N)).view(B2, NT, 32) == 0
    want = torch.where(bad.all(-1), 2, torch.where(bad.any(-1), 1, 0)).to(torch.int32)
    assert torch.equal(fl, want)
    out = torch.empty(B2 * N, H * 32, dtype=dtype, device=dev)
    _lib.attention_fwd(out, qt, kt, vt, bt, kb, fl, gate, B2=B2, H=H, Nq=N, Nk=N)
    # oracle on exactly the operands the kernel saw (q rounded after scaling, bias rounded after log2e)
    q_eff = _np(qs) / scale * math.sqrt(32) / math.sqrt(32)
    b_eff = _np((bias[0].float() * LOG2E).to(dtype))[None] / LOG2E if use_bias else None
    ref = ops_np.attention_core(q_eff, _np(k), _np(v), _np(mask), b_eff)[0]          # [B2, N, H*32]
    if use_gate:
        ref = ref * _np(gate).reshape(B2, N, H * 32)
    assert _rel(_np(out).reshape(B2, N, H * 32), ref) < tol
    if use_gate:     # the same gate handed over in accumulator-tile order gives the same bits
        gate_t = layouts.tile_rows_acc(gate.view(B2, N, H, 32).permute(0, 2, 1, 3))
        out2 = torch.empty_like(out)
        _lib.attention_fwd(out2, qt, kt, vt, bt, kb, fl, gate_t, B2=B2, H=H, Nq=N, Nk=N, gate_tiled=True)
        assert torch.equal(out, out2)
    if use_bias:     # the same bias with one unused tile after every query-tile row gives the same bits
        bp = torch.full((H, NT, NT + 1, 1024), float("nan"), dtype=dtype, device=dev)
        bp[:, :, :NT] = bt.reshape(H, NT, NT, 1024)
        out3 = torch.empty_like(out)
        _lib.attention_fwd(out3, qt, kt, vt, bp, kb, fl, gate, B2=B2, H=H, Nq=N, Nk=N, bias_padded=True)
        assert torch.equal(out, out3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("use_bias", [False, True])
def test_attention_half_k_flag(dev, dtype, use_bias):
    """Heads of 8 channels zero-padded to 32 (FFK_TILE_QK order: channels 8 .. 15 and 24 .. 31 are elements 8 .. 15 of a
    lane's sixteen): with FFK_ATT_HALF_K the kernel skips the second half of the score product and gives the same bits."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    B2, H, N = 3, 4, 100
    g = torch.Generator().manual_seed(11)
    q, k, v = (torch.randn(B2, H, N, 32, generator=g).to(dev, dtype) for _ in range(3))
    q[..., 8:] = 0
    k[..., 8:] = 0
    bt = layouts.tile_bias(torch.randn(H, N, N, generator=g).to(dev, dtype)) if use_bias else None
    kb = torch.empty(B2, 128, dtype=torch.float32, device=dev)
    fl = torch.empty(B2, 4, dtype=torch.int32, device=dev)
    _lib.key_bias(kb, fl, None, B=B2, N=N)
    outs = []
    for half_k in (False, True):
        out = torch.empty(B2 * N, H * 32, dtype=dtype, device=dev)
        _lib.attention_fwd(out, layouts.tile_qk(q), layouts.tile_qk(k), layouts.tile_v(v), bt, kb, fl, None,
                           B2=B2, H=H, Nq=N, Nk=N, half_k=half_k)
        outs.append(out)
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_attention_tiling_invariance_and_masked_keys(dev, dtype, tol):
    """Changing K/V at masked keys must not change the output; all-valid mask == no mask."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    B2, H, N = 2, 4, 100
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(B2, H, N, 32, generator=g).to(dev, dtype) for _ in range(3))
    mask = torch.ones(B2, N, device=dev, dtype=dtype)
    mask[:, 90:] = 0
    kb = torch.empty(B2, 128, dtype=torch.float32, device=dev)
    fl = torch.empty(B2, 4, dtype=torch.int32, device=dev)
    _lib.key_bias(kb, fl, mask, B=B2, N=N, mask_sb=N, mask_sn=1)
    outs = []
    for delta in (0.0, 5.0):
        k2, v2 = k.clone(), v.clone()
        k2[:, :, 90:] += delta
        v2[:, :, 90:] -= delta
        out = torch.empty(B2 * N, H * 32, dtype=dtype, device=dev)
        _lib.attention_fwd(out, layouts.tile_qk(q), layouts.tile_qk(k2), layouts.tile_v(v2), None, kb, fl, None,
                           B2=B2, H=H, Nq=N, Nk=N)
        outs.append(_np(out))
    assert np.abs(outs[0] - outs[1]).max() == 0.0
    # same as attending over the first 90 keys only
    kb90 = torch.empty(B2, 96, dtype=torch.float32, device=dev)
    fl90 = torch.empty(B2, 3, dtype=torch.int32, device=dev)
    _lib.key_bias(kb90, fl90, None, B=B2, N=90)
    out = torch.empty(B2 * N, H * 32, dtype=dtype, device=dev)
    _lib.attention_fwd(out, layouts.tile_qk(q), layouts.tile_qk(k[:, :, :90].contiguous()),
                       layouts.tile_v(v[:, :, :90].contiguous()), None, kb90, fl90, None, B2=B2, H=H, Nq=N, Nk=90)
    assert _rel(_np(out), outs[0]) < tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("slope", [0.05, 0.6, 5.0])
def test_attention_moving_reference(dev, dtype, tol, slope):
    """Scores that climb (or fall) steadily along the keys: the kernel's running reference has to move
    several times, by a little (slope 0.05), by more than its slack per tile (0.6) and by more than the
    fp32 exponent range per tile (5.0: exp2 overflows before the move).  Half of the queries see the
    keys in descending order, so only part of a wave asks for the move."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    B2, H, N = 2, 4, 200
    g = torch.Generator().manual_seed(int(slope * 100))
    u = torch.nn.functional.normalize(torch.randn(H, 32, generator=g), dim=-1)          # one direction per head
    ramp = torch.arange(N, dtype=torch.float32) * slope                                   # score of key j ~ +-ramp[j]
    sign = torch.where(torch.arange(N) % 2 == 0, 1.0, -1.0)
    q = (sign[None, None, :, None] * u[None, :, None, :] + 0.05 * torch.randn(B2, H, N, 32, generator=g)).to(dev, dtype)
    k = (ramp[None, None, :, None] * u[None, :, None, :] + 0.05 * torch.randn(B2, H, N, 32, generator=g)).to(dev, dtype)
    v = torch.randn(B2, H, N, 32, generator=g).to(dev, dtype)
    mask = torch.ones(B2, N, device=dev, dtype=dtype)
    mask[1, 150:] = 0
    NT = layouts.n_tiles(N)
    kb = torch.empty(B2, NT * 32, dtype=torch.float32, device=dev)
    fl = torch.empty(B2, NT, dtype=torch.int32, device=dev)
    _lib.key_bias(kb, fl, mask, B=B2, N=N, mask_sb=N, mask_sn=1)
    out = torch.empty(B2 * N, H * 32, dtype=dtype, device=dev)
    # q is handed over unscaled: logits are q.k in log2 units, i.e. ln2 * q.k for the oracle
    _lib.attention_fwd(out, layouts.tile_qk(q), layouts.tile_qk(k), layouts.tile_v(v), None, kb, fl, None,
                       B2=B2, H=H, Nq=N, Nk=N)
    ref = ops_np.attention_core(_np(q)[None] * math.log(2.0) * math.sqrt(32), _np(k)[None], _np(v)[None], _np(mask)[None], None)[0]
    got = _np(out).reshape(B2, N, H * 32)
    assert np.isfinite(got).all()
    assert _rel(got, ref) < tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("r", [52, 128, 200])
def test_bgemm_trimul_contraction(dev, dtype, tol, r):
    """p[c,i,j] = sum_k l[c,i,k] r[c,j,k] on channel-major, K-padded operands."""
    from fastfold_amd import _lib
    C = 16
    kpad = (r + 7) // 8 * 8
    g = torch.Generator().manual_seed(r)
    left = torch.zeros(C, r, kpad, dtype=dtype, device=dev)
    right = torch.zeros(C, r, kpad, dtype=dtype, device=dev)
    left[:, :, :r] = torch.randn(C, r, r, generator=g).to(dev, dtype)
    right[:, :, :r] = torch.randn(C, r, r, generator=g).to(dev, dtype)
    out = torch.zeros(C, r, kpad, dtype=dtype, device=dev)
    _lib.bgemm_nt(left, right, out, M=r, N=r, K=kpad, lda=kpad, ldb=kpad, batch=C, a_bs=r * kpad, b_bs=r * kpad,
                  o_bs=r * kpad, s_i=kpad)
    a = _np(left)[:, :, :r].transpose(1, 2, 0)      # [i, k, c]
    b = _np(right)[:, :, :r].transpose(1, 2, 0)     # [j, k, c]
    ref = ops_np.trimul_outgoing(a, b)              # [i, j, c]
    assert _rel(_np(out)[:, :, :r].transpose(1, 2, 0), ref) < tol


@pytest.mark.parametrize("C,M,N,K", [
    (3, 256, 256, 96),       # exactly the three chunks the ring is primed with
    (2, 300, 528, 160),      # ragged tiles in both directions, an odd number of chunks
    (9, 512, 256, 128),      # XCD-contiguous tile order (batch >= 8), 256 x 128 tiles
    (40, 768, 768, 128),     # 360 full 256 x 256 tiles on 256 workgroups: a second tile behind a full one
    (40, 700, 656, 96),      # ... and behind ragged ones
])
def test_bgemm_large_tiles(dev, C, M, N, K):
    """The persistent large-tile kernel (M >= 256, bf16): its chunk pipeline runs on across tiles, and the wait
    counts right after a tile depend on whether that tile stored every row."""
    from fastfold_amd import _lib
    g = torch.Generator().manual_seed(C * M + N + K)
    a = torch.randn(C, M, K, generator=g).to(dev, torch.bfloat16)
    b = torch.randn(C, N, K, generator=g).to(dev, torch.bfloat16)
    out = torch.full((C, M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    _lib.bgemm_nt(a, b, out, M=M, N=N, K=K, lda=K, ldb=K, batch=C, a_bs=M * K, b_bs=N * K, o_bs=M * N, scale=0.125)
    ref = 0.125 * np.einsum("cmk,cnk->cmn", _np(a).astype(np.float32), _np(b).astype(np.float32))
    got = _np(out)
    assert np.isfinite(got).all()
    assert _rel(got, ref) < 4e-3
    assert np.abs(got - ref).max() < 2e-2 * np.abs(ref).max()


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("s,r", [(24, 10), (128, 9), (50, 33)])
def test_bgemm_outer_product_and_projection(dev, dtype, tol, s, r):
    """OPM: O[(i,j),(d,e)] = sum_s a[s,i,d] b[s,j,e] from K-padded transposed operands, then
    z + (O Wo^T + bo) / (norm + eps) with an fp32 normaliser."""
    from fastfold_amd import _lib
    spad = (s + 7) // 8 * 8
    g = torch.Generator().manual_seed(s + r)
    a = torch.randn(s, r, 32, generator=g).to(dev, dtype)
    b = torch.randn(s, r, 32, generator=g).to(dev, dtype)
    aT = torch.zeros(r * 32, spad, dtype=dtype, device=dev)
    bT = torch.zeros(r * 32, spad, dtype=dtype, device=dev)
    aT[:, :s] = a.permute(1, 2, 0).reshape(r * 32, s)
    bT[:, :s] = b.permute(1, 2, 0).reshape(r * 32, s)
    O = torch.zeros(r * r, 1024, dtype=dtype, device=dev)
    _lib.bgemm_nt(aT, bT, O, M=32 * r, N=32 * r, K=spad, lda=spad, ldb=spad, inner=32, s_o=r * 1024, s_i=32,
                  s_h=1024, s_d=1)
    ref_o = ops_np.outer_product(_np(a), _np(b)).reshape(r * r, 1024)
    assert _rel(_np(O), ref_o) < tol
    wo = (torch.randn(128, 1024, generator=g) / 32).to(dev, dtype)
    bo = torch.randn(128, generator=g).to(dev, dtype)
    norm = (torch.rand(r * r, generator=g) * s).to(dev)
    z = torch.randn(r * r, 128, generator=g).to(dev, dtype)
    z0 = z.clone()
    _lib.bgemm_nt(O, wo, z, M=r * r, N=128, K=1024, lda=1024, ldb=1024, bias=bo, resid=z, rowdiv=norm, div_eps=1e-3)
    ref = _np(z0) + ops_np.linear(_np(O), _np(wo), _np(bo)) / (_np(norm)[:, None] + 1e-3)
    assert _rel(_np(z), ref) < tol
    # fp32 output of a bf16 product (mask normaliser): exact small integers
    mk = (torch.rand(r, spad, generator=g) > 0.3).to(dev, dtype)
    mk[:, s:] = 0
    nrm = torch.empty(r, r, dtype=torch.float32, device=dev)
    _lib.bgemm_nt(mk, mk, nrm, M=r, N=r, K=spad, lda=spad, ldb=spad, out_f32=True)
    assert np.array_equal(_np(nrm), _np(mk) @ _np(mk).T)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("b1,b2,h,n", [(1, 3, 4, 77), (2, 2, 8, 64)])
def test_fused_attention_core_op(dev, dtype, tol, b1, b2, h, n):
    """The exported op against the textbook formula the reference tests it with
    (tests/test_fastnn/test_attention_core.py:16-31)."""
    from fastfold_amd.model.fastnn.kernel import fused_attention_core
    g = torch.Generator().manual_seed(b2 * n)
    q, k, v = (torch.randn(b1, b2, h, n, 32, generator=g).to(dev, dtype) for _ in range(3))
    bias = torch.randn(b1, h, n, n, generator=g).to(dev, dtype)
    mask = (torch.rand(b1, b2, n, generator=g) > 0.25).to(dev, dtype)
    mask[..., 0] = 1
    out = fused_attention_core(q, k, v, mask, bias)
    assert out.shape == (b1, b2, n, h * 32) and out.dtype == dtype
    ref = ops_np.attention_core(_np(q), _np(k), _np(v), _np(mask), _np(bias))
    assert _rel(_np(out), ref) < tol
    # narrower heads run zero-padded (8 and 16: the widths of the extra-MSA and template stacks)
    for d in (16, 8):
        qd, kd, vd = (t[..., :d].contiguous() for t in (q, k, v))
        outd = fused_attention_core(qd, kd, vd, mask, bias)
        assert outd.shape == (b1, b2, n, h * d)
        assert _rel(_np(outd), ops_np.attention_core(_np(qd), _np(kd), _np(vd), _np(mask), _np(bias))) < tol
    # 64 / 128: the other widths the reference's Triton kernel takes (kernel/triton/attention_core.py:142)
    for d in (64, 128):
        qd, kd, vd = (torch.randn(b1, b2, h, n, d, generator=g).to(dev, dtype) for _ in range(3))
        outd = fused_attention_core(qd, kd, vd, mask, bias)
        assert outd.shape == (b1, b2, n, h * d) and outd.dtype == dtype
        assert _rel(_np(outd), ops_np.attention_core(_np(qd), _np(kd), _np(vd), _np(mask), _np(bias))) < tol, d
        # without bias, and as strided views of a fused projection
        qkv = torch.randn(b1, b2, n, 3 * h * d, generator=g).to(dev, dtype)
        qs, ks, vs = (t.unflatten(-1, (h, d)).transpose(-2, -3) for t in qkv.chunk(3, dim=-1))
        outs = fused_attention_core(qs, ks, vs, mask, None)
        zero_bias = torch.zeros(b1, h, n, n)
        assert _rel(_np(outs), ops_np.attention_core(_np(qs), _np(ks), _np(vs), _np(mask), zero_bias.numpy())) < tol, d
    with pytest.raises(RuntimeError, match="not supported"):
        fused_attention_core(q[..., :24], k[..., :24], v[..., :24], mask, bias)
    with pytest.raises(RuntimeError, match="bfloat16 or float32"):       # fp16 is refused before anything is launched
        fused_attention_core(q.half(), k.half(), v.half(), mask.half(), bias.half())
    with pytest.raises(RuntimeError):
        fused_attention_core(q.cpu(), k.cpu(), v.cpu(), mask.cpu(), bias.cpu())


@pytest.mark.parametrize("n", [32, 256, 370, 512])
@pytest.mark.parametrize("d", [32, 64, 128])
def test_fused_attention_core_reference_shapes(dev, n, d):
    """Shapes of the reference's own test of the operator (tests/test_fastnn/test_attention_core.py:36-44: batch 1,
    chunk 8, 4 heads, std-0.5 operands, a random 0/1 key mask, sequence lengths from its list), bf16, against the
    float64 formula."""
    from fastfold_amd.model.fastnn.kernel import fused_attention_core
    g = torch.Generator().manual_seed(n + d)
    q, k, v = (0.5 * torch.randn(1, 8, 4, n, d, generator=g) for _ in range(3))
    q, k, v = (t.to(dev, torch.bfloat16) for t in (q, k, v))
    mask = (torch.randn(1, 8, n, generator=g) > 0).to(dev, torch.bfloat16)
    mask[..., 0] = 1
    bias = torch.randn(1, 4, n, n, generator=g).to(dev, torch.bfloat16)
    out = fused_attention_core(q, k, v, mask, bias)
    ref = ops_np.attention_core(_np(q), _np(k), _np(v), _np(mask), _np(bias))
    assert _rel(_np(out), ref) < 2e-2


def _torch_attention_core(q, k, v, mask, bias):
    """The reference's formula (fastfold/model/fastnn/kernel/attention_core.py:17-31) in float64, differentiable."""
    logits = torch.matmul(q / math.sqrt(q.shape[-1]), k.transpose(-1, -2))
    if bias is not None:
        logits = logits + bias[:, None]
    logits = logits + (1e9 * (mask - 1))[:, :, None, None, :]
    w = torch.softmax(logits, -1)
    o = torch.matmul(w, v)                                    # [b1, b2, h, n, d]
    return o.permute(0, 1, 3, 2, 4).reshape(o.shape[0], o.shape[1], o.shape[3], -1)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("b1,b2,h,n,d,use_bias", [(1, 3, 4, 77, 32, True), (2, 2, 8, 64, 32, True), (1, 2, 4, 130, 32, False),
                                                  (1, 2, 4, 50, 16, True), (1, 3, 8, 40, 8, True),
                                                  (1, 43, 4, 70, 32, True),       # several batch-row slices in the dbias kernel
                                                  (1, 3, 4, 77, 64, True), (2, 2, 4, 64, 128, True), (1, 2, 4, 45, 128, False),
                                                  (1, 19, 4, 70, 64, True)])
def test_fused_attention_core_backward(dev, dtype, tol, b1, b2, h, n, d, use_bias):
    """dq, dk, dv, dbias of the exported op (``ffk_attention_bwd``: logits recomputed tile by tile) against torch
    autograd of the reference's formula in float64, with masked keys, a ragged last tile and the narrow heads."""
    from fastfold_amd.model.fastnn.kernel import fused_attention_core
    g = torch.Generator().manual_seed(b2 * n + d)
    q, k, v = (torch.randn(b1, b2, h, n, d, generator=g).to(dev, dtype).requires_grad_() for _ in range(3))
    bias = torch.randn(b1, h, n, n, generator=g).to(dev, dtype).requires_grad_() if use_bias else None
    mask = (torch.rand(b1, b2, n, generator=g) > 0.25).to(dev, dtype)
    mask[..., 0] = 1
    dout = torch.randn(b1, b2, n, h * d, generator=g).to(dev, dtype)
    out = fused_attention_core(q, k, v, mask, bias)
    out.backward(dout)
    refs = [t.detach().double().cpu().requires_grad_() for t in (q, k, v)]
    rbias = bias.detach().double().cpu().requires_grad_() if use_bias else None
    ro = _torch_attention_core(refs[0], refs[1], refs[2], mask.double().cpu(), rbias)
    ro.backward(dout.double().cpu())
    assert _rel(_np(out), ro.detach().numpy()) < tol
    for name, got, want in zip("qkv", (q, k, v), refs):
        assert got.grad is not None and got.grad.shape == got.shape and got.grad.dtype == dtype
        assert _rel(_np(got.grad), want.grad.numpy()) < tol, "d" + name
    if use_bias:
        assert bias.grad.shape == bias.shape
        assert _rel(_np(bias.grad), rbias.grad.numpy()) < tol, "dbias"
        # masked keys receive no gradient through k and v, and none reaches the bias at masked columns
        dead = (mask == 0)[:, :, None, :, None].expand_as(k)
        assert float(k.grad[dead].abs().max()) == 0.0 and float(v.grad[dead].abs().max()) == 0.0


def test_fused_attention_core_backward_fully_masked_rows(dev):
    """A batch row whose keys are all masked gives zero output in the forward pass and zero gradients here."""
    from fastfold_amd.model.fastnn.kernel import fused_attention_core
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(1, 2, 4, 40, 32, generator=g).to(dev).requires_grad_() for _ in range(3))
    mask = torch.ones(1, 2, 40, device=dev)
    mask[0, 1] = 0
    out = fused_attention_core(q, k, v, mask, None)
    out.backward(torch.ones_like(out))
    for t in (q, k, v):
        assert bool(torch.isfinite(t.grad).all()) and float(t.grad[0, 1].abs().max()) == 0.0
        assert float(t.grad[0, 0].abs().max()) > 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b2,h,n,d", [(3, 4, 70, 32), (2, 8, 33, 16), (1, 4, 128, 8), (5, 4, 31, 32)])
def test_tile_pack_matches_the_torch_layout_helpers(dev, dtype, b2, h, n, d):
    """ffk_tile_pack against the pad / view / permute formulation of the same tiles (layouts.tile_qk / tile_v), bit
    for bit, on a contiguous tensor and on the strided [b2, h, n, d] view of a fused [b2, n, 3 * h * d] projection."""
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel import layouts
    g = torch.Generator().manual_seed(n + d)
    qkv = torch.randn(b2, n, 3 * h * d, generator=g).to(dev, dtype)
    views = [t.unflatten(-1, (h, d)).transpose(-2, -3) for t in qkv.chunk(3, dim=-1)]     # not contiguous
    pad = torch.nn.functional.pad
    for x in views + [views[1].contiguous()]:
        x32 = pad(x, (0, 32 - d))
        for scale in (1.0, 0.255):
            ref = (x32.float() * scale).to(dtype) if scale != 1.0 else x32
            assert torch.equal(_lib.tile_pack(x, _lib.FFK_TILE_QK, scale).view(-1), layouts.tile_qk(ref).reshape(-1))
            assert torch.equal(_lib.tile_pack(x, _lib.FFK_TILE_V, scale).view(-1), layouts.tile_v(ref).reshape(-1))
