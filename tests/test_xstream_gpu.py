"""Extended residual stream (bf16 value + int8 tail = the fp32 bit pattern (h << 16) + (t << 8), include/ffk.h):
every kernel that adds an update to a residual tensor, in tail mode.

Three checks per kernel: a zero update leaves (value, tail) bit-identical; a known constant update (bias only,
zero weights) gives exactly round24(value + bias), computed here with integer arithmetic on the bit patterns; a
random update matches the float64 update to the tolerance of the bf16 products while the plain bf16 output of the
same launch is the tail-mode value rounded."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def xs_decode(h, t):
    """float32 value of a (bf16 tensor, int8 tensor) pair."""
    hw = h.view(torch.int16).cpu().numpy().astype(np.uint16).astype(np.uint32) << 16
    tw = (t.cpu().numpy().astype(np.int32) << 8).astype(np.uint32)
    return (hw + tw).view(np.float32)


def xs_round(x):
    """(bf16 bits as uint16, int8 tail) of float32 values: round to 24 bits, then split with the upper half rounded."""
    w24 = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) + np.uint32(0x80)
    h = ((w24 + np.uint32(0x8000)) >> 16).astype(np.uint16)
    t = ((w24 >> 8) & 0xFF).astype(np.uint8).view(np.int8)
    return h, t


def _stream(shape, dev, seed):
    """A random residual tensor with a random valid tail."""
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(shape, generator=g) * 3).float().numpy()
    h, t = xs_round(x)
    hv = torch.from_numpy(h.view(np.int16)).view(BF).to(dev)
    return hv, torch.from_numpy(t.copy()).to(dev)


def _bits(h, t):
    return h.view(torch.int16).cpu().numpy().astype(np.uint16), t.cpu().numpy()


def test_numpy_model_of_the_format():
    x = (np.random.RandomState(0).standard_normal(200000) * 10).astype(np.float32)
    h, t = xs_round(x)
    hv = torch.from_numpy(h.view(np.int16)).view(BF)
    back = xs_decode(hv, torch.from_numpy(t.copy()))
    assert np.abs(back - x).max() <= np.abs(x).max() * 2.0 ** -16
    assert np.abs(hv.float().numpy() - x).max() <= np.abs(x).max() * 2.0 ** -8      # h alone is x rounded to bf16
    h2, t2 = xs_round(back)                                                          # re-rounding is the identity
    assert np.array_equal(h2, h) and np.array_equal(t2, t)


def _linear_case(dev, M, K, N, seed, staged, zero_w, zero_b):
    from fastfold_amd import _lib
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).to(dev, BF)
    w = torch.zeros(128 * ((N + 127) // 128), K)
    if not zero_w:
        w[:N] = torch.randn(N, K, generator=g) / K ** 0.5
    w = w.to(dev, BF)
    b = torch.zeros(w.shape[0]) if zero_b else torch.randn(w.shape[0], generator=g)
    b = b.to(dev, BF)
    return _lib, a, w, b


@pytest.mark.parametrize("M,K,N,staged", [(1000, 128, 128, False), (520, 256, 256, False), (300, 128, 128, True),
                                          (77, 96, 64, False), (130, 64, 64, False)])
def test_fused_linear_residual_tail(dev, M, K, N, staged):
    """Output projection onto the stream: weights-stationary kernel (K = 128, 256), the LDS-staged kernels
    (forced, odd K, K = 64 with a tail)."""
    def run(zero_w, zero_b, tail):
        _lib, a, w, b = _linear_case(dev, M, K, N, 7, staged, zero_w, zero_b)
        h, t = _stream((M, N), dev, 11)
        h0, t0 = h.clone(), t.clone()
        tiles = [_lib.make_tile(h.data_ptr() + c * 128 * 2, bias=b.data_ptr() + c * 128 * 2, resid=h.data_ptr() + c * 128 * 2,
                                xtail=(t.data_ptr() + c * 128) if tail else None, inner=M, s_i=N,
                                ncols=min(128, N - c * 128)) for c in range((N + 127) // 128)]
        _lib.fused_linear(a, w, tiles, M=M, K=K, staged=staged)
        return a, w, b, h0, t0, h, t
    # zero update
    _, _, _, h0, t0, h, t = run(True, True, True)
    assert torch.equal(h, h0) and torch.equal(t, t0)
    # bias only: exact
    _, _, b, h0, t0, h, t = run(True, False, True)
    want = xs_decode(h0, t0) + b.float().cpu().numpy()[None, :N]
    hw, tw = xs_round(want)
    hb, tb = _bits(h, t)
    assert np.array_equal(hb, hw) and np.array_equal(tb, tw)
    # random update
    a, w, b, h0, t0, h, t = run(False, False, True)
    upd = a.double().cpu().numpy() @ w.double().cpu().numpy()[:N].T + b.double().cpu().numpy()[:N]
    got = xs_decode(h, t).astype(np.float64) - xs_decode(h0, t0).astype(np.float64)
    assert np.linalg.norm(got - upd) / np.linalg.norm(upd) < 6e-3
    # ... and the error of the sum is that of the update, not of a bf16 rounding of the sum
    err = np.abs(xs_decode(h, t).astype(np.float64) - (xs_decode(h0, t0).astype(np.float64) + upd))
    assert err.max() < 0.05 and np.sqrt((err ** 2).mean()) < 4e-3
    # the tail is ignored (and untouched) without the pointer
    _, _, _, h0, t0, hp, tp = run(False, False, False)
    assert torch.equal(tp, t0)
    assert np.abs(hp.float().cpu().numpy() - (h0.float().cpu().numpy() + upd)).max() < 0.1


@pytest.mark.parametrize("M,N,K", [(512, 128, 512), (96, 256, 1024), (300, 48, 64)])
def test_bgemm_residual_tail(dev, M, N, K):
    """Second linear of a transition / output projection of the outer product: large-tile and small-tile kernels."""
    from fastfold_amd import _lib
    g = torch.Generator().manual_seed(M + N)
    def run(zero_w, zero_b, tail):
        a = torch.randn(M, K, generator=g).to(dev, BF)
        w = (torch.zeros(N, K) if zero_w else torch.randn(N, K, generator=g) / K ** 0.5).to(dev, BF)
        b = (torch.zeros(N) if zero_b else torch.randn(N, generator=g)).to(dev, BF)
        h, t = _stream((M, N), dev, 5)
        h0, t0 = h.clone(), t.clone()
        _lib.bgemm_nt(a, w, h, M=M, N=N, K=K, lda=K, ldb=K, bias=b, resid=h, xtail=t if tail else None)
        return a, w, b, h0, t0, h, t
    _, _, _, h0, t0, h, t = run(True, True, True)
    assert torch.equal(h, h0) and torch.equal(t, t0)
    _, _, b, h0, t0, h, t = run(True, False, True)
    hw, tw = xs_round(xs_decode(h0, t0) + b.float().cpu().numpy()[None, :])
    hb, tb = _bits(h, t)
    assert np.array_equal(hb, hw) and np.array_equal(tb, tw)
    a, w, b, h0, t0, h, t = run(False, False, True)
    upd = a.double().cpu().numpy() @ w.double().cpu().numpy().T + b.double().cpu().numpy()
    err = np.abs(xs_decode(h, t).astype(np.float64) - (xs_decode(h0, t0).astype(np.float64) + upd))
    assert np.sqrt((err ** 2).mean()) < 5e-3 and err.max() < 0.05


@pytest.mark.parametrize("C", [128, 256])
def test_transition_fused_residual_tail(dev, C):
    from fastfold_amd import _lib
    M, Hd = 700, 4 * C
    g = torch.Generator().manual_seed(3)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, BF)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, BF)
    w1 = (torch.randn(Hd, C, generator=g) / C ** 0.5).to(dev, BF)
    b1 = (0.1 * torch.randn(Hd, generator=g)).to(dev, BF)
    b2 = torch.randn(C, generator=g).to(dev, BF)
    w2 = (torch.randn(C, Hd, generator=g) / Hd ** 0.5).to(dev, BF)
    def run(w2_, b2_):
        h, t = _stream((M, C), dev, 9)
        h0, t0 = h.clone(), t.clone()
        _lib.transition_fused(h, h, gam, bet, w1, b1, w2_, b2_, M=M, C=C, hidden=Hd, xtail=t)
        return h0, t0, h, t
    h0, t0, h, t = run(torch.zeros_like(w2), torch.zeros_like(b2))
    assert torch.equal(h, h0) and torch.equal(t, t0)
    h0, t0, h, t = run(torch.zeros_like(w2), b2)
    hw, tw = xs_round(xs_decode(h0, t0) + b2.float().cpu().numpy()[None, :])
    hb, tb = _bits(h, t)
    assert np.array_equal(hb, hw) and np.array_equal(tb, tw)
    h0, t0, h, t = run(w2, b2)
    x = h0.double().cpu()                                   # the LayerNorm reads the bf16 value alone
    ln = torch.nn.functional.layer_norm(x, (C,), gam.double().cpu(), bet.double().cpu(), 1e-5)
    hid = torch.relu(ln.to(BF).double() @ w1.double().cpu().T + b1.double().cpu())
    upd = (hid.to(BF).double() @ w2.double().cpu().T + b2.double().cpu()).numpy()
    err = np.abs(xs_decode(h, t).astype(np.float64) - (xs_decode(h0, t0).astype(np.float64) + upd))
    assert np.sqrt((err ** 2).mean()) < 5e-3 and err.max() < 0.06


def test_opm_fused_residual_tail(dev):
    from fastfold_amd import _lib
    r, s = 64, 64
    g = torch.Generator().manual_seed(4)
    a_t = (torch.randn(r * 32, s, generator=g) * 0.5).to(dev, BF)
    b_t = (torch.randn(r * 32, s, generator=g) * 0.5).to(dev, BF)
    w = (torch.randn(128, 32, 32, generator=g) / 32).to(dev, BF)
    bias = torch.randn(128, generator=g).to(dev, BF)
    norm = (torch.rand(r, r, generator=g) * s + 1).to(dev)
    w_ed = w.transpose(1, 2).reshape(128, 1024).contiguous()
    def run(w_, b_):
        h, t = _stream((r * r, 128), dev, 13)
        h0, t0 = h.clone(), t.clone()
        _lib.opm_fused(h, h, a_t, b_t, w_, b_, norm, r=r, spad=s, eps=1e-3, xtail=t)
        return h0, t0, h, t
    h0, t0, h, t = run(torch.zeros_like(w_ed), torch.zeros_like(bias))
    assert torch.equal(h, h0) and torch.equal(t, t0)
    h0, t0, h, t = run(w_ed, bias)
    A = a_t.double().cpu().numpy().reshape(r, 32, s)
    B = b_t.double().cpu().numpy().reshape(r, 32, s)
    O = torch.from_numpy(np.einsum("ids,jes->ijde", A, B)).to(BF).double().numpy()
    upd = (np.einsum("ijde,cde->ijc", O, w.double().cpu().numpy()) + bias.double().cpu().numpy()) \
        / (norm.double().cpu().numpy()[..., None] + 1e-3)
    err = np.abs(xs_decode(h, t).astype(np.float64).reshape(r, r, 128) - (xs_decode(h0, t0).astype(np.float64).reshape(r, r, 128) + upd))
    assert np.sqrt((err ** 2).mean()) < 3e-3 and err.max() < 0.05


@pytest.mark.parametrize("name", ["tmo", "tmi", "tas", "tae", "ptrans", "opm", "row", "col", "mtrans"])
@pytest.mark.parametrize("r,s", [(64, 32), (40, 24)])
def test_submodules_with_tail_round_to_the_plain_result(dev, name, r, s):
    """Each sub-module of a block with a zero input tail: the bf16 tensor it leaves is the plain result up to the
    one rounding the tail replaces (the plain path rounds the update to bf16 before adding, the tail path does
    not), and value + tail is closer to the fp32 oracle's sum than the rounded value is.  r = 64 takes the fast
    kernels, r = 40 the fall-backs."""
    import copy
    from fastfold_amd.synthetic import bf16_round, synth_inputs, synth_nn_state
    from fastfold_amd.utils.inject_fastnn import inject_fastnn
    from oracle.evoformer_ref import OracleModel
    from test_evoformer_gpu import KW, _oracle_sub
    model = OracleModel(no_blocks=1, **KW).eval()
    sd = synth_nn_state(seed=50, no_blocks=1, fan_in_scaled=True)
    model.evoformer.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    fast = inject_fastnn(copy.deepcopy(model)).evoformer.to(dev, BF).eval().blocks[0]
    m, z, mm, pm = synth_inputs(50, s, r, mask_tail_frac=0.1)
    m, z = bf16_round(m), bf16_round(z)
    tm, tz, tmm, tpm = (torch.from_numpy(a).to(dev, BF)[None] for a in (m, z, mm, pm))
    mod, args, x = {
        "row": (fast.msa.MSARowAttentionWithPairBias, (tm, tz, tmm), tm), "col": (fast.msa.MSAColumnAttention, (tm, tmm), tm),
        "mtrans": (fast.msa.MSATransition, (tm,), tm), "opm": (fast.communication, (tm, tmm, tz), tz),
        "tmo": (fast.pair.TriangleMultiplicationOutgoing, (tz, tpm), tz),
        "tmi": (fast.pair.TriangleMultiplicationIncoming, (tz, tpm), tz),
        "tas": (fast.pair.TriangleAttentionStartingNode, (tz, tpm), tz),
        "tae": (fast.pair.TriangleAttentionEndingNode, (tz, tpm), tz), "ptrans": (fast.pair.PairTransition, (tz,), tz)}[name]
    with torch.no_grad():
        plain = torch.empty_like(x)
        mod._run(*args, plain)
        out, tail = torch.empty_like(x), torch.zeros(x.shape, dtype=torch.int8, device=dev)
        mod._run(*args, out, tail)
        which, upd = _oracle_sub(model.evoformer.blocks[0], name, *(torch.from_numpy(a) for a in (m, z, mm, pm)))
    ref = (torch.from_numpy(m if which == "m" else z) + upd).numpy()
    nv = r - int(round(0.1 * r))
    sl = (slice(None), slice(0, nv)) if which == "m" else (slice(0, nv), slice(0, nv))
    full = xs_decode(out[0], tail[0])
    # the bf16 tensor agrees with the plain result to one ulp (two roundings against one)
    d = np.abs(out[0].float().cpu().numpy() - plain[0].float().cpu().numpy())[sl]
    assert d.max() <= 2.0 ** -7 * max(1.0, float(np.abs(ref[sl]).max()))
    e_full = np.sqrt(((full - ref)[sl] ** 2).mean())
    e_plain = np.sqrt(((plain[0].float().cpu().numpy() - ref)[sl] ** 2).mean())
    assert e_full <= e_plain * 1.02 + 1e-6, (e_full, e_plain)
    assert int((tail != 0).sum()) > tail.numel() // 2       # the tail is really written
