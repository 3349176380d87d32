"""GPU parity of the template pair stack (the pair modules at c_t = 64, 4 heads of 16, multiplication
width 64, transition factor 2) against the CPU oracle, itself pinned by golden vectors written by the
reference's fastfold.model.nn.template.TemplatePairStack.

Tolerances: fp32 max-abs <= 1e-4; bf16 relative L2 <= 2e-2 against the fp32 oracle."""
import copy
import os

import numpy as np
import pytest
import torch

from fastfold_amd.synthetic import synth_template_inputs, synth_template_nn_state
from oracle.evoformer_ref import TemplatePairStack as OracleStack

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "template_pair_nn_golden.npz")


class _Embedder(torch.nn.Module):
    def __init__(self, stack):
        super().__init__()
        self.template_pair_stack = stack


def _t(x, dev, dtype):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev, dtype)


def _f(t):
    return t.detach().float().cpu().numpy()


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def _oracle(seed, nb, fis=True):
    st = OracleStack(no_blocks=nb).eval()
    sd = synth_template_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis)
    st.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return st


def _fast(oracle, dev, dtype):
    from fastfold_amd.utils.inject_fastnn import inject_template_pair_stack
    e = inject_template_pair_stack(_Embedder(copy.deepcopy(oracle)))
    return e.template_pair_stack.to(device=dev, dtype=dtype).eval()


SUB = ["tas", "tae", "tmo", "tmi", "ptrans"]


def _oracle_sub(blk, name, z, pm):
    with torch.no_grad():
        if name == "tas":
            return blk.tri_att_start(z, mask=pm)
        if name == "tae":
            return blk.tri_att_end(z, mask=pm)
        if name == "tmo":
            return blk.tri_mul_out(z, mask=pm)
        if name == "tmi":
            return blk.tri_mul_in(z, mask=pm)
        return blk.pair_transition(z, mask=None)


def _fast_sub(blk, name, z, pm):
    with torch.no_grad():
        if name == "tas":
            return blk.TriangleAttentionStartingNode(z, pm) - z
        if name == "tae":
            return blk.TriangleAttentionEndingNode(z, pm) - z
        if name == "tmo":
            return blk.TriangleMultiplicationOutgoing(z, pm) - z
        if name == "tmi":
            return blk.TriangleMultiplicationIncoming(z, pm) - z
        return blk.PairTransition(z) - z


@pytest.mark.parametrize("r,tail", [(40, 0.2), (33, 0.0), (64, 0.1)])
@pytest.mark.parametrize("name", SUB)
def test_template_submodule_updates_fp32(dev, name, r, tail):
    oracle = _oracle(51, 1)
    fast = _fast(oracle, dev, torch.float32)
    t, pm = synth_template_inputs(19, 1, r, mask_tail_frac=tail)
    ref = _oracle_sub(oracle.blocks[0], name, torch.from_numpy(t), torch.from_numpy(pm)[None])[0].numpy()
    got = _f(_fast_sub(fast.blocks[0], name, _t(t, dev, torch.float32), _t(pm[None], dev, torch.float32)))[0]
    nv = r - int(round(tail * r))
    got, ref = got[:nv, :nv], ref[:nv, :nv]
    scale = max(1.0, float(np.abs(ref).max()))
    assert np.abs(got - ref).max() <= 1e-4 * scale, (name, np.abs(got - ref).max(), scale)


@pytest.mark.parametrize("r,tail", [(64, 0.1), (96, 0.0)])
@pytest.mark.parametrize("name", SUB)
def test_template_submodule_updates_bf16(dev, name, r, tail):
    oracle = _oracle(52, 1)
    fast = _fast(oracle, dev, torch.bfloat16)
    t, pm = synth_template_inputs(20, 1, r, mask_tail_frac=tail)
    tb = _f(_t(t, dev, torch.bfloat16))
    ref = _oracle_sub(oracle.blocks[0], name, torch.from_numpy(tb), torch.from_numpy(pm)[None])[0].numpy()
    out = _f(_fast_sub(fast.blocks[0], name, _t(tb, dev, torch.bfloat16), _t(pm[None], dev, torch.bfloat16)))[0]
    nv = r - int(round(tail * r))
    got, ref, base = out[:nv, :nv], ref[:nv, :nv], tb[0, :nv, :nv]
    err = np.linalg.norm(got - ref)
    bound = 2e-2 * np.linalg.norm(ref) + 2.0 ** -8 * np.linalg.norm(base + ref)
    assert err <= bound, (name, err, bound)


def test_template_golden_vectors_fp32(dev):
    g = np.load(GOLDEN)
    for name in sorted({k.split(".")[0] for k in g.files}):
        seed, nb, nt, r, tail, fis = (int(v) for v in g[name + ".cfg"])
        fast = _fast(_oracle(seed, nb, bool(fis)), dev, torch.float32)
        t, pm = synth_template_inputs(seed, nt, r, mask_tail_frac=tail / 100)
        tt, tpm = _t(t, dev, torch.float32), _t(pm[None], dev, torch.float32)
        keep = tt.clone()
        with torch.no_grad():
            to = fast(tt, tpm, chunk_size=None)
        assert torch.equal(tt, keep), "forward must not modify its input"
        nv = r - int(round(tail / 100 * r))
        got, ref = _f(to)[:, :nv, :nv], g[name + ".t"][:, :nv, :nv]
        assert np.abs(got - ref).max() <= 1e-4, (name, np.abs(got - ref).max())
        tl = [tt.clone()]
        with torch.no_grad():
            tl = fast.inplace(tl, tpm, chunk_size=None)
        assert torch.equal(tl[0], to)


def test_template_block_interface_padding_and_chaining(dev):
    oracle = _oracle(53, 3)
    fast = _fast(oracle, dev, torch.float32)
    r = 24
    t, pm = synth_template_inputs(53, 1, r, mask_tail_frac=0.1)
    tt, tpm = _t(t, dev, torch.float32), _t(pm[None], dev, torch.float32)
    with torch.no_grad():
        want = fast(tt, tpm, chunk_size=None)
        a = fast.blocks[0](tt, tpm)
        assert a.shape == (1, r + 1, r + 1, 64)
        a = fast.blocks[1](a, tpm)
        assert a.shape == (1, r + 1, r + 1, 64)
        a = fast.blocks[2](a, tpm)
        assert a.shape == (1, r, r, 64)
        a = fast.layer_norm(a)
    assert torch.equal(a, want)


def test_template_stack_bf16_rel_l2(dev):
    nb, nt, r, tail = 2, 2, 72, 0.1
    oracle = _oracle(54, nb)
    fast = _fast(oracle, dev, torch.bfloat16)
    t, pm = synth_template_inputs(54, nt, r, mask_tail_frac=tail)
    tb = _f(_t(t, dev, torch.bfloat16))
    with torch.no_grad():
        ref = oracle(torch.from_numpy(tb), torch.from_numpy(pm)[None], _mask_trans=False).numpy()
        got = _f(fast(_t(tb, dev, torch.bfloat16), _t(pm[None], dev, torch.bfloat16), chunk_size=None))
    nv = r - int(round(tail * r))
    assert _rel_l2(got[:, :nv, :nv], ref[:, :nv, :nv]) <= 2e-2


@pytest.mark.parametrize("nt,r,tail", [(1, 1, 0.0), (4, 2, 0.0), (1, 17, 0.1), (2, 130, 0.2)])
def test_template_stack_extreme_shapes(dev, nt, r, tail):
    """One residue, two residues with four templates, sizes just past a tile edge: two blocks, both precisions."""
    oracle = _oracle(54, 2)
    t, pm = synth_template_inputs(5, nt, r, mask_tail_frac=tail)
    with torch.no_grad():
        ref = oracle(torch.from_numpy(t), torch.from_numpy(pm)[None], _mask_trans=False).numpy()
    nv = r - int(round(tail * r))
    for dtype in (torch.float32, torch.bfloat16):
        fast = _fast(oracle, dev, dtype)
        with torch.no_grad():
            got = _f(fast(_t(t, dev, dtype), _t(pm[None], dev, dtype), chunk_size=None))
        if dtype == torch.float32:
            assert np.abs(got[:, :nv, :nv] - ref[:, :nv, :nv]).max() <= 1e-4 * max(1.0, float(np.abs(ref).max()))
        else:
            assert _rel_l2(got[:, :nv, :nv], ref[:, :nv, :nv]) <= 2e-2


# ---------------------------------------------------------------- template point-wise attention ----
def _pointwise(seed, dev, dtype):
    from fastfold_amd.model.fastnn import TemplatePointwiseAttention
    from fastfold_amd.synthetic import synth_pointwise_nn_state
    from oracle.evoformer_ref import TemplatePointwiseAttention as OraclePW
    sd = {k: torch.from_numpy(v) for k, v in synth_pointwise_nn_state(seed=seed).items()}
    ref = OraclePW().eval()
    ref.load_state_dict(sd, strict=True)
    fast = TemplatePointwiseAttention(c_t=64, c_z=128, c_hidden=16, no_heads=4, inf=1e5)
    missing, unexpected = fast.load_state_dict(sd, strict=True)       # same keys as the reference's module
    assert not missing and not unexpected
    return ref, fast.to(dev, dtype).eval()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nt,r,tmask", [(4, 12, (1, 1, 1, 1)), (4, 9, (1, 0, 1, 0)), (1, 7, (1,)), (2, 5, (0, 0)),
                                        (8, 33, (1, 1, 0, 1, 1, 0, 1, 1)), (3, 1, (0, 1, 1))])
def test_template_pointwise_attention(dev, dtype, nt, r, tmask):
    """fastnn/template.py:83-131 against the oracle (pinned by the reference's vectors); the fastnn module zeroes
    the update itself when no template is valid (template.py:117-119)."""
    from fastfold_amd.synthetic import synth_pointwise_inputs
    ref, fast = _pointwise(70 + nt, dev, dtype)
    t, z = synth_pointwise_inputs(70 + r, nt, r)
    tm = torch.tensor([float(x) for x in tmask])
    tb, zb = (torch.from_numpy(x).to(dtype).float() for x in (t, z))
    with torch.no_grad():
        want = ref(tb, zb, template_mask=tm).numpy() * float(tm.sum() > 0)
        got = fast(tb.to(dev, dtype), zb.to(dev, dtype), template_mask=tm.to(dev, dtype))
        zin = zb.to(dev, dtype)
        zres = fast.inplace(tb.to(dev, dtype), zin, template_mask=tm.to(dev, dtype))
    assert got.shape == (r, r, 128) and got.dtype == dtype
    assert zres.data_ptr() == zin.data_ptr()
    got, zres = _f(got), _f(zres)
    if dtype == torch.float32:
        assert np.abs(got - want).max() <= 1e-4 * max(1.0, float(np.abs(want).max()))
        assert np.abs(zres - (zb.numpy() + want)).max() <= 1e-4 * max(1.0, float(np.abs(want).max()))
    else:
        if tm.sum() > 0:
            assert _rel_l2(got, want) <= 2e-2
        else:
            assert np.abs(got).max() == 0.0
        assert _rel_l2(zres, zb.numpy() + want) <= 2e-2


def test_template_pointwise_golden_vectors(dev):
    """The reference's own outputs (tests/golden/make_golden.py pointwise), fp32."""
    from fastfold_amd.synthetic import synth_pointwise_inputs
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "template_pointwise_nn_golden.npz"))
    for name in sorted(k[:-4] for k in g.files if k.endswith(".cfg")):
        cfg = g[name + ".cfg"]
        seed, nt, r, tmask = int(cfg[0]), int(cfg[1]), int(cfg[2]), [float(x) for x in cfg[3:]]
        if sum(tmask) == 0:
            continue          # the fastnn module returns zeros there; the reference's nn module leaves that to its caller
        _, fast = _pointwise(seed, dev, torch.float32)
        t, z = synth_pointwise_inputs(seed, nt, r)
        with torch.no_grad():
            got = _f(fast(_t(t, dev, torch.float32), _t(z, dev, torch.float32), template_mask=torch.tensor(tmask, device=dev)))
        assert np.abs(got - g[name + ".out"]).max() <= 1e-4, name


def test_pointwise_core_rejects_bad_arguments(dev):
    from fastfold_amd import _lib
    q = torch.zeros(4, 64, device=dev)
    kv = torch.zeros(2, 4, 128, device=dev)
    o = torch.empty(4, 64, device=dev)
    b = torch.zeros(2, device=dev)
    with pytest.raises(RuntimeError, match="head width"):
        _lib.pointwise_attention_core(o, q, kv, b, P=4, H=4, D=12, NT=2, kv_st=512, kv_sp=128, v_off=64)
    with pytest.raises(RuntimeError, match="NT"):
        _lib.pointwise_attention_core(o, q, kv, torch.zeros(9, device=dev), P=4, H=4, D=16, NT=9, kv_st=512, kv_sp=128, v_off=64)
    with pytest.raises(RuntimeError, match="v_off"):
        _lib.pointwise_attention_core(o, q, kv, b, P=4, H=4, D=16, NT=2, kv_st=512, kv_sp=128, v_off=32)


def test_inject_swaps_the_pointwise_attention_too(dev):
    """An embedder that carries both the pair stack and the point-wise attention gets both swapped, parameters
    copied (inject_fastnn.py:271-279)."""
    from fastfold_amd.model.fastnn import TemplatePairStack, TemplatePointwiseAttention
    from fastfold_amd.synthetic import synth_pointwise_inputs, synth_pointwise_nn_state
    from fastfold_amd.utils.inject_fastnn import inject_template_pair_stack
    from oracle.evoformer_ref import TemplatePointwiseAttention as OraclePW
    e = _Embedder(copy.deepcopy(_oracle(54, 1)))
    e.template_pointwise_att = OraclePW().eval()
    e.template_pointwise_att.load_state_dict({k: torch.from_numpy(v) for k, v in synth_pointwise_nn_state(seed=5).items()})
    ref = copy.deepcopy(e.template_pointwise_att)
    inject_template_pair_stack(e)
    assert isinstance(e.template_pair_stack, TemplatePairStack)
    assert isinstance(e.template_pointwise_att, TemplatePointwiseAttention) and not e.template_pointwise_att.training
    t, z = synth_pointwise_inputs(5, 2, 6)
    e = e.to(dev)
    with torch.no_grad():
        got = _f(e.template_pointwise_att(_t(t, dev, torch.float32), _t(z, dev, torch.float32)))
        want = ref(torch.from_numpy(t), torch.from_numpy(z)).numpy()
    assert np.abs(got - want).max() <= 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("P,H,D,NT", [(37, 4, 16, 4), (130, 8, 8, 3), (65, 2, 32, 8), (1, 1, 8, 1)])
def test_pointwise_core_widths(dev, dtype, P, H, D, NT):
    """The core at every supported head width, with strided key / value rows, against float64 torch."""
    from fastfold_amd import _lib
    g = torch.Generator().manual_seed(P + D)
    hc = H * D
    pitch = 2 * hc + 16                                   # rows padded: strides are arguments
    q = torch.randn(P, hc, generator=g).to(dev, dtype)
    kv = torch.randn(NT, P, pitch, generator=g).to(dev, dtype)
    bias = torch.where(torch.rand(NT, generator=g) < 0.3, torch.tensor(-1e5), torch.tensor(0.0))
    bias[0] = 0.0
    o = torch.empty(P, hc, device=dev, dtype=dtype)
    _lib.pointwise_attention_core(o, q, kv, bias.to(dev), P=P, H=H, D=D, NT=NT, kv_st=P * pitch, kv_sp=pitch, v_off=hc + 16,
                                  out_scale=torch.full((1,), 0.5, device=dev))
    qd = q.double().cpu().view(P, H, D)
    kd = kv.double().cpu()[..., :hc].reshape(NT, P, H, D)
    vd = kv.double().cpu()[..., hc + 16:2 * hc + 16].reshape(NT, P, H, D)
    logits = torch.einsum("phd,tphd->pht", qd, kd) + bias.double()
    want = 0.5 * torch.einsum("pht,tphd->phd", torch.softmax(logits, -1), vd).reshape(P, hc).numpy()
    got = _f(o)
    if dtype == torch.float32:
        assert np.abs(got - want).max() <= 1e-4 * max(1.0, float(np.abs(want).max()))
    else:
        assert _rel_l2(got, want) <= 2e-2
