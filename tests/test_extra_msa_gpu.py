"""GPU parity of the extra-MSA path (global column attention kernel, head-dim-8 row attention, block and
stack) against the CPU oracle (oracle.evoformer_ref, pinned by golden vectors from the reference and a
float64 brute force of the global attention).

Tolerances: fp32 max-abs <= 1e-4 (scaled by the size of the reference where updates are O(10));
bf16 relative L2 <= 2e-2 against the fp32 oracle."""
import copy
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fastfold_amd.synthetic import synth_extra_nn_state, synth_inputs
from oracle.evoformer_ref import ExtraMSAStack as OracleExtraStack, GlobalAttention as OracleGlobalAttention, OracleModel

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "extra_msa_nn_golden.npz")


def _t(x, dev, dtype):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev, dtype)


def _f(t):
    return t.detach().float().cpu().numpy()


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def _oracle(seed, nb, fis=True):
    model = OracleModel(no_blocks=1, extra_msa_kwargs=dict(no_blocks=nb)).eval()
    sd = synth_extra_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis)
    model.extra_msa_stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return model


def _fast(model, dev, dtype):
    from fastfold_amd.utils.inject_fastnn import inject_extramsa
    m2 = copy.deepcopy(model)
    inject_extramsa(m2)
    return m2.extra_msa_stack.to(device=dev, dtype=dtype).eval()


def _core_ref(m, mask, gamma, beta, wq, wk, wv, H, D, eps, ln=True):
    """float64 o[j, h*D+d] of the global attention for m [S, R, C], mask [S, R]."""
    m, mask, gamma, beta, wq, wk, wv = (torch.as_tensor(x, dtype=torch.float64) for x in (m, mask, gamma, beta, wq, wk, wv))
    x = F.layer_norm(m, (m.shape[-1],), gamma, beta, 1e-5) if ln else m
    x = x.transpose(0, 1)                     # [R, S, C]
    mk = mask.transpose(0, 1)                 # [R, S]
    q = (x * mk[..., None]).sum(1) / (mk.sum(1, keepdim=True) + eps)
    q = (q @ wq.T).view(-1, H, D) * D ** -0.5
    k, v = x @ wk.T, x @ wv.T                 # [R, S, D]
    a = torch.einsum("rhd,rsd->rhs", q, k)
    a = torch.where(mk[:, None, :] != 0, a, torch.full_like(a, -1e9))
    w = torch.softmax(a, -1)
    return torch.einsum("rhs,rsd->rhd", w, v).reshape(x.shape[0], H * D).numpy()


@pytest.mark.parametrize("S,R,C,H,D", [(40, 9, 64, 8, 8), (133, 5, 64, 8, 8), (7, 3, 32, 4, 8), (70, 4, 128, 8, 16),
                                       (1, 2, 64, 8, 8), (515, 3, 64, 8, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_global_attention_core(dev, S, R, C, H, D, dtype):
    from fastfold_amd import _lib
    rng = np.random.RandomState(S * 7 + R)
    m = rng.standard_normal((S, R, C)).astype(np.float32) * 1.5 + 0.3
    mask = (rng.uniform(size=(S, R)) > 0.25).astype(np.float32)
    mask[0, :] = 1
    if R > 1:
        mask[:, R - 1] = 0                     # a fully masked column: plain mean of v
    gamma = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(C)).astype(np.float32)
    wq, wk, wv = (rng.standard_normal(sh).astype(np.float32) / np.sqrt(C) * 2.0 for sh in ((H * D, C), (D, C), (D, C)))
    tm, tmask, tg, tb, twq, twk, twv = (_t(x, dev, dtype) for x in (m, mask, gamma, beta, wq, wk, wv))
    rnd = [_f(t) for t in (tm, tmask, tg, tb, twq, twk, twv)]     # what the kernel really reads
    ref = _core_ref(*rnd, H, D, 1e-10)
    o = torch.full((R, H * D), float("nan"), dtype=dtype, device=dev)
    _lib.global_attention_core(o, tm, tmask, tg, tb, twq, twk, twv, S=S, R=R, C=C, H=H, D=D, m_ss=R * C, m_sr=C,
                               mask_ss=R, mask_sr=1, scaling=D ** -0.5, eps=1e-10)
    got = _f(o)
    if dtype == torch.float32:
        assert np.abs(got - ref).max() <= 1e-4, np.abs(got - ref).max()
    else:
        assert _rel_l2(got, ref) <= 2e-2, _rel_l2(got, ref)
    # transposed storage [R, S, C], no LayerNorm, no mask
    xt = tm.transpose(0, 1).contiguous()
    ref2 = _core_ref(rnd[0], np.ones((S, R)), rnd[2], rnd[3], rnd[4], rnd[5], rnd[6], H, D, 1e-10, ln=False)
    o2 = torch.empty_like(o)
    _lib.global_attention_core(o2, xt, None, None, None, twq, twk, twv, S=S, R=R, C=C, H=H, D=D, m_ss=C, m_sr=S * C,
                               mask_ss=0, mask_sr=0, scaling=D ** -0.5, eps=1e-10)
    if dtype == torch.float32:
        assert np.abs(_f(o2) - ref2).max() <= 1e-4
    else:
        assert _rel_l2(_f(o2), ref2) <= 2e-2


def test_global_attention_core_rejects_bad_arguments(dev):
    from fastfold_amd import _lib
    x = torch.zeros(4, 2, 48, device=dev)
    w = torch.zeros(64, 48, device=dev)
    with pytest.raises(RuntimeError, match="C must be"):
        _lib.global_attention_core(torch.zeros(2, 64, device=dev), x, None, None, None, w, w[:8], w[:8], S=4, R=2, C=48,
                                   H=8, D=8, m_ss=96, m_sr=48, mask_ss=0, mask_sr=0, scaling=1.0, eps=1e-10)
    x = torch.zeros(4, 2, 64, device=dev)
    w = torch.zeros(144, 64, device=dev)
    with pytest.raises(RuntimeError, match="H"):
        _lib.global_attention_core(torch.zeros(2, 144, device=dev), x, None, None, None, w, w[:16], w[:16], S=4, R=2,
                                   C=64, H=9, D=16, m_ss=128, m_sr=64, mask_ss=0, mask_sr=0, scaling=1.0, eps=1e-10)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_global_attention_module(dev, dtype):
    """Public GlobalAttention.forward(m [1, R, S, C], mask [1, R, S]) against the oracle module."""
    from fastfold_amd.model.fastnn.ops import GlobalAttention
    from fastfold_amd.utils.inject_fastnn import copy_global_attention
    torch.manual_seed(5)
    ref = OracleGlobalAttention(64, 8, 8, inf=1e9, eps=1e-10)
    with torch.no_grad():
        for p in ref.parameters():
            p.copy_(torch.randn_like(p) * 0.2)
    fast = GlobalAttention(64, 8, 8, 64)
    with torch.no_grad():
        copy_global_attention(fast, ref)
    fast = fast.to(dev, dtype).eval()
    rng = np.random.RandomState(6)
    R, S = 6, 50
    m = rng.standard_normal((1, R, S, 64)).astype(np.float32)
    mask = (rng.uniform(size=(1, R, S)) > 0.2).astype(np.float32)
    mask[..., 0] = 1
    mb = _f(_t(m, dev, dtype))
    ref = copy.deepcopy(ref).to(torch.float32)
    if dtype == torch.bfloat16:
        with torch.no_grad():
            for p in ref.parameters():
                p.copy_(p.to(torch.bfloat16).float())
    with torch.no_grad():
        want = ref(torch.from_numpy(mb), torch.from_numpy(mask)).numpy()
        got = _f(fast(_t(mb, dev, dtype), _t(mask, dev, dtype)))
        # the same through a transposed view, as the reference's column module passes it
        got2 = _f(fast(_t(mb, dev, dtype).transpose(1, 2).contiguous().transpose(1, 2), _t(mask, dev, dtype)))
    if dtype == torch.float32:
        assert np.abs(got - want).max() <= 1e-4 and np.abs(got2 - want).max() <= 1e-4
    else:
        assert _rel_l2(got, want) <= 2e-2 and _rel_l2(got2, want) <= 2e-2


SUB = ["row", "col", "mtrans", "opm"]


def _oracle_sub(blk, name, m, z, mm):
    with torch.no_grad():
        if name == "row":
            return blk.msa_att_row(m, z=z, mask=mm), "m"
        if name == "col":
            return blk.msa_att_col(m, mask=mm), "m"
        if name == "mtrans":
            return blk.core.msa_transition(m, mask=None), "m"
        return blk.core.outer_product_mean(m, mask=mm), "z"


def _fast_sub(blk, name, m, z, mm):
    with torch.no_grad():
        if name == "row":
            return blk.msa_stack.MSARowAttentionWithPairBias(m, z, mm) - m
        if name == "col":
            return blk.msa_stack.MSAColumnAttention(m, mm) - m
        if name == "mtrans":
            return blk.msa_stack.MSATransition(m) - m
        return blk.communication(m, mm, z) - z


@pytest.mark.parametrize("s,r,tail", [(12, 40, 0.2), (70, 33, 0.0), (140, 64, 0.1)])
@pytest.mark.parametrize("name", SUB)
def test_extra_submodule_updates_fp32(dev, name, s, r, tail):
    model = _oracle(41, 1)
    fast = _fast(model, dev, torch.float32)
    m, z, mm, pm = synth_inputs(17, s, r, c_m=64, mask_tail_frac=tail)
    ref, which = _oracle_sub(model.extra_msa_stack.blocks[0], name, *(torch.from_numpy(t) for t in (m, z, mm)))
    got = _fast_sub(fast.blocks[0], name, *(_t(x[None], dev, torch.float32) for x in (m, z, mm)))[0]
    nv = r - int(round(tail * r))
    ref = ref.numpy()
    got, ref = (_f(got)[:, :nv], ref[:, :nv]) if which == "m" else (_f(got)[:nv, :nv], ref[:nv, :nv])
    scale = max(1.0, float(np.abs(ref).max()))
    assert np.abs(got - ref).max() <= 1e-4 * scale, (name, np.abs(got - ref).max(), scale)


@pytest.mark.parametrize("s,r,tail", [(48, 64, 0.1), (256, 96, 0.0)])
@pytest.mark.parametrize("name", SUB)
def test_extra_submodule_updates_bf16(dev, name, s, r, tail):
    model = _oracle(42, 1)
    fast = _fast(model, dev, torch.bfloat16)
    m, z, mm, pm = synth_inputs(18, s, r, c_m=64, mask_tail_frac=tail)
    mb, zb = (_f(_t(x, dev, torch.bfloat16)) for x in (m, z))
    ref, which = _oracle_sub(model.extra_msa_stack.blocks[0], name, torch.from_numpy(mb), torch.from_numpy(zb),
                             torch.from_numpy(mm))
    out = _fast_sub(fast.blocks[0], name, *(_t(x[None], dev, torch.bfloat16) for x in (mb, zb, mm)))[0]
    nv = r - int(round(tail * r))
    ref = ref.numpy()
    base = mb if which == "m" else zb
    if which == "m":
        got, ref, base = _f(out)[:, :nv], ref[:, :nv], base[:, :nv]
    else:
        got, ref, base = _f(out)[:nv, :nv], ref[:nv, :nv], base[:nv, :nv]
    err = np.linalg.norm(got - ref)
    bound = 2e-2 * np.linalg.norm(ref) + 2.0 ** -8 * np.linalg.norm(base + ref)
    assert err <= bound, (name, err, bound)


def test_extra_golden_vectors_fp32(dev):
    """The reference's own ExtraMSAStack outputs (un-masked region: the reference masks its transitions,
    fastnn does not, which only changes masked positions)."""
    g = np.load(GOLDEN)
    for name in sorted({k.split(".")[0] for k in g.files}):
        seed, nb, s, r, tail, fis = (int(v) for v in g[name + ".cfg"])
        fast = _fast(_oracle(seed, nb, bool(fis)), dev, torch.float32)
        m, z, mm, pm = synth_inputs(seed, s, r, c_m=64, mask_tail_frac=tail / 100)
        tm, tz, tmm, tpm = (_t(x, dev, torch.float32) for x in (m, z, mm, pm))
        keep = [t.clone() for t in (tm, tz)]
        with torch.no_grad():
            zo = fast(tm, tz, chunk_size=None, msa_mask=tmm, pair_mask=tpm)
        assert torch.equal(tm, keep[0]) and torch.equal(tz, keep[1]), "forward must not modify its inputs"
        nv = r - int(round(tail / 100 * r))
        got, ref = _f(zo)[:nv, :nv], g[name + ".z"][:nv, :nv]
        scale = max(1.0, float(np.abs(ref).max()))
        assert np.abs(got - ref).max() <= 1e-4 * scale, (name, np.abs(got - ref).max(), scale)
        # list-passing variant
        ml, zl = [tm.clone()], [tz.clone()]
        with torch.no_grad():
            zl = fast.inplace(ml, zl, chunk_size=None, msa_mask=tmm, pair_mask=tpm)
        assert torch.equal(zl[0], zo)


def test_extra_block_interface_padding_and_chaining(dev):
    """first / middle / last stand-alone blocks carry [1, s+1, r+1, c] / [1, r+1, r+1, c] between them."""
    model = _oracle(43, 3)
    fast = _fast(model, dev, torch.float32)
    s, r = 11, 24
    m, z, mm, pm = synth_inputs(43, s, r, c_m=64, mask_tail_frac=0.1)
    tm, tz, tmm, tpm = (_t(x, dev, torch.float32) for x in (m, z, mm, pm))
    with torch.no_grad():
        sz = fast(tm, tz, chunk_size=None, msa_mask=tmm, pair_mask=tpm)
        a, b = fast.blocks[0](tm, tz, tmm, tpm)
        assert a.shape == (1, s + 1, r + 1, 64) and b.shape == (1, r + 1, r + 1, 128)
        a, b = fast.blocks[1](a, b, tmm, tpm)
        assert a.shape == (1, s + 1, r + 1, 64) and b.shape == (1, r + 1, r + 1, 128)
        a, b = fast.blocks[2](a, b, tmm, tpm)
    assert a.shape == (s, r, 64) and b.shape == (r, r, 128)
    assert torch.equal(b, sz)


def test_extra_stack_bf16_rel_l2(dev):
    nb, s, r, tail = 4, 96, 72, 0.1
    model = _oracle(44, nb)
    fast = _fast(model, dev, torch.bfloat16)
    m, z, mm, pm = synth_inputs(44, s, r, c_m=64, mask_tail_frac=tail)
    mb, zb = (_f(_t(x, dev, torch.bfloat16)) for x in (m, z))
    with torch.no_grad():
        rz = model.extra_msa_stack(torch.from_numpy(mb), torch.from_numpy(zb), msa_mask=torch.from_numpy(mm),
                                   pair_mask=torch.from_numpy(pm), _mask_trans=False).numpy()
        gz = fast(*(_t(x, dev, torch.bfloat16) for x in (mb, zb)), chunk_size=None,
                  msa_mask=_t(mm, dev, torch.bfloat16), pair_mask=_t(pm, dev, torch.bfloat16))
    nv = r - int(round(tail * r))
    assert _rel_l2(_f(gz)[:nv, :nv], rz[:nv, :nv]) <= 2e-2


def test_inject_fastnn_swaps_both_stacks_and_keys(dev):
    from fastfold_amd.model.fastnn import ExtraMSAStack
    from fastfold_amd.utils.inject_fastnn import inject_fastnn
    model = inject_fastnn(copy.deepcopy(_oracle(45, 1)))
    assert isinstance(model.extra_msa_stack, ExtraMSAStack)
    keys = set(model.extra_msa_stack.state_dict().keys())
    for k in ("blocks.0.msa_stack.MSARowAttentionWithPairBias.attention.to_qkv.weight",
              "blocks.0.msa_stack.MSAColumnAttention.global_attention.to_kv.weight",
              "blocks.0.msa_stack.MSAColumnAttention.global_attention.gating_bias",
              "blocks.0.msa_stack.MSATransition.linear1.weight", "blocks.0.communication.linear_a.weight",
              "blocks.0.pair_stack.TriangleAttentionEndingNode.out_bias"):
        assert k in keys, k
    assert model.extra_msa_stack.blocks[0].msa_stack.MSARowAttentionWithPairBias.attention.to_qkv.weight.shape == (192, 64)


@pytest.mark.parametrize("inplace", [False, True])
def test_multimer_block_order(dev, inplace):
    """is_multimer blocks run outer product mean and pair stack first and the MSA stack on the pair tensor in
    between (fastnn/evoformer.py:70-76, fastnn/msa.py:264-270): checked against the same modules called in
    that order by hand."""
    from fastfold_amd.model.fastnn import Evoformer, ExtraMSABlock
    torch.manual_seed(11)
    for cls, c_m in ((Evoformer, 256), (ExtraMSABlock, 64)):
        blk = cls(c_m, 128, first_block=True, last_block=True, is_multimer=True)
        with torch.no_grad():
            for n, p in blk.named_parameters():
                p.copy_((1.0 if ("norm" in n and n.endswith("weight")) else 0.0) + 0.05 * torch.randn_like(p))
        blk = blk.to(dev).eval()
        s, r = 9, 20
        m, z, mm, pm = (_t(x, dev, torch.float32) for x in synth_inputs(12, s, r, c_m=c_m, mask_tail_frac=0.1))
        msa = blk.msa if cls is Evoformer else blk.msa_stack
        pair = blk.pair if cls is Evoformer else blk.pair_stack
        with torch.no_grad():
            z1 = blk.communication(m[None], mm[None], z[None])
            z2 = pair(z1, pm[None])
            m2 = msa(m[None], z1, mm[None])
            if inplace:
                ml, zl = [m.clone()], [z.clone()]
                ml, zl = blk.inplace(ml, zl, mm, pm)
                gm, gz = ml[0], zl[0]
            else:
                gm, gz = blk(m, z, mm, pm)
        assert torch.equal(gm, m2[0]) and torch.equal(gz, z2[0]), cls.__name__


@pytest.mark.parametrize("s,r,tail", [(1, 1, 0.0), (3, 1, 0.0), (2, 17, 0.1), (1025, 33, 0.1)])
def test_extra_stack_extreme_shapes(dev, s, r, tail):
    """A single extra sequence, a single residue, N_extra just past a 1024 boundary: two blocks, both precisions."""
    model = _oracle(44, 2)
    m, z, mm, pm = synth_inputs(4, s, r, c_m=64, mask_tail_frac=tail)
    with torch.no_grad():
        rz = model.extra_msa_stack(torch.from_numpy(m), torch.from_numpy(z), msa_mask=torch.from_numpy(mm),
                                   pair_mask=torch.from_numpy(pm), _mask_trans=False).numpy()
    nv = r - int(round(tail * r))
    for dtype in (torch.float32, torch.bfloat16):
        fast = _fast(model, dev, dtype)
        with torch.no_grad():
            gz = _f(fast(*(_t(x, dev, dtype) for x in (m, z)), chunk_size=None, msa_mask=_t(mm, dev, dtype),
                         pair_mask=_t(pm, dev, dtype)))
        if dtype == torch.float32:
            assert np.abs(gz[:nv, :nv] - rz[:nv, :nv]).max() <= 1e-4 * max(1.0, float(np.abs(rz).max()))
        else:
            assert _rel_l2(gz[:nv, :nv], rz[:nv, :nv]) <= 2e-2
