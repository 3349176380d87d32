"""GPU parity of the fastnn modules, block and stack (HIP kernels through the C ABI) against
the CPU oracle (oracle.evoformer_ref, pinned by the reference's golden vectors).

Tolerances: fp32 max-abs <= 1e-4 (north star); bf16 relative L2 <= 2e-2 against the fp32 oracle.
The "update" checks compare (out - in), so a wrong update cannot hide behind the residual
stream; weights there are fan-in scaled so every update is O(1)."""
import os

import numpy as np
import pytest
import torch

from fastfold_amd.synthetic import synth_inputs, synth_nn_state
from oracle.evoformer_ref import OracleModel

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "evoformer_nn_golden.npz")
KW = dict(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128, c_hidden_pair_att=32, c_s=384,
          no_heads_msa=8, no_heads_pair=4, transition_n=4, msa_dropout=0.15, pair_dropout=0.25, blocks_per_ckpt=1,
          inf=1e9, eps=1e-8)


def _oracle(seed, nb, fis=True, std=0.02):
    model = OracleModel(no_blocks=nb, **KW).eval()
    sd = synth_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis, std=std)
    model.evoformer.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return model


def _fast(model, dev, dtype):
    import copy
    from fastfold_amd.utils.inject_fastnn import inject_fastnn
    m2 = inject_fastnn(copy.deepcopy(model))
    return m2.evoformer.to(device=dev, dtype=dtype).eval()


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def _t(x, dev, dtype):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev, dtype)


def _f(t):
    return t.detach().float().cpu().numpy()


SUBMODULES = ["row", "col", "mtrans", "opm", "tmo", "tmi", "tas", "tae", "ptrans"]


def _oracle_sub(blk, name, m, z, mm, pm):
    c = blk.core
    with torch.no_grad():
        if name == "row":
            return "m", blk.msa_att_row(m, z=z, mask=mm)
        if name == "col":
            return "m", blk.msa_att_col(m, mask=mm)
        if name == "mtrans":
            return "m", c.msa_transition(m, mask=None)
        if name == "opm":
            return "z", c.outer_product_mean(m, mask=mm)
        if name == "tmo":
            return "z", c.tri_mul_out(z, mask=pm)
        if name == "tmi":
            return "z", c.tri_mul_in(z, mask=pm)
        if name == "tas":
            return "z", c.tri_att_start(z, mask=pm)
        if name == "tae":
            return "z", c.tri_att_end(z, mask=pm)
        return "z", c.pair_transition(z, mask=None)


def _fast_sub(blk, name, m, z, mm, pm):
    with torch.no_grad():
        if name == "row":
            return blk.msa.MSARowAttentionWithPairBias(m, z, mm) - m
        if name == "col":
            return blk.msa.MSAColumnAttention(m, mm) - m
        if name == "mtrans":
            return blk.msa.MSATransition(m) - m
        if name == "opm":
            return blk.communication(m, mm, z) - z
        if name == "tmo":
            return blk.pair.TriangleMultiplicationOutgoing(z, pm) - z
        if name == "tmi":
            return blk.pair.TriangleMultiplicationIncoming(z, pm) - z
        if name == "tas":
            return blk.pair.TriangleAttentionStartingNode(z, pm) - z
        if name == "tae":
            return blk.pair.TriangleAttentionEndingNode(z, pm) - z
        return blk.pair.PairTransition(z) - z


@pytest.mark.parametrize("s,r,tail", [(12, 40, 0.2), (33, 64, 0.0), (9, 21, 0.15)])
@pytest.mark.parametrize("name", SUBMODULES)
def test_submodule_updates_fp32(dev, name, s, r, tail):
    model = _oracle(21, 1)
    fast = _fast(model, dev, torch.float32)
    m, z, mm, pm = synth_inputs(7, s, r, mask_tail_frac=tail)
    which, ref = _oracle_sub(model.evoformer.blocks[0], name, *(torch.from_numpy(t) for t in (m, z, mm, pm)))
    got = _fast_sub(fast.blocks[0], name, _t(m[None], dev, torch.float32), _t(z[None], dev, torch.float32),
                    _t(mm[None], dev, torch.float32), _t(pm[None], dev, torch.float32))[0]
    ref = ref.numpy()
    # padded query rows are garbage by construction in both implementations: compare valid rows
    nv = r - int(round(tail * r))
    if which == "m":
        got, ref = _f(got)[:, :nv], ref[:, :nv]
    else:
        got, ref = _f(got)[:nv, :nv], ref[:nv, :nv]
    scale = max(1.0, float(np.abs(ref).max()))
    assert np.abs(got - ref).max() <= 1e-4 * scale, (name, np.abs(got - ref).max(), scale)


@pytest.mark.parametrize("s,r,tail", [(16, 48, 0.1), (128, 64, 0.1), (64, 96, 0.0)])
@pytest.mark.parametrize("name", SUBMODULES)
def test_submodule_updates_bf16(dev, name, s, r, tail):
    model = _oracle(22, 1)
    fast = _fast(model, dev, torch.bfloat16)
    m, z, mm, pm = synth_inputs(8, s, r, mask_tail_frac=tail)
    # feed the oracle the bf16-rounded inputs so only arithmetic differs
    mb, zb = (_f(_t(x, dev, torch.bfloat16)) for x in (m, z))
    which, ref = _oracle_sub(model.evoformer.blocks[0], name, torch.from_numpy(mb), torch.from_numpy(zb),
                             torch.from_numpy(mm), torch.from_numpy(pm))
    inp = _t(mb[None], dev, torch.bfloat16) if which == "m" else _t(zb[None], dev, torch.bfloat16)
    out = _fast_sub(fast.blocks[0], name, _t(mb[None], dev, torch.bfloat16), _t(zb[None], dev, torch.bfloat16),
                    _t(mm[None], dev, torch.bfloat16), _t(pm[None], dev, torch.bfloat16))[0]
    nv = r - int(round(tail * r))
    ref = ref.numpy()
    base = mb if which == "m" else zb
    if which == "m":
        got, ref, base = _f(out)[:, :nv], ref[:, :nv], base[:, :nv]
    else:
        got, ref, base = _f(out)[:nv, :nv], ref[:nv, :nv], base[:nv, :nv]
    # the module rounds (in + update) to bf16: allow that rounding of the sum on top of 2e-2 of the update
    err = np.linalg.norm(got - ref)
    bound = 2e-2 * np.linalg.norm(ref) + 2.0 ** -8 * np.linalg.norm(base + ref)
    assert err <= bound, (name, err, bound)


def test_golden_vectors_fp32(dev):
    """The reference's own outputs (written by fastfold.model.nn in the build container)."""
    g = np.load(GOLDEN)
    for name in sorted({k.split(".")[0] for k in g.files}):
        seed, nb, s, r, tail, fis = (int(v) for v in g[name + ".cfg"])
        fast = _fast(_oracle(seed, nb, bool(fis)), dev, torch.float32)
        m, z, mm, pm = synth_inputs(seed, s, r, mask_tail_frac=tail / 100)
        with torch.no_grad():
            mo, zo, so = fast(*(_t(x, dev, torch.float32) for x in (m, z, mm, pm)), chunk_size=None)
        nv = r - int(round(tail / 100 * r))
        for got, ref in ((_f(mo)[:, :nv], g[name + ".m"][:, :nv]), (_f(zo)[:nv, :nv], g[name + ".z"][:nv, :nv]),
                         (_f(so)[:nv], g[name + ".s"][:nv])):
            scale = max(1.0, float(np.abs(ref).max()))
            assert np.abs(got - ref).max() <= 1e-4 * scale, (name, np.abs(got - ref).max(), scale)


def test_config1_block_fp32(dev):
    """Benchmark configuration 1: one block, fp32, s=32, r=64, weights N(0, 0.02^2): max-abs <= 1e-4."""
    model = _oracle(1, 1, fis=False)
    fast = _fast(model, dev, torch.float32)
    m, z, mm, pm = synth_inputs(1, 32, 64)
    with torch.no_grad():
        rm, rz, rs = model.evoformer(*(torch.from_numpy(t) for t in (m, z, mm, pm)), _mask_trans=False)
        inputs = [_t(x, dev, torch.float32) for x in (m, z, mm, pm)]
        keep = [t.clone() for t in inputs]
        gm, gz, gs = fast(*inputs, chunk_size=None)
    assert all(torch.equal(a, b) for a, b in zip(inputs, keep)), "forward must not modify its inputs"
    assert np.abs(_f(gm) - rm.numpy()).max() <= 1e-4
    assert np.abs(_f(gz) - rz.numpy()).max() <= 1e-4
    assert np.abs(_f(gs) - rs.numpy()).max() <= 1e-4
    # in-place list-passing variant gives the same result and overwrites its lists
    ml, zl = [inputs[0].clone()], [inputs[1].clone()]
    with torch.no_grad():
        ml, zl, s2 = fast.inplace(ml, zl, inputs[2], inputs[3], chunk_size=None)
    assert torch.equal(ml[0], gm) and torch.equal(zl[0], gz) and torch.equal(s2, gs)


def test_block_interface_padding_and_chaining(dev):
    """first / middle / last stand-alone blocks chained the reference way carry [1, s, r+1, c]."""
    from fastfold_amd.model.fastnn import Evoformer
    model = _oracle(3, 3)
    fast = _fast(model, dev, torch.float32)
    s, r = 10, 24
    m, z, mm, pm = synth_inputs(3, s, r, mask_tail_frac=0.1)
    tm, tz, tmm, tpm = (_t(x, dev, torch.float32) for x in (m, z, mm, pm))
    with torch.no_grad():
        sm, sz, _ = fast(tm, tz, tmm, tpm, chunk_size=None)
        a, b = fast.blocks[0](tm, tz, tmm, tpm)
        assert a.shape == (1, s, r + 1, 256) and b.shape == (1, r + 1, r + 1, 128)
        a, b = fast.blocks[1](a, b, tmm, tpm)
        assert a.shape == (1, s, r + 1, 256) and b.shape == (1, r + 1, r + 1, 128)
        a, b = fast.blocks[2](a, b, tmm, tpm)
    assert a.shape == (s, r, 256) and b.shape == (r, r, 128)
    assert torch.equal(a, sm) and torch.equal(b, sz)
    assert isinstance(fast.blocks[0], Evoformer)


@pytest.mark.parametrize("extended", [True, False])
@pytest.mark.parametrize("nb,s,r,tail", [(4, 24, 72, 0.1)])
def test_stack_bf16_rel_l2(dev, nb, s, r, tail, extended):
    """bf16 stack vs fp32 oracle: relative L2 <= 2e-2 on m and z (north star), O(1) updates; with the extended
    residual stream (the default) and with the reference's plain bf16 stream (the switch bench.py --plain-residual uses)."""
    model = _oracle(31, nb)
    fast = _fast(model, dev, torch.bfloat16)
    fast.extended_residual = extended
    m, z, mm, pm = synth_inputs(31, s, r, mask_tail_frac=tail)
    mb, zb = (_f(_t(x, dev, torch.bfloat16)) for x in (m, z))
    with torch.no_grad():
        rm, rz, rs = model.evoformer(torch.from_numpy(mb), torch.from_numpy(zb), torch.from_numpy(mm),
                                     torch.from_numpy(pm), _mask_trans=False)
        gm, gz, gs = fast(*(_t(x, dev, torch.bfloat16) for x in (mb, zb, mm, pm)), chunk_size=None)
    nv = r - int(round(tail * r))
    assert _rel_l2(_f(gm)[:, :nv], rm.numpy()[:, :nv]) <= 2e-2
    assert _rel_l2(_f(gz)[:nv, :nv], rz.numpy()[:nv, :nv]) <= 2e-2
    assert _rel_l2(_f(gs)[:nv], rs.numpy()[:nv]) <= 2e-2


def test_state_dict_keys_and_cpu_error(dev):
    from fastfold_amd.model.fastnn import EvoformerStack
    st = EvoformerStack(c_m=256, c_z=128, c_s=384, no_blocks=1, blocks_per_ckpt=1)
    keys = set(st.state_dict().keys())
    for k in ("blocks.0.msa.MSARowAttentionWithPairBias.linear_b_weights",
              "blocks.0.msa.MSARowAttentionWithPairBias.attention.to_qkv.weight",
              "blocks.0.msa.MSAColumnAttention.attention.o_linear.bias",
              "blocks.0.communication.o_linear.weight",
              "blocks.0.pair.TriangleMultiplicationIncoming.left_right_gate.bias",
              "blocks.0.pair.TriangleAttentionEndingNode.out_bias",
              "blocks.0.pair.PairTransition.linear2.weight", "linear.weight", "linear.bias"):
        assert k in keys, k
    with pytest.raises(RuntimeError):
        with torch.no_grad():
            st(torch.zeros(4, 8, 256), torch.zeros(8, 8, 128), torch.ones(4, 8), torch.ones(8, 8), chunk_size=None)


@pytest.mark.parametrize("s,r,tail", [(1, 1, 0.0), (2, 1, 0.0), (1, 17, 0.0), (5, 8, 0.25), (129, 33, 0.1), (7, 130, 0.3)])
def test_stack_extreme_shapes(dev, s, r, tail):
    """Degenerate and ragged sizes (a single sequence, a single residue, sizes just past a tile edge) through a
    two-block stack, both precisions, against the oracle."""
    model = _oracle(5, 2)
    m, z, mm, pm = synth_inputs(3, s, r, mask_tail_frac=tail)
    with torch.no_grad():
        rm, rz, rs = model.evoformer(*(torch.from_numpy(x) for x in (m, z, mm, pm)), chunk_size=None, _mask_trans=False)
    nv = r - int(round(tail * r))
    rm, rz, rs = rm.numpy()[:, :nv], rz.numpy()[:nv, :nv], rs.numpy()[:nv]
    for dtype in (torch.float32, torch.bfloat16):
        fast = _fast(model, dev, dtype)
        with torch.no_grad():
            gm, gz, gs = fast(*(_t(x, dev, dtype) for x in (m, z, mm, pm)), chunk_size=None, _mask_trans=False)
        gm, gz, gs = _f(gm)[:, :nv], _f(gz)[:nv, :nv], _f(gs)[:nv]
        if dtype == torch.float32:
            for g, ref in ((gm, rm), (gz, rz), (gs, rs)):
                assert np.abs(g - ref).max() <= 1e-4 * max(1.0, float(np.abs(ref).max()))
        else:
            assert _rel_l2(gm, rm) <= 2e-2 and _rel_l2(gz, rz) <= 2e-2 and _rel_l2(gs, rs) <= 2e-2
