"""Pins the CPU oracle (oracle/) - no GPU, no product code under test.

* golden vectors written by the reference's own fastfold.model.nn Evoformer (tests/golden/)
* library routines (torch.softmax, F.layer_norm, F.linear) and float64 brute force
* invariants: identity at default init, permutation equivariance, masked-key invariance
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fastfold_amd.synthetic import synth_inputs, synth_nn_state
from oracle import ops_np
from oracle.evoformer_ref import EvoformerStack

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "evoformer_nn_golden.npz")


def _stack(seed, nb, fis=True, std=0.02):
    st = EvoformerStack(no_blocks=nb).eval()
    sd = synth_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis, std=std)
    st.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return st


def _run(st, m, z, mm, pm):
    with torch.no_grad():
        return [t.numpy() for t in st(*(torch.from_numpy(np.ascontiguousarray(t)) for t in (m, z, mm, pm)),
                                      _mask_trans=False)]


def test_golden_vectors_from_reference():
    g = np.load(GOLDEN)
    names = sorted({k.split(".")[0] for k in g.files})
    assert len(names) == 3
    for name in names:
        seed, nb, s, r, tail, fis = (int(v) for v in g[name + ".cfg"])
        st = _stack(seed, nb, bool(fis))
        m, z, mm, pm = synth_inputs(seed, s, r, mask_tail_frac=tail / 100)
        mo, zo, so = _run(st, m, z, mm, pm)
        # same arithmetic, possibly different op order: fp32 round-off only
        assert np.abs(mo - g[name + ".m"]).max() < 2e-5, name
        assert np.abs(zo - g[name + ".z"]).max() < 2e-4, name
        assert np.abs(so - g[name + ".s"]).max() < 2e-5, name


def test_default_init_block_is_identity():
    # every update ends in a zero-initialised ("final") layer: nn/primitives.py:164-165
    torch.manual_seed(0)
    st = EvoformerStack(no_blocks=2).eval()
    m, z, mm, pm = synth_inputs(3, 4, 7)
    mo, zo, _ = _run(st, m, z, mm, pm)
    assert np.array_equal(mo, m) and np.array_equal(zo, z)


def test_permutation_equivariance():
    st = _stack(5, 1)
    m, z, mm, pm = synth_inputs(5, 6, 9, mask_tail_frac=0.2)
    mo, zo, _ = _run(st, m, z, mm, pm)
    ps = np.random.RandomState(0).permutation(6)
    pr = np.random.RandomState(1).permutation(9)
    mo2, zo2, _ = _run(st, m[ps][:, pr], z[pr][:, pr], mm[ps][:, pr], pm[pr][:, pr])
    assert np.abs(mo2 - mo[ps][:, pr]).max() < 1e-4
    assert np.abs(zo2 - zo[pr][:, pr]).max() < 1e-3


def test_masked_positions_do_not_leak():
    st = _stack(6, 1)
    m, z, mm, pm = synth_inputs(6, 5, 10, mask_tail_frac=0.3)
    mo, zo, _ = _run(st, m, z, mm, pm)
    m2, z2 = m.copy(), z.copy()
    m2[:, 7:] += 3.0
    z2[7:, :] -= 2.0
    z2[:, 7:] += 1.5
    mo2, zo2, _ = _run(st, m2, z2, mm, pm)
    assert np.abs(mo2[:, :7] - mo[:, :7]).max() < 1e-4
    assert np.abs(zo2[:7, :7] - zo[:7, :7]).max() < 1e-3


def test_ops_np_softmax_layernorm_linear_against_torch():
    rng = np.random.RandomState(0)
    x = rng.standard_normal((1, 3, 2, 5, 7)).astype(np.float32)
    bias = rng.standard_normal((1, 1, 2, 5, 7)).astype(np.float32)
    mask = (rng.uniform(size=(1, 3, 7)) > 0.3).astype(np.float32)
    mask[..., 0] = 1
    ref = torch.softmax(torch.from_numpy(x) + torch.from_numpy(bias)
                        + 1e9 * (torch.from_numpy(mask) - 1)[:, :, None, None, :], -1).numpy()
    got = ops_np.fused_softmax(x, mask, bias)
    assert np.abs(got - ref).max() < 1e-6
    assert np.allclose(got.sum(-1), 1.0) and np.all(got[np.broadcast_to(mask[:, :, None, None, :] == 0, got.shape)] == 0)
    # shift invariance
    assert np.abs(ops_np.fused_softmax(x.astype(np.float64) + 3.0, mask, bias) - got).max() < 1e-12
    xx = rng.standard_normal((11, 129)).astype(np.float32)
    gm, bt = rng.standard_normal(129).astype(np.float32), rng.standard_normal(129).astype(np.float32)
    ref = F.layer_norm(torch.from_numpy(xx).double(), (129,), torch.from_numpy(gm).double(),
                       torch.from_numpy(bt).double(), 1e-5).numpy()
    assert np.abs(ops_np.layer_norm(xx, gm, bt) - ref).max() < 1e-12
    y = ops_np.layer_norm(xx, np.ones(129), np.zeros(129), eps=0.0)
    assert np.abs(y.mean(-1)).max() < 1e-12 and np.abs(y.var(-1) - 1).max() < 1e-9
    w = rng.standard_normal((5, 129)).astype(np.float32)
    assert np.abs(ops_np.linear(xx, w, bt[:5]) - F.linear(torch.from_numpy(xx).double(), torch.from_numpy(w).double(),
                                                          torch.from_numpy(bt[:5]).double()).numpy()).max() < 1e-12


def test_ops_np_attention_and_contractions_brute_force():
    rng = np.random.RandomState(1)
    b2, h, n, d = 2, 3, 5, 4
    q, k, v = (rng.standard_normal((1, b2, h, n, d)) for _ in range(3))
    bias = rng.standard_normal((1, h, n, n))
    mask = np.ones((1, b2, n))
    mask[0, 1, 3] = 0
    got = ops_np.attention_core(q, k, v, mask, bias)
    for b in range(b2):
        for hh in range(h):
            for i in range(n):
                lg = np.array([q[0, b, hh, i] @ k[0, b, hh, j] / np.sqrt(d) + bias[0, hh, i, j] for j in range(n)])
                lg[mask[0, b] == 0] = -np.inf
                w = np.exp(lg - lg.max())
                w /= w.sum()
                o = sum(w[j] * v[0, b, hh, j] for j in range(n))
                assert np.abs(got[0, b, i, hh * d:(hh + 1) * d] - o).max() < 1e-12
    a, bb = rng.standard_normal((4, 5, 3)), rng.standard_normal((4, 5, 3))
    po = ops_np.trimul_outgoing(a, bb)
    pi = ops_np.trimul_incoming(a.transpose(1, 0, 2), bb.transpose(1, 0, 2))
    for i in range(4):
        for j in range(4):
            for c in range(3):
                assert abs(po[i, j, c] - sum(a[i, kk, c] * bb[j, kk, c] for kk in range(5))) < 1e-12
    assert np.abs(po - pi).max() < 1e-12        # incoming(z) == outgoing on transposed operands
    la, lb = rng.standard_normal((6, 3, 2)), rng.standard_normal((6, 4, 5))
    o = ops_np.outer_product(la, lb)
    assert o.shape == (3, 4, 10)
    assert abs(o[2, 3, 1 * 5 + 4] - sum(la[s, 2, 1] * lb[s, 3, 4] for s in range(6))) < 1e-12


def test_ops_np_elementwise_closed_forms():
    rng = np.random.RandomState(2)
    y, z, r = (rng.standard_normal((2, 3, 4, 8)) for _ in range(3))
    b = rng.standard_normal(8)
    assert np.abs(ops_np.bias_sigmod_ele(y, b, z) - (torch.sigmoid(torch.from_numpy(y + b)) * torch.from_numpy(z)).numpy()).max() < 1e-12
    dm = np.ones((2, 1, 4, 8))
    assert np.abs(ops_np.bias_dropout_add(y, b, dm, r) - (r + y + b)).max() < 1e-12
    assert np.abs(ops_np.bias_ele_dropout_residual(y, b, z, dm, r) - (r + z * (y + b))).max() < 1e-12
    dy = rng.standard_normal((3, 9))
    yy = ops_np.fused_softmax(rng.standard_normal((1, 1, 1, 3, 9)))[0, 0, 0]
    xt = torch.from_numpy(np.log(yy)).requires_grad_(True)
    torch.softmax(xt, -1).backward(torch.from_numpy(dy))
    assert np.abs(ops_np.softmax_bwd(dy, yy) - xt.grad.numpy()).max() < 1e-10
