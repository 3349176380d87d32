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


# ------------------------------------------------------------------ extra-MSA stack ----
EXTRA_GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "extra_msa_nn_golden.npz")


def _extra_stack(seed, nb, fis=True):
    from fastfold_amd.synthetic import synth_extra_nn_state
    from oracle.evoformer_ref import ExtraMSAStack
    st = ExtraMSAStack(no_blocks=nb).eval()
    sd = synth_extra_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis)
    st.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return st


def test_extra_msa_golden_vectors_from_reference():
    g = np.load(EXTRA_GOLDEN)
    names = sorted({k.split(".")[0] for k in g.files})
    assert len(names) == 3
    for name in names:
        seed, nb, s, r, tail, fis = (int(v) for v in g[name + ".cfg"])
        st = _extra_stack(seed, nb, bool(fis))
        m, z, mm, pm = synth_inputs(seed, s, r, c_m=64, mask_tail_frac=tail / 100)
        with torch.no_grad():
            zo = st(torch.from_numpy(m), torch.from_numpy(z), msa_mask=torch.from_numpy(mm),
                    pair_mask=torch.from_numpy(pm)).numpy()
        ref = g[name + ".z"]
        assert np.abs(zo - ref).max() <= 2e-5 * max(1.0, np.abs(ref).max()), name


def test_global_attention_brute_force():
    # float64 loops over the published formula (one query per column, shared key / value head)
    from oracle.evoformer_ref import GlobalAttention
    torch.manual_seed(3)
    ga = GlobalAttention(12, 4, 3, inf=1e9, eps=1e-10).double()
    with torch.no_grad():
        for p in ga.parameters():
            p.copy_(torch.randn_like(p) * 0.5)
    rng = np.random.RandomState(4)
    R, S = 3, 6
    m = rng.standard_normal((R, S, 12))
    mask = np.ones((R, S))
    mask[1, 2:4] = 0
    with torch.no_grad():
        got = ga(torch.from_numpy(m), torch.from_numpy(mask)).numpy()
    P = {k: v.detach().numpy() for k, v in ga.named_parameters()}
    for j in range(R):
        qa = sum(mask[j, s] * m[j, s] for s in range(S)) / (mask[j].sum() + 1e-10)
        q = (P["linear_q.weight"] @ qa).reshape(3, 4) / 2.0
        k = [P["linear_k.weight"] @ m[j, s] for s in range(S)]
        v = [P["linear_v.weight"] @ m[j, s] for s in range(S)]
        o = np.zeros((3, 4))
        for h in range(3):
            lg = np.array([q[h] @ k[s] if mask[j, s] else -np.inf for s in range(S)])
            w = np.exp(lg - lg.max())
            w /= w.sum()
            o[h] = sum(w[s] * v[s] for s in range(S))
        for s in range(S):
            gate = 1.0 / (1.0 + np.exp(-(P["linear_g.weight"] @ m[j, s] + P["linear_g.bias"])))
            out = P["linear_o.weight"] @ (gate * o.reshape(-1)) + P["linear_o.bias"]
            assert np.abs(out - got[j, s]).max() < 1e-10


def test_extra_msa_default_init_is_identity_and_masked_positions_do_not_leak():
    from oracle.evoformer_ref import ExtraMSAStack
    torch.manual_seed(0)
    st = ExtraMSAStack(no_blocks=2).eval()
    m, z, mm, pm = synth_inputs(8, 5, 7, c_m=64)
    with torch.no_grad():
        zo = st(torch.from_numpy(m), torch.from_numpy(z), msa_mask=torch.from_numpy(mm), pair_mask=torch.from_numpy(pm))
    assert np.array_equal(zo.numpy(), z)
    st = _extra_stack(9, 1)
    m, z, mm, pm = synth_inputs(9, 6, 10, c_m=64, mask_tail_frac=0.3)
    m2, z2 = m.copy(), z.copy()
    m2[:, 7:] += 3.0
    z2[7:, :] -= 2.0
    z2[:, 7:] += 1.5
    outs = []
    for mt in (True, False):          # masked transitions only change masked positions
        for mi, zi in ((m, z), (m2, z2)):
            with torch.no_grad():
                outs.append(st(torch.from_numpy(mi), torch.from_numpy(zi), msa_mask=torch.from_numpy(mm),
                               pair_mask=torch.from_numpy(pm), _mask_trans=mt).numpy()[:7, :7])
    for o in outs[1:]:
        assert np.abs(o - outs[0]).max() < 1e-3


# -------------------------------------------------------------- template pair stack ----
TEMPLATE_GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "template_pair_nn_golden.npz")


def test_template_pair_stack_golden_vectors_from_reference():
    from fastfold_amd.synthetic import synth_template_inputs, synth_template_nn_state
    from oracle.evoformer_ref import TemplatePairStack
    g = np.load(TEMPLATE_GOLDEN)
    names = sorted({k.split(".")[0] for k in g.files})
    assert len(names) == 3
    for name in names:
        seed, nb, nt, r, tail, fis = (int(v) for v in g[name + ".cfg"])
        st = TemplatePairStack(no_blocks=nb).eval()
        sd = synth_template_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=bool(fis))
        st.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
        t, pm = synth_template_inputs(seed, nt, r, mask_tail_frac=tail / 100)
        with torch.no_grad():
            to = st(torch.from_numpy(t), torch.from_numpy(pm)[None], _mask_trans=False).numpy()
        assert np.abs(to - g[name + ".t"]).max() <= 2e-5, name


# ------------------------------------------------------------------------ embedders ----
def test_embedders_brute_force():
    """No golden vectors here: the reference's nn/embedders.py imports dm-tree, which this image lacks.
    A linear layer on a one-hot vector is a column pick, so both embedders have closed forms that the
    float64 loops below restate independently (indices by explicit comparison, not by one_hot)."""
    from oracle.evoformer_ref import InputEmbedder, RecyclingEmbedder
    torch.manual_seed(0)
    ie = InputEmbedder(tf_dim=22, msa_dim=49, c_z=16, c_m=24, relpos_k=4).double()
    with torch.no_grad():
        for p in ie.parameters():
            p.copy_(torch.randn_like(p))
    rng = np.random.RandomState(0)
    r, s = 9, 3
    tf, msa = rng.standard_normal((r, 22)), rng.standard_normal((s, r, 49))
    ri = np.array([0, 1, 2, 3, 10, 11, 12, 40, 41], dtype=np.float64)      # gaps beyond the +-4 window
    with torch.no_grad():
        m_emb, z_emb = (t.numpy() for t in ie(torch.from_numpy(tf), torch.from_numpy(ri), torch.from_numpy(msa)))
    P = {k: v.detach().numpy() for k, v in ie.named_parameters()}
    for i in range(r):
        for j in range(r):
            b = int(min(max(ri[i] - ri[j], -4), 4)) + 4
            want = (P["linear_tf_z_i.weight"] @ tf[i] + P["linear_tf_z_i.bias"] + P["linear_tf_z_j.weight"] @ tf[j]
                    + P["linear_tf_z_j.bias"] + P["linear_relpos.weight"][:, b] + P["linear_relpos.bias"])
            assert np.abs(z_emb[i, j] - want).max() < 1e-10
        for q in range(s):
            want = (P["linear_msa_m.weight"] @ msa[q, i] + P["linear_msa_m.bias"] + P["linear_tf_m.weight"] @ tf[i]
                    + P["linear_tf_m.bias"])
            assert np.abs(m_emb[q, i] - want).max() < 1e-10
    re_ = RecyclingEmbedder(c_m=24, c_z=16, min_bin=3.25, max_bin=20.75, no_bins=15).double()
    with torch.no_grad():
        for p in re_.parameters():
            p.copy_(torch.randn_like(p))
    x = rng.standard_normal((r, 3)) * 8.0
    x[1] = x[0] + np.array([3.25, 0.0, 0.0])       # exactly on the first edge: no bin
    m, z = rng.standard_normal((r, 24)), rng.standard_normal((r, r, 16))
    with torch.no_grad():
        mu, zu = (t.numpy() for t in re_(torch.from_numpy(m), torch.from_numpy(z), torch.from_numpy(x)))
    P = {k: v.detach().numpy() for k, v in re_.named_parameters()}
    edges = np.linspace(3.25, 20.75, 15)

    def ln(v, g, b):
        return (v - v.mean()) / np.sqrt(v.var() + 1e-5) * g + b
    none_hit = 0
    for i in range(r):
        assert np.abs(mu[i] - ln(m[i], P["layer_norm_m.weight"], P["layer_norm_m.bias"])).max() < 1e-10
        for j in range(r):
            d2 = float(((x[i] - x[j]) ** 2).sum())
            hit = [b for b in range(15) if d2 > edges[b] ** 2 and d2 < (edges[b + 1] ** 2 if b < 14 else 1e8)]
            assert len(hit) <= 1
            none_hit += not hit
            want = ln(z[i, j], P["layer_norm_z.weight"], P["layer_norm_z.bias"]) + P["linear.bias"]
            if hit:
                want = want + P["linear.weight"][:, hit[0]]
            assert np.abs(zu[i, j] - want).max() < 1e-10
    assert none_hit >= r + 2        # the diagonal and the pair on the edge


def test_template_pointwise_golden_and_brute_force():
    """The point-wise template attention against the reference's vectors (tests/golden/make_golden.py pointwise)
    and against float64 loops over positions, heads and templates."""
    from fastfold_amd.synthetic import synth_pointwise_inputs, synth_pointwise_nn_state
    from oracle.evoformer_ref import TemplatePointwiseAttention
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "template_pointwise_nn_golden.npz"))
    names = sorted(k[:-4] for k in g.files if k.endswith(".cfg"))
    assert len(names) == 4
    for name in names:
        cfg = g[name + ".cfg"]
        seed, nt, r, tmask = int(cfg[0]), int(cfg[1]), int(cfg[2]), [float(x) for x in cfg[3:]]
        mod = TemplatePointwiseAttention().eval()
        sd = synth_pointwise_nn_state(seed=seed)
        mod.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
        t, z = synth_pointwise_inputs(seed, nt, r)
        with torch.no_grad():
            out = mod(torch.from_numpy(t), torch.from_numpy(z), template_mask=torch.tensor(tmask)).numpy()
        assert np.abs(out - g[name + ".out"]).max() <= 2e-5, name
        # brute force on a few positions (not when every template is masked: the reference adds -1e5 to the fp32
        # logits there, which rounds them to multiples of 2^-7; that case is pinned by the vectors alone)
        if sum(tmask) == 0:
            continue
        W = {k: v.astype(np.float64) for k, v in sd.items()}
        H, D = 4, 16
        for (i, j) in ((0, 0), (r - 1, 2), (3, r - 1)):
            q = (W["mha.linear_q.weight"] @ z[i, j].astype(np.float64)) / np.sqrt(D)
            o = np.zeros(H * D)
            for h in range(H):
                logit = np.array([q[h * D:(h + 1) * D] @ (W["mha.linear_k.weight"] @ t[n, i, j].astype(np.float64))[h * D:(h + 1) * D]
                                  + 1e5 * (tmask[n] - 1) for n in range(nt)])
                w = np.exp(logit - logit.max())
                w /= w.sum()
                for n in range(nt):
                    o[h * D:(h + 1) * D] += w[n] * (W["mha.linear_v.weight"] @ t[n, i, j].astype(np.float64))[h * D:(h + 1) * D]
            ref = W["mha.linear_o.weight"] @ o + W["mha.linear_o.bias"]
            assert np.abs(out[i, j] - ref).max() <= 1e-4, (name, i, j)
