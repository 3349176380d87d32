"""AlphaFold-2 parameter ingestion (fastfold_amd/utils/import_weights.py), CPU only.

No AF2 checkpoint exists offline, so the importer is pinned (a) against AlphaFold's own use of each
array - the einsum conventions of its haiku modules, restated below - and (b) by a round trip through a
synthetic AF2-layout file built from a seeded nn-layout state."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fastfold_amd.synthetic import synth_nn_state
from fastfold_amd.utils import import_weights as iw
from fastfold_amd.utils.inject_fastnn import convert_nn_state_dict

P = iw.NPZ_PREFIX + "evoformer/"


def _to_jax_layout(sd, nb):
    """Inverse of the importer: nn-layout arrays -> AF2 arrays stacked over blocks (test-side only)."""
    heads = {"msa_att_row": 8, "msa_att_col": 8, "tri_att_start": 4, "tri_att_end": 4}
    out = {}
    for key, dst, fn in iw.block_translation():
        per_block = []
        for i in range(nb):
            w = np.asarray(sd["blocks.%d.%s" % (i, dst)])
            H = next((h for n, h in heads.items() if n in dst), None)
            if fn is iw._linear_weight:
                a = w.T
            elif fn is iw._linear_weight_mha:                 # [H*d, in] -> [in, H, d]
                a = w.T.reshape(w.shape[1], H, -1)
            elif fn is iw._mha_output_weight and "outer_product" in dst:   # [c_z, c*c] -> [c, c, c_z]
                c = int(round(w.shape[1] ** 0.5))
                a = w.T.reshape(c, c, w.shape[0])
            elif fn is iw._mha_output_weight:                 # [out, H*d] -> [H, d, out]
                a = w.T.reshape(H, -1, w.shape[0])
            elif fn is iw._linear_bias_mha:                   # [H*d] -> [H, d]
                a = w.reshape(H, -1)
            else:
                a = w
            per_block.append(a)
        out[P + "evoformer_iteration/" + key] = np.stack(per_block, 0)
    out[P + "single_activations//weights"] = np.asarray(sd["linear.weight"]).T
    out[P + "single_activations//bias"] = np.asarray(sd["linear.bias"])
    return out


def test_array_conventions_match_alphafold_einsums():
    """AlphaFold applies its arrays as  q = einsum('bqa,ahc->bqhc', x, query_w),
    out = einsum('bqhc,hco->bqo', o, output_w) + output_b,  gate = einsum('bqc,chv->bqhv', x, gating_w) + gating_b,
    y = x @ weights + bias  and  opm = einsum('...ce,cez->...z', outer, output_w): the imported tensors must
    give the same numbers through F.linear and the [heads * head_dim] feature order of this package."""
    g = np.random.RandomState(0)
    x = g.randn(2, 5, 12)
    H, d = 3, 4
    qw = g.randn(12, H, d)
    q = F.linear(torch.from_numpy(x), torch.from_numpy(np.ascontiguousarray(iw._linear_weight_mha(qw)))).numpy()
    assert np.allclose(q.reshape(2, 5, H, d), np.einsum("bqa,ahc->bqhc", x, qw))
    o = g.randn(2, 5, H, d)
    ow, ob = g.randn(H, d, 7), g.randn(7)
    y = F.linear(torch.from_numpy(o.reshape(2, 5, H * d)), torch.from_numpy(np.ascontiguousarray(iw._mha_output_weight(ow))),
                 torch.from_numpy(ob)).numpy()
    assert np.allclose(y, np.einsum("bqhc,hco->bqo", o, ow) + ob)
    gb = g.randn(H, d)
    assert np.allclose(iw._linear_bias_mha(gb).reshape(H, d), gb)
    w = g.randn(12, 9)
    assert np.allclose(F.linear(torch.from_numpy(x), torch.from_numpy(np.ascontiguousarray(iw._linear_weight(w)))).numpy(), x @ w)
    outer = g.randn(4, 6, 5, 5)                                   # [..., c (left), e (right)]
    opw = g.randn(5, 5, 8)
    z = F.linear(torch.from_numpy(outer.reshape(4, 6, 25)), torch.from_numpy(np.ascontiguousarray(iw._opm_weight(opw)))).numpy()
    assert np.allclose(z, np.einsum("abce,cez->abz", outer, opw))


def test_key_names_and_shapes():
    nb = 2
    jax = _to_jax_layout(synth_nn_state(seed=3, no_blocks=nb), nb)
    it = P + "evoformer_iteration/"
    # haiku separates module path and parameter name with a double slash (import_weights.py:61-76)
    assert jax[it + "msa_row_attention_with_pair_bias/attention//query_w"].shape == (nb, 256, 8, 32)
    assert jax[it + "msa_row_attention_with_pair_bias/attention//output_w"].shape == (nb, 8, 32, 256)
    assert jax[it + "msa_row_attention_with_pair_bias/attention//gating_b"].shape == (nb, 8, 32)
    assert jax[it + "msa_row_attention_with_pair_bias//feat_2d_weights"].shape == (nb, 128, 8)
    assert jax[it + "triangle_attention_ending_node/attention//key_w"].shape == (nb, 128, 4, 32)
    assert jax[it + "outer_product_mean//output_w"].shape == (nb, 32, 32, 128)
    assert jax[it + "triangle_multiplication_incoming/left_projection//weights"].shape == (nb, 128, 128)
    assert jax[it + "pair_transition/transition1//weights"].shape == (nb, 128, 512)
    assert jax[P + "single_activations//weights"].shape == (256, 384)
    assert len(jax) == len(iw.block_translation()) + 2


def test_round_trip_and_incoming_swap():
    nb = 2
    sd = synth_nn_state(seed=5, no_blocks=nb)
    jax = _to_jax_layout(sd, nb)
    got = iw.evoformer_nn_state_dict_from_jax(jax)
    assert set(got) == set(sd)
    for k in sd:
        assert np.array_equal(got[k].numpy(), np.asarray(sd[k])), k
    # AlphaFold's "left" of the incoming update is the nn module's b projection (import_weights.py:222-236)
    left = jax[P + "evoformer_iteration/triangle_multiplication_incoming/left_projection//weights"][1]
    assert np.array_equal(left.T, np.asarray(sd["blocks.1.core.tri_mul_in.linear_b_p.weight"]))
    left = jax[P + "evoformer_iteration/triangle_multiplication_outgoing/left_projection//weights"][1]
    assert np.array_equal(left.T, np.asarray(sd["blocks.1.core.tri_mul_out.linear_a_p.weight"]))
    # errors: a missing array is named, a wrong block count is refused
    bad = dict(jax)
    del bad[P + "evoformer_iteration/pair_transition/transition2//bias"]
    with pytest.raises(KeyError, match="transition2//bias"):
        iw.evoformer_nn_state_dict_from_jax(bad)
    with pytest.raises(ValueError):
        iw.evoformer_nn_state_dict_from_jax(jax, no_blocks=3)


def test_import_into_fastnn_stack(tmp_path):
    from fastfold_amd.model.fastnn import EvoformerStack
    nb = 1
    sd = synth_nn_state(seed=7, no_blocks=nb)
    path = tmp_path / "params_model_x.npz"
    np.savez(path, **_to_jax_layout(sd, nb))
    stack = EvoformerStack(c_m=256, c_z=128, c_s=384, no_blocks=nb, blocks_per_ckpt=1)
    res = iw.import_jax_evoformer_(stack, str(path))
    assert not res.missing_keys and not res.unexpected_keys
    want = convert_nn_state_dict({k: torch.from_numpy(np.asarray(v)) for k, v in sd.items()})
    have = stack.state_dict()
    assert set(want) == set(have)
    for k, v in want.items():
        assert torch.equal(have[k], v.to(have[k].dtype)), k


def _af2_case(seed=9, nb=2, s=6, r=10):
    from oracle import af2_einsum_ref as af2
    from fastfold_amd.synthetic import synth_inputs
    params = af2.random_params(seed, nb)
    m, z, mm, pm = synth_inputs(seed, s, r, mask_tail_frac=0.2)
    return af2, params, m, z, mm, pm


def test_importer_against_alphafold_einsum_oracle():
    """Two independent routes from the same AlphaFold-layout arrays: AlphaFold's einsum conventions
    (oracle/af2_einsum_ref.py, float64, no translation table) and importer -> nn layout -> CPU oracle.  A wrong
    transposition, head split, left / right swap or key name in the importer's table breaks the agreement."""
    from oracle.evoformer_ref import EvoformerStack as OracleStack
    af2, params, m, z, mm, pm = _af2_case()
    want_m, want_z, want_s = af2.evoformer_stack(m, z, mm, pm, params)
    st = OracleStack(no_blocks=2).eval()
    st.load_state_dict(iw.evoformer_nn_state_dict_from_jax(params), strict=True)
    with torch.no_grad():
        gm, gz, gs = st(*(torch.from_numpy(t) for t in (m, z, mm, pm)), _mask_trans=False)
    nv = 8
    assert float(np.abs(want_z[:nv, :nv] - z[:nv, :nv]).mean()) > 0.3           # O(1) updates
    scale = float(np.abs(want_z).max())
    assert np.abs(gm.numpy() - want_m)[:, :nv].max() <= 1e-4 * scale
    assert np.abs(gz.numpy() - want_z)[:nv, :nv].max() <= 1e-4 * scale
    assert np.abs(gs.numpy() - want_s)[:nv].max() <= 1e-4 * scale


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_imported_weights_on_the_hip_path(dev, dtype, tmp_path):
    """A synthetic AlphaFold-layout ``.npz`` -> ``import_jax_evoformer_`` -> HIP forward, against AlphaFold's own
    einsum conventions applied to the same arrays (no real checkpoint exists offline)."""
    from fastfold_amd.model.fastnn import EvoformerStack
    from fastfold_amd.synthetic import bf16_round
    s, r, nv = 24, 40, 32
    af2, params, m, z, mm, pm = _af2_case(seed=10, nb=2, s=s, r=r)
    m, z = bf16_round(m), bf16_round(z)
    path = tmp_path / "params_model_synth.npz"
    np.savez(path, **params)
    stack = EvoformerStack(c_m=256, c_z=128, c_s=384, no_blocks=2, blocks_per_ckpt=1).to(dev, dtype).eval()
    res = iw.import_jax_evoformer_(stack, str(path))
    assert not res.missing_keys and not res.unexpected_keys
    want_m, want_z, want_s = af2.evoformer_stack(m, z, mm, pm, params)
    with torch.no_grad():
        gm, gz, gs = stack(*(torch.from_numpy(t).to(dev, dtype) for t in (m, z, mm, pm)), chunk_size=None)
    gm, gz, gs = (t.float().cpu().numpy() for t in (gm, gz, gs))
    if dtype == torch.float32:
        scale = float(np.abs(want_z).max())
        assert np.abs(gm - want_m)[:, :nv].max() <= 1e-4 * scale and np.abs(gz - want_z)[:nv, :nv].max() <= 1e-4 * scale
        assert np.abs(gs - want_s)[:nv].max() <= 1e-4 * scale
    else:
        def rel(a, b):
            return float(np.linalg.norm(a - b) / np.linalg.norm(b))
        assert rel(gm[:, :nv], want_m[:, :nv]) <= 2e-2 and rel(gz[:nv, :nv], want_z[:nv, :nv]) <= 2e-2
        assert rel(gs[:nv], want_s[:nv]) <= 2e-2
