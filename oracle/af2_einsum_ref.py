"""AlphaFold-2's Evoformer iteration computed straight from AlphaFold-layout parameter arrays, float64 numpy.

TEST INFRASTRUCTURE ONLY - never imported by the product package.

Purpose: an oracle for the weight importer (``fastfold_amd/utils/import_weights.py``) that does not share its
translation table.  The arrays are used the way AlphaFold's own haiku modules use them - the einsum strings of
``alphafold/model/modules.py`` (AlphaFold v2.x, the code the reference's ``fastfold/utils/import_weights.py:131-360``
tables were written against; it is not vendored in the reference, so the published algorithm is restated here:
Jumper et al. 2021, supplementary Algorithms 6-15):

    Attention            q = einsum('bqa,ahc->bqhc', q_data, query_w) * key_dim**-0.5
                         k = einsum('bka,ahc->bkhc', m_data, key_w);  v likewise with value_w
                         logits = einsum('bqhc,bkhc->bhqk', q, k) + bias (+ nonbatched_bias)
                         o = einsum('bhqk,bkhc->bqhc', softmax(logits), v)
                         o *= sigmoid(einsum('bqc,chv->bqhv', q_data, gating_w) + gating_b)
                         out = einsum('bqhc,hco->bqo', o, output_w) + output_b
    pair bias            einsum('qkc,ch->hqk', LayerNorm(pair), feat_2d_weights)
    Linear               x @ weights + bias                                     (weights are [in, out])
    OuterProductMean     einsum over sequences of left[s,i,c] right[s,j,e], then einsum('ijce,cef->ijf', ., output_w)
    TriangleMultiplication   outgoing 'ikc,jkc->ijc', incoming 'kjc,kic->ijc' on (left, right)

Pinned by ``tests/test_import_weights.py``: against the CPU oracle (``oracle/evoformer_ref.py``, itself pinned by the
reference's golden vectors) loaded through the importer - two independent routes from the same arrays to the same
numbers - and by the closed-form checks there.  Parameter names follow haiku's ``module//parameter`` convention.
"""
import numpy as np

PREFIX = "alphafold/alphafold_iteration/evoformer/"
IT = PREFIX + "evoformer_iteration/"


def param_shapes(c_m=256, c_z=128, hm=8, hz=4, d=32, c_opm=32, c_mul=128, n=4, c_s=384):
    """name below ``evoformer_iteration/`` -> per-block shape, in AlphaFold's layout."""
    sh = {}

    def ln(mod, c):
        sh[mod + "//scale"] = (c,)
        sh[mod + "//offset"] = (c,)

    def lin(mod, cin, cout):
        sh[mod + "//weights"] = (cin, cout)
        sh[mod + "//bias"] = (cout,)

    def att(mod, c, h):
        for w in ("query_w", "key_w", "value_w", "gating_w"):
            sh[mod + "//" + w] = (c, h, d)
        sh[mod + "//gating_b"] = (h, d)
        sh[mod + "//output_w"] = (h, d, c)
        sh[mod + "//output_b"] = (c,)

    row, col = "msa_row_attention_with_pair_bias", "msa_column_attention"
    ln(row + "/query_norm", c_m)
    ln(row + "/feat_2d_norm", c_z)
    sh[row + "//feat_2d_weights"] = (c_z, hm)
    att(row + "/attention", c_m, hm)
    ln(col + "/query_norm", c_m)
    att(col + "/attention", c_m, hm)
    for mod, c in (("msa_transition", c_m), ("pair_transition", c_z)):
        ln(mod + "/input_layer_norm", c)
        lin(mod + "/transition1", c, n * c)
        lin(mod + "/transition2", n * c, c)
    opm = "outer_product_mean"
    ln(opm + "/layer_norm_input", c_m)
    lin(opm + "/left_projection", c_m, c_opm)
    lin(opm + "/right_projection", c_m, c_opm)
    sh[opm + "//output_w"] = (c_opm, c_opm, c_z)
    sh[opm + "//output_b"] = (c_z,)
    for mod in ("triangle_multiplication_outgoing", "triangle_multiplication_incoming"):
        ln(mod + "/layer_norm_input", c_z)
        for p in ("left_projection", "right_projection", "left_gate", "right_gate"):
            lin(mod + "/" + p, c_z, c_mul)
        ln(mod + "/center_layer_norm", c_mul)
        lin(mod + "/output_projection", c_mul, c_z)
        lin(mod + "/gating_linear", c_z, c_z)
    for mod in ("triangle_attention_starting_node", "triangle_attention_ending_node"):
        ln(mod + "/query_norm", c_z)
        sh[mod + "//feat_2d_weights"] = (c_z, hz)
        att(mod + "/attention", c_z, hz)
    return sh


def random_params(seed, no_blocks, c_m=256, c_z=128, c_s=384, **dims):
    """A seeded AlphaFold-layout parameter mapping (block parameters stacked over the blocks), fan-in scaled so
    that every update is O(1)."""
    rng = np.random.RandomState(seed)
    out = {}
    for name, shape in param_shapes(c_m=c_m, c_z=c_z, c_s=c_s, **dims).items():
        leaf = name.split("//")[1]
        x = rng.standard_normal((no_blocks,) + shape)
        if leaf == "scale":
            x = 1.0 + 0.1 * x
        elif leaf in ("offset", "bias", "output_b", "gating_b"):
            x = 0.1 * x
        elif leaf == "output_w" and len(shape) == 3 and "attention" in name:
            x = x / np.sqrt(shape[0] * shape[1])          # [h, d, out]: fan-in h * d
        elif leaf == "output_w":
            x = x / np.sqrt(shape[0] * shape[1])          # outer product mean [c, c, c_z]
        else:
            x = x / np.sqrt(shape[0])                      # [in, ...]
        out[IT + name] = x.astype(np.float32)
    out[PREFIX + "single_activations//weights"] = (rng.standard_normal((c_m, c_s)) / np.sqrt(c_m)).astype(np.float32)
    out[PREFIX + "single_activations//bias"] = (0.1 * rng.standard_normal((c_s,))).astype(np.float32)
    return out


def _ln(x, p, mod, eps=1e-5):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * p[mod + "//scale"] + p[mod + "//offset"]


def _lin(x, p, mod):
    return x @ p[mod + "//weights"] + p[mod + "//bias"]


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def _softmax(x):
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def _attention(q_data, m_data, bias, nonbatched_bias, p, mod):
    qw, kw, vw = p[mod + "//query_w"], p[mod + "//key_w"], p[mod + "//value_w"]
    q = np.einsum("bqa,ahc->bqhc", q_data, qw) * qw.shape[-1] ** -0.5
    k = np.einsum("bka,ahc->bkhc", m_data, kw)
    v = np.einsum("bka,ahc->bkhc", m_data, vw)
    logits = np.einsum("bqhc,bkhc->bhqk", q, k) + bias
    if nonbatched_bias is not None:
        logits = logits + nonbatched_bias[None]
    o = np.einsum("bhqk,bkhc->bqhc", _softmax(logits), v)
    o = o * _sigmoid(np.einsum("bqc,chv->bqhv", q_data, p[mod + "//gating_w"]) + p[mod + "//gating_b"])
    return np.einsum("bqhc,hco->bqo", o, p[mod + "//output_w"]) + p[mod + "//output_b"]


def _transition(x, p, mod):
    h = np.maximum(_lin(_ln(x, p, mod + "/input_layer_norm"), p, mod + "/transition1"), 0.0)
    return _lin(h, p, mod + "/transition2")


def _tri_mul(z, mask, p, mod, equation):
    act = _ln(z, p, mod + "/layer_norm_input")
    left = mask[..., None] * _lin(act, p, mod + "/left_projection") * _sigmoid(_lin(act, p, mod + "/left_gate"))
    right = mask[..., None] * _lin(act, p, mod + "/right_projection") * _sigmoid(_lin(act, p, mod + "/right_gate"))
    out = np.einsum(equation, left, right)
    out = _lin(_ln(out, p, mod + "/center_layer_norm"), p, mod + "/output_projection")
    return out * _sigmoid(_lin(act, p, mod + "/gating_linear"))


def _tri_att(z, mask, p, mod, per_column):
    if per_column:
        z, mask = z.swapaxes(0, 1), mask.swapaxes(0, 1)
    act = _ln(z, p, mod + "/query_norm")
    bias = (1e9 * (mask - 1.0))[:, None, None, :]
    nb = np.einsum("qkc,ch->hqk", act, p[mod + "//feat_2d_weights"])
    out = _attention(act, act, bias, nb, p, mod + "/attention")
    return out.swapaxes(0, 1) if per_column else out


def evoformer_iteration(m, z, msa_mask, pair_mask, p):
    """One block (supplementary Algorithm 6, lines 2-10, in AlphaFold's order: row attention, column attention, MSA
    transition, outer product mean, the two triangle multiplications, the two triangle attentions, pair transition).
    ``p`` maps the names of ``param_shapes`` to this block's arrays.  Transitions are not masked."""
    row, col = "msa_row_attention_with_pair_bias", "msa_column_attention"
    act = _ln(m, p, row + "/query_norm")
    nb = np.einsum("qkc,ch->hqk", _ln(z, p, row + "/feat_2d_norm"), p[row + "//feat_2d_weights"])
    m = m + _attention(act, act, (1e9 * (msa_mask - 1.0))[:, None, None, :], nb, p, row + "/attention")
    act = _ln(m.swapaxes(0, 1), p, col + "/query_norm")
    mt = msa_mask.swapaxes(0, 1)
    m = m + _attention(act, act, (1e9 * (mt - 1.0))[:, None, None, :], None, p, col + "/attention").swapaxes(0, 1)
    m = m + _transition(m, p, "msa_transition")
    opm = "outer_product_mean"
    act = _ln(m, p, opm + "/layer_norm_input")
    left = msa_mask[..., None] * _lin(act, p, opm + "/left_projection")
    right = msa_mask[..., None] * _lin(act, p, opm + "/right_projection")
    outer = np.einsum("sic,sje->ijce", left, right)
    upd = np.einsum("ijce,cef->ijf", outer, p[opm + "//output_w"]) + p[opm + "//output_b"]
    z = z + upd / (1e-3 + np.einsum("si,sj->ij", msa_mask, msa_mask))[..., None]
    z = z + _tri_mul(z, pair_mask, p, "triangle_multiplication_outgoing", "ikc,jkc->ijc")
    z = z + _tri_mul(z, pair_mask, p, "triangle_multiplication_incoming", "kjc,kic->ijc")
    z = z + _tri_att(z, pair_mask, p, "triangle_attention_starting_node", False)
    z = z + _tri_att(z, pair_mask, p, "triangle_attention_ending_node", True)
    z = z + _transition(z, p, "pair_transition")
    return m, z


def evoformer_stack(m, z, msa_mask, pair_mask, params):
    """All blocks of an AlphaFold-layout mapping (arrays stacked over blocks), then the single representation."""
    m, z = np.asarray(m, np.float64), np.asarray(z, np.float64)
    msa_mask, pair_mask = np.asarray(msa_mask, np.float64), np.asarray(pair_mask, np.float64)
    names = [k[len(IT):] for k in params if k.startswith(IT)]
    nb = params[IT + names[0]].shape[0]
    for i in range(nb):
        p = {n: np.asarray(params[IT + n][i], np.float64) for n in names}
        m, z = evoformer_iteration(m, z, msa_mask, pair_mask, p)
    s = m[0] @ np.asarray(params[PREFIX + "single_activations//weights"], np.float64) \
        + np.asarray(params[PREFIX + "single_activations//bias"], np.float64)
    return m, z, s
