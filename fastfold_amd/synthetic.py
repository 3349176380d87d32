"""Deterministic synthetic parameters and inputs for the Evoformer stack.

Everything is drawn from ``numpy.random.RandomState(seed)`` in a fixed, documented order,
so any machine regenerates bit-identical tensors.  Parameters are produced in the
reference's *nn layout* (the names of ``fastfold.model.nn.evoformer.EvoformerStack``'s
state dict); ``fastfold_amd.utils.inject_fastnn`` re-packs them into the fastnn layout.

Order of draws for one block (prefix ``blocks.<i>.``), each tensor ``std * N(0,1)`` in
fp32 (LayerNorm weights are ``1 + std * N(0,1)``), weight before bias:
  msa_att_row:  layer_norm_m, layer_norm_z, linear_z.weight, mha.linear_{q,k,v}.weight,
                mha.linear_o, mha.linear_g
  msa_att_col._msa_att:  layer_norm_m, mha.linear_{q,k,v}.weight, mha.linear_o, mha.linear_g
  core.msa_transition:   layer_norm, linear_1, linear_2
  core.outer_product_mean: layer_norm, linear_1, linear_2, linear_out
  core.tri_mul_out / core.tri_mul_in: layer_norm_in, linear_a_p, linear_a_g, linear_b_p,
                linear_b_g, linear_g, linear_z, layer_norm_out
  core.tri_att_start / core.tri_att_end: layer_norm, linear.weight, mha.linear_{q,k,v}.weight,
                mha.linear_o, mha.linear_g
  core.pair_transition:  layer_norm, linear_1, linear_2
then, after all blocks, ``linear.weight``, ``linear.bias``.
"""
from collections import OrderedDict

import numpy as np


def nn_layout_block_shapes(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128,
                           c_hidden_pair_att=32, no_heads_msa=8, no_heads_pair=4, transition_n=4):
    """(name, shape, kind) triples of one block in draw order; kind in {'w', 'b', 'ln_w', 'ln_b'}."""
    out = []

    def ln(p, c):
        out.append((p + ".weight", (c,), "ln_w"))
        out.append((p + ".bias", (c,), "ln_b"))

    def lin(p, cin, cout, bias=True):
        out.append((p + ".weight", (cout, cin), "w"))
        if bias:
            out.append((p + ".bias", (cout,), "b"))

    def mha(p, c, hid, heads):
        hc = hid * heads
        lin(p + ".linear_q", c, hc, bias=False)
        lin(p + ".linear_k", c, hc, bias=False)
        lin(p + ".linear_v", c, hc, bias=False)
        lin(p + ".linear_o", hc, c)
        lin(p + ".linear_g", c, hc)

    ln("msa_att_row.layer_norm_m", c_m)
    ln("msa_att_row.layer_norm_z", c_z)
    lin("msa_att_row.linear_z", c_z, no_heads_msa, bias=False)
    mha("msa_att_row.mha", c_m, c_hidden_msa_att, no_heads_msa)
    ln("msa_att_col._msa_att.layer_norm_m", c_m)
    mha("msa_att_col._msa_att.mha", c_m, c_hidden_msa_att, no_heads_msa)
    ln("core.msa_transition.layer_norm", c_m)
    lin("core.msa_transition.linear_1", c_m, transition_n * c_m)
    lin("core.msa_transition.linear_2", transition_n * c_m, c_m)
    ln("core.outer_product_mean.layer_norm", c_m)
    lin("core.outer_product_mean.linear_1", c_m, c_hidden_opm)
    lin("core.outer_product_mean.linear_2", c_m, c_hidden_opm)
    lin("core.outer_product_mean.linear_out", c_hidden_opm ** 2, c_z)
    for tm in ("core.tri_mul_out", "core.tri_mul_in"):
        ln(tm + ".layer_norm_in", c_z)
        lin(tm + ".linear_a_p", c_z, c_hidden_mul)
        lin(tm + ".linear_a_g", c_z, c_hidden_mul)
        lin(tm + ".linear_b_p", c_z, c_hidden_mul)
        lin(tm + ".linear_b_g", c_z, c_hidden_mul)
        lin(tm + ".linear_g", c_z, c_z)
        lin(tm + ".linear_z", c_hidden_mul, c_z)
        ln(tm + ".layer_norm_out", c_hidden_mul)
    for ta in ("core.tri_att_start", "core.tri_att_end"):
        ln(ta + ".layer_norm", c_z)
        lin(ta + ".linear", c_z, no_heads_pair, bias=False)
        mha(ta + ".mha", c_z, c_hidden_pair_att, no_heads_pair)
    ln("core.pair_transition.layer_norm", c_z)
    lin("core.pair_transition.linear_1", c_z, transition_n * c_z)
    lin("core.pair_transition.linear_2", transition_n * c_z, c_z)
    return out


def extra_nn_layout_block_shapes(c_m=64, c_z=128, c_hidden_msa_att=8, c_hidden_opm=32, c_hidden_mul=128,
                                 c_hidden_pair_att=32, no_heads_msa=8, no_heads_pair=4, transition_n=4):
    """One extra-MSA block (``fastfold.model.nn.evoformer.ExtraMSABlock``) in draw order: as an Evoformer
    block, with the column attention replaced by
      msa_att_col: layer_norm_m, global_attention.linear_{q,k,v}.weight, .linear_g, .linear_o"""
    base = nn_layout_block_shapes(c_m=c_m, c_z=c_z, c_hidden_msa_att=c_hidden_msa_att, c_hidden_opm=c_hidden_opm,
                                  c_hidden_mul=c_hidden_mul, c_hidden_pair_att=c_hidden_pair_att,
                                  no_heads_msa=no_heads_msa, no_heads_pair=no_heads_pair, transition_n=transition_n)
    hc = c_hidden_msa_att * no_heads_msa
    g = "msa_att_col.global_attention."
    col = [("msa_att_col.layer_norm_m.weight", (c_m,), "ln_w"), ("msa_att_col.layer_norm_m.bias", (c_m,), "ln_b"),
           (g + "linear_q.weight", (hc, c_m), "w"), (g + "linear_k.weight", (c_hidden_msa_att, c_m), "w"),
           (g + "linear_v.weight", (c_hidden_msa_att, c_m), "w"),
           (g + "linear_g.weight", (hc, c_m), "w"), (g + "linear_g.bias", (hc,), "b"),
           (g + "linear_o.weight", (c_m, hc), "w"), (g + "linear_o.bias", (c_m,), "b")]
    out, done = [], False
    for ent in base:
        if ent[0].startswith("msa_att_col."):
            if not done:
                out += col
                done = True
            continue
        out.append(ent)
    return out


def synth_extra_nn_state(seed=0, no_blocks=1, std=0.02, fan_in_scaled=False, **dims):
    """nn-layout state of an ``ExtraMSAStack`` (no final linear), drawn like ``synth_nn_state``."""
    rng = np.random.RandomState(seed)
    sd = OrderedDict()
    for i in range(no_blocks):
        for name, shape, kind in extra_nn_layout_block_shapes(**dims):
            x = rng.standard_normal(shape).astype(np.float32)
            if kind == "ln_w":
                x = 1.0 + std * x
            elif kind == "w" and fan_in_scaled:
                x = x / np.sqrt(shape[1])
            else:
                x = std * x
            sd["blocks.%d.%s" % (i, name)] = x.astype(np.float32)
    return sd


def template_nn_layout_block_shapes(c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_heads=4, pair_transition_n=2):
    """One ``TemplatePairStackBlock`` in draw order: tri_att_start, tri_att_end (layer_norm, linear.weight,
    mha.linear_{q,k,v}.weight, mha.linear_o, mha.linear_g), tri_mul_out, tri_mul_in (layer_norm_in, linear_a_p,
    linear_a_g, linear_b_p, linear_b_g, linear_g, linear_z, layer_norm_out), pair_transition."""
    base = nn_layout_block_shapes(c_m=c_t, c_z=c_t, c_hidden_mul=c_hidden_tri_mul, c_hidden_pair_att=c_hidden_tri_att,
                                  no_heads_pair=no_heads, transition_n=pair_transition_n)
    out = []
    for prefix in ("core.tri_att_start.", "core.tri_att_end.", "core.tri_mul_out.", "core.tri_mul_in.",
                   "core.pair_transition."):
        out += [(n[len("core."):], sh, k) for n, sh, k in base if n.startswith(prefix)]
    return out


def synth_template_nn_state(seed=0, no_blocks=2, std=0.02, fan_in_scaled=False, c_t=64, **dims):
    """nn-layout state of a ``TemplatePairStack`` (blocks, then ``layer_norm``), drawn like ``synth_nn_state``."""
    rng = np.random.RandomState(seed)
    sd = OrderedDict()

    def draw(shape, kind):
        x = rng.standard_normal(shape).astype(np.float32)
        if kind == "ln_w":
            return (1.0 + std * x).astype(np.float32)
        if kind == "w" and fan_in_scaled:
            return (x / np.sqrt(shape[1])).astype(np.float32)
        return (std * x).astype(np.float32)

    for i in range(no_blocks):
        for name, shape, kind in template_nn_layout_block_shapes(c_t=c_t, **dims):
            sd["blocks.%d.%s" % (i, name)] = draw(shape, kind)
    sd["layer_norm.weight"] = draw((c_t,), "ln_w")
    sd["layer_norm.bias"] = draw((c_t,), "ln_b")
    return sd


def synth_pointwise_nn_state(seed=0, c_t=64, c_z=128, c_hidden=16, no_heads=4):
    """nn-layout state of a ``TemplatePointwiseAttention`` (``mha.linear_{q,k,v,o}``), fan-in scaled weights so
    that the logits over the templates are O(1)."""
    rng = np.random.RandomState(seed)
    hc = c_hidden * no_heads
    sd = OrderedDict()
    for name, shape in (("mha.linear_q.weight", (hc, c_z)), ("mha.linear_k.weight", (hc, c_t)),
                        ("mha.linear_v.weight", (hc, c_t)), ("mha.linear_o.weight", (c_z, hc))):
        sd[name] = (rng.standard_normal(shape) * (2.0 if name.endswith("q.weight") else 1.0)
                    / np.sqrt(shape[1])).astype(np.float32)
    sd["mha.linear_o.bias"] = (0.1 * rng.standard_normal((c_z,))).astype(np.float32)
    return sd


def synth_pointwise_inputs(seed, n_templ, n_res, c_t=64, c_z=128):
    """t [n_templ, r, r, c_t], z [r, r, c_z] ~ N(0, 1) fp32."""
    rng = np.random.RandomState(seed + 7)
    t = rng.standard_normal((n_templ, n_res, n_res, c_t)).astype(np.float32)
    z = rng.standard_normal((n_res, n_res, c_z)).astype(np.float32)
    return t, z


def synth_nn_state(seed=0, no_blocks=1, std=0.02, c_m=256, c_z=128, c_s=384, fan_in_scaled=False, **dims):
    """OrderedDict name -> float32 numpy array, nn layout, for an ``EvoformerStack``.

    ``fan_in_scaled=True`` draws linear weights with std ``1/sqrt(fan_in)`` (and biases / LayerNorm
    offsets with ``std``) so that every update is O(1): used by parity tests that must not hide a
    wrong update behind a dominant residual stream."""
    rng = np.random.RandomState(seed)
    sd = OrderedDict()
    shapes = nn_layout_block_shapes(c_m=c_m, c_z=c_z, **dims)

    def draw(shape, kind):
        x = rng.standard_normal(shape).astype(np.float32)
        if kind == "ln_w":
            return (1.0 + std * x).astype(np.float32)
        if kind == "w" and fan_in_scaled:
            return (x / np.sqrt(shape[1])).astype(np.float32)
        return (std * x).astype(np.float32)

    for i in range(no_blocks):
        for name, shape, kind in shapes:
            sd["blocks.%d.%s" % (i, name)] = draw(shape, kind)
    sd["linear.weight"] = draw((c_s, c_m), "w")
    sd["linear.bias"] = draw((c_s,), "b")
    return sd


def synth_inputs(seed, n_seq, n_res, c_m=256, c_z=128, mask_tail_frac=0.0):
    """m [s,r,c_m], z [r,r,c_z] ~ N(0,1) fp32; masks as the reference builds them from a
    residue mask (hub/alphafold.py:193-195): the last ``mask_tail_frac`` of residues are padding,
    ``pair_mask = seq_mask x seq_mask``, ``msa_mask = ones[s] x seq_mask``."""
    rng = np.random.RandomState(seed + 1000003)
    m = rng.standard_normal((n_seq, n_res, c_m)).astype(np.float32)
    z = rng.standard_normal((n_res, n_res, c_z)).astype(np.float32)
    seq_mask = np.ones((n_res,), np.float32)
    n_pad = int(round(mask_tail_frac * n_res))
    if n_pad > 0:
        seq_mask[n_res - n_pad:] = 0.0
    msa_mask = np.ones((n_seq, 1), np.float32) * seq_mask[None, :]
    pair_mask = seq_mask[:, None] * seq_mask[None, :]
    return m, z, msa_mask, pair_mask


def bf16_round(x):
    """fp32 array rounded to the nearest bf16 value (round-to-nearest-even on the upper 16 bits), still fp32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(x))


def synth_template_inputs(seed, n_templ, n_res, c_t=64, mask_tail_frac=0.0):
    """t [n_templ, r, r, c_t] ~ N(0,1) fp32 and the pair mask [r, r] shared by the templates."""
    t = synth_inputs(seed, n_templ, n_res * n_res, c_m=c_t, c_z=1)[0].reshape(n_templ, n_res, n_res, c_t)
    pair_mask = synth_inputs(seed, 1, n_res, c_m=1, c_z=1, mask_tail_frac=mask_tail_frac)[3]
    return t, pair_mask
