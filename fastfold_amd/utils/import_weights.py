"""AlphaFold 2 (JAX / haiku) Evoformer parameters -> this package's layouts.

The reference reads a DeepMind ``params_model_*.npz`` into its plain-PyTorch model
(``fastfold/utils/import_weights.py:31-57`` parameter transformations, ``:131-360`` per-module
translation tables, ``:406-444`` the ``evoformer`` entry, ``:588-610`` ``import_jax_weights_``) and then
re-packs that model for fastnn (``fastfold/utils/inject_fastnn.py``).  Here the same two steps are
functions on plain mappings, for the Evoformer stack only:

    nn_sd   = evoformer_nn_state_dict_from_jax(np.load(path))        # AF2 arrays -> nn-layout state dict
    fast_sd = convert_nn_state_dict(nn_sd)                           # nn layout  -> fastnn layout
    stack.load_state_dict(fast_sd)

or ``import_jax_evoformer_(stack, path_or_mapping)`` for both at once.

AF2 stores every Evoformer block parameter stacked over the blocks (leading axis), linear weights as
[in, out], attention projections as [in, heads, head_dim] (output: [heads, head_dim, out]; gating bias
[heads, head_dim]) and the outer-product-mean output weight as [c, c, c_z]; haiku separates the module
path from the parameter name with a double slash.  No AF2 checkpoint is available offline, so the key
names and shapes below follow the reference's tables, not a file.
"""
import numpy as np
import torch

from fastfold_amd.utils.inject_fastnn import convert_nn_state_dict

NPZ_PREFIX = "alphafold/alphafold_iteration/"      # reference: import_weights.py:25


# ---- parameter transformations (reference: import_weights.py:31-52) ----
def _linear_weight(w):          # [..., in, out] -> [..., out, in]
    return np.swapaxes(w, -1, -2)


def _linear_weight_mha(w):      # [..., in, H, d] -> [..., H*d, in]
    return np.swapaxes(w.reshape(w.shape[:-2] + (-1,)), -1, -2)


def _mha_output_weight(w):      # [..., H, d, out] -> [..., out, H*d]
    return np.swapaxes(w.reshape(w.shape[:-3] + (-1, w.shape[-1])), -1, -2)


def _linear_bias_mha(b):        # [..., H, d] -> [..., H*d]
    return b.reshape(b.shape[:-2] + (-1,))


_opm_weight = _mha_output_weight    # [..., c, c, c_z] -> [..., c_z, c*c]   (same reshape: import_weights.py:40-42)


def _same(x):
    return x


def _layer_norm(dst):
    return [("scale", dst + ".weight", _same), ("offset", dst + ".bias", _same)]


def _linear(dst):
    return [("weights", dst + ".weight", _linear_weight), ("bias", dst + ".bias", _same)]


def _attention(dst):            # gated attention (reference: AttentionGatedParams, import_weights.py:60-80)
    return [("query_w", dst + ".linear_q.weight", _linear_weight_mha),
            ("key_w", dst + ".linear_k.weight", _linear_weight_mha),
            ("value_w", dst + ".linear_v.weight", _linear_weight_mha),
            ("output_w", dst + ".linear_o.weight", _mha_output_weight),
            ("output_b", dst + ".linear_o.bias", _same),
            ("gating_w", dst + ".linear_g.weight", _linear_weight_mha),
            ("gating_b", dst + ".linear_g.bias", _linear_bias_mha)]


def _sub(module, entries):
    return [(module + "//" + leaf, dst, fn) for leaf, dst, fn in entries]


def _transition(module, dst):
    return (_sub(module + "/input_layer_norm", _layer_norm(dst + ".layer_norm")) +
            _sub(module + "/transition1", _linear(dst + ".linear_1")) +
            _sub(module + "/transition2", _linear(dst + ".linear_2")))


def _tri_mul(module, dst, incoming):
    # AlphaFold swaps "left" and "right" between the outgoing and the incoming update; the nn modules do
    # not (reference: import_weights.py:222-236)
    a, b = ("b", "a") if incoming else ("a", "b")
    return (_sub(module + "/layer_norm_input", _layer_norm(dst + ".layer_norm_in")) +
            _sub(module + "/left_projection", _linear(dst + ".linear_%s_p" % a)) +
            _sub(module + "/right_projection", _linear(dst + ".linear_%s_p" % b)) +
            _sub(module + "/left_gate", _linear(dst + ".linear_%s_g" % a)) +
            _sub(module + "/right_gate", _linear(dst + ".linear_%s_g" % b)) +
            _sub(module + "/center_layer_norm", _layer_norm(dst + ".layer_norm_out")) +
            _sub(module + "/output_projection", _linear(dst + ".linear_z")) +
            _sub(module + "/gating_linear", _linear(dst + ".linear_g")))


def _tri_att(module, dst):
    return (_sub(module + "/query_norm", _layer_norm(dst + ".layer_norm")) +
            _sub(module, [("feat_2d_weights", dst + ".linear.weight", _linear_weight)]) +
            _sub(module + "/attention", _attention(dst + ".mha")))


def block_translation():
    """[(key below ``evoformer/evoformer_iteration/``, nn-layout name below ``blocks.N.``, transformation)]
    for one Evoformer block (reference: EvoformerBlockParams, import_weights.py:340-360)."""
    row, col = "msa_row_attention_with_pair_bias", "msa_column_attention"
    opm = "outer_product_mean"
    t = []
    t += _sub(row + "/query_norm", _layer_norm("msa_att_row.layer_norm_m"))
    t += _sub(row + "/feat_2d_norm", _layer_norm("msa_att_row.layer_norm_z"))
    t += _sub(row, [("feat_2d_weights", "msa_att_row.linear_z.weight", _linear_weight)])
    t += _sub(row + "/attention", _attention("msa_att_row.mha"))
    t += _sub(col + "/query_norm", _layer_norm("msa_att_col._msa_att.layer_norm_m"))
    t += _sub(col + "/attention", _attention("msa_att_col._msa_att.mha"))
    t += _transition("msa_transition", "core.msa_transition")
    t += _sub(opm + "/layer_norm_input", _layer_norm("core.outer_product_mean.layer_norm"))
    t += _sub(opm + "/left_projection", _linear("core.outer_product_mean.linear_1"))
    t += _sub(opm + "/right_projection", _linear("core.outer_product_mean.linear_2"))
    t += _sub(opm, [("output_w", "core.outer_product_mean.linear_out.weight", _opm_weight),
                    ("output_b", "core.outer_product_mean.linear_out.bias", _same)])
    t += _tri_mul("triangle_multiplication_outgoing", "core.tri_mul_out", False)
    t += _tri_mul("triangle_multiplication_incoming", "core.tri_mul_in", True)
    t += _tri_att("triangle_attention_starting_node", "core.tri_att_start")
    t += _tri_att("triangle_attention_ending_node", "core.tri_att_end")
    t += _transition("pair_transition", "core.pair_transition")
    return t


def evoformer_nn_state_dict_from_jax(params, no_blocks=None, prefix=NPZ_PREFIX + "evoformer/"):
    """AF2 parameter mapping (``np.load`` of a ``params_model_*.npz``, or any dict of arrays) -> nn-layout
    state dict of the Evoformer stack (``blocks.N.msa_att_row...``, ``linear.{weight,bias}``) as torch
    tensors.  Raises KeyError naming the first missing array, ValueError on a block-count mismatch."""
    out = {}
    n = no_blocks
    for key, dst, fn in block_translation():
        full = prefix + "evoformer_iteration/" + key
        if full not in params:
            raise KeyError("AlphaFold parameter %r not found" % full)
        arr = np.asarray(params[full])
        if n is None:
            n = arr.shape[0]
        if arr.shape[0] != n:
            raise ValueError("%r is stacked over %d blocks, expected %d" % (full, arr.shape[0], n))
        for i in range(n):
            out["blocks.%d.%s" % (i, dst)] = torch.from_numpy(np.ascontiguousarray(fn(arr[i])))
    for leaf, dst, fn in _linear("linear"):
        full = prefix + "single_activations//" + leaf
        if full not in params:
            raise KeyError("AlphaFold parameter %r not found" % full)
        out[dst] = torch.from_numpy(np.ascontiguousarray(fn(np.asarray(params[full]))))
    return out


def import_jax_evoformer_(stack, params, strict=True):
    """Loads AF2 Evoformer parameters into a ``fastfold_amd.model.fastnn.EvoformerStack`` (in place);
    ``params`` is a path to an ``.npz`` or a mapping of arrays.  Returns ``load_state_dict``'s result."""
    if isinstance(params, (str, bytes)) or hasattr(params, "__fspath__"):
        params = np.load(params)        # allow_pickle stays False: arrays only
    nn_sd = evoformer_nn_state_dict_from_jax(params, no_blocks=len(stack.blocks))
    ref = next(stack.parameters())
    fast_sd = {k: v.to(device=ref.device, dtype=ref.dtype) for k, v in convert_nn_state_dict(nn_sd).items()}
    return stack.load_state_dict(fast_sd, strict=strict)
