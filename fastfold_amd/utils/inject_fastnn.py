"""Drop-in seam: swap a model's plain-PyTorch Evoformer (nn layout) for the HIP-backed
``fastfold_amd.model.fastnn.EvoformerStack`` and re-pack its weights.

Same entry points as the reference's ``fastfold/utils/inject_fastnn.py`` for the Evoformer
path (``inject_fastnn``, ``inject_evoformer``, ``copy_*``; reference lines 24-152,321-338,
418-423).  The weight re-layout is:
  q/k/v weights            -> rows of ``to_qkv.weight`` in that order
  linear_g.{weight,bias}   -> ``gating_linear.weight`` / ``gating_bias``
  linear_o.weight          -> ``o_linear.weight``; its bias -> ``out_bias`` (row / triangle
                              attention) or ``o_linear.bias`` (column attention)
  linear_z.weight (row)    -> ``linear_b_weights``
  tri-mul a_p|b_p, a_g|b_g -> ``left_right_projection`` / ``left_right_gate`` (left rows first),
  linear_g -> ``output_gate``, linear_z.{weight,bias} -> ``output_projection.weight`` / ``output_bias``
  OPM linear_1/2/out       -> ``linear_a`` / ``linear_b`` / ``o_linear``
The extra-MSA stack (``inject_extramsa``, reference lines 154-236,341-355) follows the same re-layout,
with the global column attention's linear_q -> ``to_q``, linear_k | linear_v -> rows of ``to_kv``.
Of the template stage only the pair stack is built (``inject_template_pair_stack``, same triangle /
transition re-layout); ``inject_embedder`` swaps the input and recycling embedders (plain copies).
"""
import torch

from fastfold_amd.model.fastnn import EvoformerStack, ExtraMSAStack
from fastfold_amd.model.fastnn.embedders import InputEmbedder, RecyclingEmbedder
from fastfold_amd.model.fastnn.template import TemplatePairStack, TemplatePointwiseAttention


def copy_layernorm(model_fast, model_ori):
    model_fast.weight.copy_(model_ori.weight)
    model_fast.bias.copy_(model_ori.bias)


def copy_linear(model_fast, model_ori):
    model_fast.weight.copy_(model_ori.weight)
    if model_fast.use_bias:
        model_fast.bias.copy_(model_ori.bias)


def copy_qkv_linear(model_fast, ori_q, ori_k, ori_v):
    model_fast.weight.copy_(torch.cat((ori_q.weight, ori_k.weight, ori_v.weight), dim=0))


def copy_attention(model_fast, model_ori):
    copy_qkv_linear(model_fast.to_qkv, model_ori.linear_q, model_ori.linear_k, model_ori.linear_v)
    copy_linear(model_fast.gating_linear, model_ori.linear_g)
    copy_linear(model_fast.o_linear, model_ori.linear_o)
    if getattr(model_fast, "gating_bias", None) is not None and model_ori.linear_g is not None:
        model_fast.gating_bias.copy_(model_ori.linear_g.bias)


def copy_kv_linear(model_fast, ori_k, ori_v):
    model_fast.weight.copy_(torch.cat((ori_k.weight, ori_v.weight), dim=0))


def copy_global_attention(model_fast, model_ori):
    copy_linear(model_fast.to_q, model_ori.linear_q)
    copy_kv_linear(model_fast.to_kv, model_ori.linear_k, model_ori.linear_v)
    copy_linear(model_fast.gating_linear, model_ori.linear_g)
    copy_linear(model_fast.o_linear, model_ori.linear_o)
    model_fast.gating_bias.copy_(model_ori.linear_g.bias)


def copy_left_right(model_fast, ori_left, ori_right):
    model_fast.weight.copy_(torch.cat((ori_left.weight, ori_right.weight), dim=0))
    model_fast.bias.copy_(torch.cat((ori_left.bias, ori_right.bias), dim=0))


def copy_transition(model_fast, model_ori):
    copy_layernorm(model_fast.norm, model_ori.layer_norm)
    copy_linear(model_fast.linear1, model_ori.linear_1)
    copy_linear(model_fast.linear2, model_ori.linear_2)


def copy_triangle(model_fast, model_ori):
    copy_layernorm(model_fast.layernorm1, model_ori.layer_norm_in)
    copy_layernorm(model_fast.layernorm2, model_ori.layer_norm_out)
    copy_linear(model_fast.output_projection, model_ori.linear_z)
    model_fast.output_bias.copy_(model_ori.linear_z.bias)
    copy_linear(model_fast.output_gate, model_ori.linear_g)
    copy_left_right(model_fast.left_right_projection, model_ori.linear_a_p, model_ori.linear_b_p)
    copy_left_right(model_fast.left_right_gate, model_ori.linear_a_g, model_ori.linear_b_g)


def copy_triangle_att(model_fast, model_ori):
    copy_layernorm(model_fast.layernorm1, model_ori.layer_norm)
    copy_linear(model_fast.linear_b, model_ori.linear)
    copy_attention(model_fast.attention, model_ori.mha)
    model_fast.out_bias.copy_(model_ori.mha.linear_o.bias)


def copy_evoformer_para(block_fast, block_ori):
    row_f, row_o = block_fast.msa.MSARowAttentionWithPairBias, block_ori.msa_att_row
    copy_layernorm(row_f.layernormM, row_o.layer_norm_m)
    copy_layernorm(row_f.layernormZ, row_o.layer_norm_z)
    copy_attention(row_f.attention, row_o.mha)
    row_f.linear_b_weights.copy_(row_o.linear_z.weight)
    row_f.out_bias.copy_(row_o.mha.linear_o.bias)

    col_f, col_o = block_fast.msa.MSAColumnAttention, block_ori.msa_att_col._msa_att
    copy_layernorm(col_f.layernormM, col_o.layer_norm_m)
    copy_attention(col_f.attention, col_o.mha)

    copy_transition(block_fast.msa.MSATransition, block_ori.core.msa_transition)

    opm_f, opm_o = block_fast.communication, block_ori.core.outer_product_mean
    copy_layernorm(opm_f.layernormM, opm_o.layer_norm)
    copy_linear(opm_f.linear_a, opm_o.linear_1)
    copy_linear(opm_f.linear_b, opm_o.linear_2)
    copy_linear(opm_f.o_linear, opm_o.linear_out)

    copy_triangle(block_fast.pair.TriangleMultiplicationOutgoing, block_ori.core.tri_mul_out)
    copy_triangle(block_fast.pair.TriangleMultiplicationIncoming, block_ori.core.tri_mul_in)
    copy_triangle_att(block_fast.pair.TriangleAttentionStartingNode, block_ori.core.tri_att_start)
    copy_triangle_att(block_fast.pair.TriangleAttentionEndingNode, block_ori.core.tri_att_end)
    copy_transition(block_fast.pair.PairTransition, block_ori.core.pair_transition)


def copy_extra_msa_para(block_fast, block_ori):
    row_f, row_o = block_fast.msa_stack.MSARowAttentionWithPairBias, block_ori.msa_att_row
    copy_layernorm(row_f.layernormM, row_o.layer_norm_m)
    copy_layernorm(row_f.layernormZ, row_o.layer_norm_z)
    copy_attention(row_f.attention, row_o.mha)
    row_f.linear_b_weights.copy_(row_o.linear_z.weight)
    row_f.out_bias.copy_(row_o.mha.linear_o.bias)

    col_f, col_o = block_fast.msa_stack.MSAColumnAttention, block_ori.msa_att_col
    copy_layernorm(col_f.layernormM, col_o.layer_norm_m)
    copy_global_attention(col_f.global_attention, col_o.global_attention)

    copy_transition(block_fast.msa_stack.MSATransition, block_ori.core.msa_transition)

    opm_f, opm_o = block_fast.communication, block_ori.core.outer_product_mean
    copy_layernorm(opm_f.layernormM, opm_o.layer_norm)
    copy_linear(opm_f.linear_a, opm_o.linear_1)
    copy_linear(opm_f.linear_b, opm_o.linear_2)
    copy_linear(opm_f.o_linear, opm_o.linear_out)

    copy_triangle(block_fast.pair_stack.TriangleMultiplicationOutgoing, block_ori.core.tri_mul_out)
    copy_triangle(block_fast.pair_stack.TriangleMultiplicationIncoming, block_ori.core.tri_mul_in)
    copy_triangle_att(block_fast.pair_stack.TriangleAttentionStartingNode, block_ori.core.tri_att_start)
    copy_triangle_att(block_fast.pair_stack.TriangleAttentionEndingNode, block_ori.core.tri_att_end)
    copy_transition(block_fast.pair_stack.PairTransition, block_ori.core.pair_transition)


def inject_extramsa(model):
    with torch.no_grad():
        target_module = model.extra_msa_stack
        ref_param = next(target_module.parameters())
        fast_module = ExtraMSAStack(
            c_m=target_module.blocks[0].msa_att_row.c_in,
            c_z=target_module.blocks[0].msa_att_row.c_z,
            no_blocks=len(target_module.blocks),
            clear_cache_between_blocks=target_module.clear_cache_between_blocks,
            is_multimer=target_module.blocks[0].is_multimer,
        ).to(device=ref_param.device, dtype=ref_param.dtype)
        for target_block, fast_block in zip(target_module.blocks, fast_module.blocks):
            copy_extra_msa_para(fast_block, target_block)
            if target_block.training is False:
                fast_block.eval()
        if target_module.training is False:
            fast_module.eval()
        model.extra_msa_stack = fast_module


def copy_template_pair_stack_para(block_fast, block_ori):
    copy_triangle(block_fast.TriangleMultiplicationOutgoing, block_ori.tri_mul_out)
    copy_triangle(block_fast.TriangleMultiplicationIncoming, block_ori.tri_mul_in)
    copy_triangle_att(block_fast.TriangleAttentionStartingNode, block_ori.tri_att_start)
    copy_triangle_att(block_fast.TriangleAttentionEndingNode, block_ori.tri_att_end)
    copy_transition(block_fast.PairTransition, block_ori.pair_transition)


def copy_template_pair_block_para(fast_module, target_module):
    with torch.no_grad():
        for ori_block, fast_block in zip(target_module.blocks, fast_module.blocks):
            copy_template_pair_stack_para(fast_block, ori_block)
            if ori_block.training is False:
                fast_block.eval()


def inject_template_pair_stack(template_embedder):
    """Swaps ``template_embedder.template_pair_stack`` (nn layout) for the HIP-backed stack.  The
    reference's ``inject_template`` (inject_fastnn.py:358-374) replaces the whole template embedder;
    the point-wise attention is swapped too when the embedder has one; its feature embedders stay as they are."""
    with torch.no_grad():
        target = template_embedder.template_pair_stack
        blk = target.blocks[0]
        ref_param = next(target.parameters())
        fast = TemplatePairStack(
            c_t=blk.tri_att_start.c_in, c_hidden_tri_att=blk.tri_att_start.c_hidden,
            c_hidden_tri_mul=blk.tri_mul_out.c_hidden, no_blocks=len(target.blocks),
            no_heads=blk.tri_att_start.no_heads, pair_transition_n=blk.pair_transition.n,
            dropout_rate=getattr(blk, "dropout_rate", 0.25), blocks_per_ckpt=target.blocks_per_ckpt,
            inf=blk.tri_att_start.inf).to(device=ref_param.device, dtype=ref_param.dtype)
        copy_template_pair_block_para(fast, target)
        copy_layernorm(fast.layer_norm, target.layer_norm)
        if target.training is False:
            fast.eval()
        template_embedder.template_pair_stack = fast
        if getattr(template_embedder, "template_pointwise_att", None) is not None:
            inject_template_pointwise_att(template_embedder)
    return template_embedder


def copy_native_att(model_fast, model_ori):
    """linear_q / linear_k / linear_v / linear_o of an un-gated ``Attention`` (inject_fastnn.py:98-104)."""
    for name in ("linear_q", "linear_k", "linear_v"):
        getattr(model_fast, name).weight.copy_(getattr(model_ori, name).weight)
    copy_linear(model_fast.linear_o, model_ori.linear_o)


def inject_template_pointwise_att(template_embedder):
    """Swaps ``template_embedder.template_pointwise_att`` for the HIP-backed module (the reference copies its
    parameters with ``copy_native_att``, inject_fastnn.py:278-279)."""
    with torch.no_grad():
        target = template_embedder.template_pointwise_att
        ref_param = next(target.parameters())
        fast = TemplatePointwiseAttention(c_t=target.c_t, c_z=target.c_z, c_hidden=target.c_hidden,
                                          no_heads=target.no_heads, inf=target.inf).to(device=ref_param.device,
                                                                                       dtype=ref_param.dtype)
        copy_native_att(fast.mha, target.mha)
        if target.training is False:
            fast.eval()
        template_embedder.template_pointwise_att = fast
    return template_embedder


def copy_native_linear(model_fast, model_ori):
    model_fast.weight.copy_(model_ori.weight)
    model_fast.bias.copy_(model_ori.bias)


def inject_embedder(model):
    """Swaps ``model.recycling_embedder`` and ``model.input_embedder`` (inject_fastnn.py:376-416); nothing is
    done for a multimer model, as in the reference."""
    if model.evoformer.blocks[0].is_multimer:
        return
    with torch.no_grad():
        target = model.recycling_embedder
        ref_param = next(target.parameters())
        fast = RecyclingEmbedder(c_m=target.c_m, c_z=target.c_z, min_bin=target.min_bin, max_bin=target.max_bin,
                                 no_bins=target.no_bins, inf=target.inf).to(device=ref_param.device, dtype=ref_param.dtype)
        copy_native_linear(fast.linear, target.linear)
        copy_layernorm(fast.layer_norm_m, target.layer_norm_m)
        copy_layernorm(fast.layer_norm_z, target.layer_norm_z)
        if target.training is False:
            fast.eval()
        model.recycling_embedder = fast

        target = model.input_embedder
        ref_param = next(target.parameters())
        fast = InputEmbedder(tf_dim=target.tf_dim, msa_dim=target.msa_dim, c_z=target.c_z, c_m=target.c_m,
                             relpos_k=target.relpos_k).to(device=ref_param.device, dtype=ref_param.dtype)
        for name in ("linear_tf_z_i", "linear_tf_z_j", "linear_tf_m", "linear_msa_m", "linear_relpos"):
            copy_linear(getattr(fast, name), getattr(target, name))
        if target.training is False:
            fast.eval()
        model.input_embedder = fast


def inject_evoformer(model):
    with torch.no_grad():
        target_module = model.evoformer
        ref_param = next(target_module.parameters())
        fast_module = EvoformerStack(
            c_m=target_module.blocks[0].msa_att_row.c_in,
            c_z=target_module.blocks[0].msa_att_row.c_z,
            c_s=target_module.linear.out_features,
            no_blocks=len(target_module.blocks),
            blocks_per_ckpt=target_module.blocks_per_ckpt,
            clear_cache_between_blocks=target_module.clear_cache_between_blocks,
            is_multimer=target_module.blocks[0].is_multimer,
        ).to(device=ref_param.device, dtype=ref_param.dtype)
        for target_block, fast_block in zip(target_module.blocks, fast_module.blocks):
            copy_evoformer_para(fast_block, target_block)
            if target_block.training is False:
                fast_block.eval()
        copy_linear(fast_module.linear, target_module.linear)
        if target_module.training is False:
            fast_module.eval()
        model.evoformer = fast_module


def inject_fastnn(model):
    """Replaces ``model.evoformer`` and, where the model has them, ``model.extra_msa_stack``, the template
    embedder's pair stack and the input / recycling embedders; returns the model (reference:
    inject_fastnn.py:418-423)."""
    inject_evoformer(model)
    if getattr(model, "extra_msa_stack", None) is not None:
        inject_extramsa(model)
    if getattr(model, "template_embedder", None) is not None and hasattr(model.template_embedder, "template_pair_stack"):
        inject_template_pair_stack(model.template_embedder)
    if getattr(model, "input_embedder", None) is not None and getattr(model, "recycling_embedder", None) is not None:
        inject_embedder(model)
    return model


def convert_nn_state_dict(sd):
    """nn-layout state dict of an Evoformer stack (``blocks.N.msa_att_row...``) -> fastnn-layout
    state dict (``blocks.N.msa.MSARowAttentionWithPairBias...``) by the same re-layout as
    ``copy_evoformer_para``; values may be tensors or numpy arrays."""
    import numpy as np

    def T(x):
        return x if isinstance(x, torch.Tensor) else torch.from_numpy(np.ascontiguousarray(x))

    out = {}
    blocks = sorted({int(k.split(".")[1]) for k in sd if k.startswith("blocks.")})

    def ln(dst, src):
        out[dst + ".weight"], out[dst + ".bias"] = T(sd[src + ".weight"]), T(sd[src + ".bias"])

    def lin(dst, src, bias=True):
        out[dst + ".weight"] = T(sd[src + ".weight"])
        if bias:
            out[dst + ".bias"] = T(sd[src + ".bias"])

    def att(dst, src, fused_out_bias):
        out[dst + ".attention.to_qkv.weight"] = torch.cat([T(sd[src + ".linear_%s.weight" % n]) for n in "qkv"], 0)
        out[dst + ".attention.gating_linear.weight"] = T(sd[src + ".linear_g.weight"])
        out[dst + ".attention.gating_bias"] = T(sd[src + ".linear_g.bias"])
        out[dst + ".attention.o_linear.weight"] = T(sd[src + ".linear_o.weight"])
        if fused_out_bias:
            out[dst + ".out_bias"] = T(sd[src + ".linear_o.bias"])
        else:
            out[dst + ".attention.o_linear.bias"] = T(sd[src + ".linear_o.bias"])

    for i in blocks:
        s, d = "blocks.%d." % i, "blocks.%d." % i
        row = d + "msa.MSARowAttentionWithPairBias"
        ln(row + ".layernormM", s + "msa_att_row.layer_norm_m")
        ln(row + ".layernormZ", s + "msa_att_row.layer_norm_z")
        out[row + ".linear_b_weights"] = T(sd[s + "msa_att_row.linear_z.weight"])
        att(row, s + "msa_att_row.mha", True)
        col = d + "msa.MSAColumnAttention"
        ln(col + ".layernormM", s + "msa_att_col._msa_att.layer_norm_m")
        att(col, s + "msa_att_col._msa_att.mha", False)
        for dst, src in ((d + "msa.MSATransition", s + "core.msa_transition"),
                         (d + "pair.PairTransition", s + "core.pair_transition")):
            ln(dst + ".norm", src + ".layer_norm")
            lin(dst + ".linear1", src + ".linear_1")
            lin(dst + ".linear2", src + ".linear_2")
        ln(d + "communication.layernormM", s + "core.outer_product_mean.layer_norm")
        lin(d + "communication.linear_a", s + "core.outer_product_mean.linear_1")
        lin(d + "communication.linear_b", s + "core.outer_product_mean.linear_2")
        lin(d + "communication.o_linear", s + "core.outer_product_mean.linear_out")
        for dst, src in ((d + "pair.TriangleMultiplicationOutgoing", s + "core.tri_mul_out"),
                         (d + "pair.TriangleMultiplicationIncoming", s + "core.tri_mul_in")):
            ln(dst + ".layernorm1", src + ".layer_norm_in")
            ln(dst + ".layernorm2", src + ".layer_norm_out")
            for nm, a, b in ((".left_right_projection", ".linear_a_p", ".linear_b_p"),
                             (".left_right_gate", ".linear_a_g", ".linear_b_g")):
                out[dst + nm + ".weight"] = torch.cat([T(sd[src + a + ".weight"]), T(sd[src + b + ".weight"])], 0)
                out[dst + nm + ".bias"] = torch.cat([T(sd[src + a + ".bias"]), T(sd[src + b + ".bias"])], 0)
            lin(dst + ".output_gate", src + ".linear_g")
            out[dst + ".output_projection.weight"] = T(sd[src + ".linear_z.weight"])
            out[dst + ".output_bias"] = T(sd[src + ".linear_z.bias"])
        for dst, src in ((d + "pair.TriangleAttentionStartingNode", s + "core.tri_att_start"),
                         (d + "pair.TriangleAttentionEndingNode", s + "core.tri_att_end")):
            ln(dst + ".layernorm1", src + ".layer_norm")
            out[dst + ".linear_b.weight"] = T(sd[src + ".linear.weight"])
            att(dst, src + ".mha", True)
    lin("linear", "linear")
    return out
