"""Writes tests/golden/evoformer_nn_golden.npz, extra_msa_nn_golden.npz and template_pair_nn_golden.npz by
running the REFERENCE's own ``fastfold.model.nn.evoformer.EvoformerStack`` / ``ExtraMSAStack`` and
``fastfold.model.nn.template.TemplatePairStack`` (plain PyTorch, CPU, fp32) on seeded synthetic weights
and inputs.  Run only in the build container, where /root/reference is mounted:

    python tests/golden/make_golden.py            # Evoformer stack
    python tests/golden/make_golden.py extra      # extra-MSA stack
    python tests/golden/make_golden.py template   # template pair stack
    python tests/golden/make_golden.py pointwise  # template point-wise attention
    python tests/golden/make_golden.py cfg4       # one Evoformer block at N_seq=128, N_res=1024 (sampled outputs)
    python tests/golden/make_golden.py cfg4_deep 48   # the 48-block stack at that shape (about an hour of CPU)

The fixture pins what closed forms cannot: the composition of a block (order of the
sub-updates, residual placement, OPM reading the updated MSA), the q/k/v and left/right
concatenation order used when weights are re-packed, and mask handling with padded residues.
Only inputs' seeds and the reference's outputs are stored; no reference source travels.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, "/root/reference")

from fastfold_amd.synthetic import (synth_extra_nn_state, synth_nn_state, synth_inputs,  # noqa: E402
                                    synth_template_inputs, synth_template_nn_state)

CASES = [
    # name, seed, no_blocks, n_seq, n_res, mask_tail_frac, fan_in_scaled
    ("b1_s8_r12_pad", 11, 1, 8, 12, 0.17, True),
    ("b2_s6_r10_full", 12, 2, 6, 10, 0.0, True),
    ("b1_s5_r9_std002", 13, 1, 5, 9, 0.0, False),
]


def main():
    from fastfold.model.nn.evoformer import EvoformerStack  # the reference

    out = {}
    for name, seed, nb, s, r, tail, fis in CASES:
        torch.manual_seed(0)
        stack = EvoformerStack(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128,
                               c_hidden_pair_att=32, c_s=384, no_heads_msa=8, no_heads_pair=4, no_blocks=nb,
                               transition_n=4, msa_dropout=0.15, pair_dropout=0.25, blocks_per_ckpt=1,
                               inf=1e9, eps=1e-8).eval()
        sd = synth_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis)
        missing, unexpected = stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
        assert not missing and not unexpected
        m, z, msa_mask, pair_mask = synth_inputs(seed, s, r, mask_tail_frac=tail)
        with torch.no_grad():
            mo, zo, so = stack(torch.from_numpy(m), torch.from_numpy(z), torch.from_numpy(msa_mask),
                               torch.from_numpy(pair_mask), chunk_size=None, _mask_trans=False)
        out[name + ".m"] = mo.numpy()
        out[name + ".z"] = zo.numpy()
        out[name + ".s"] = so.numpy()
        out[name + ".cfg"] = np.array([seed, nb, s, r, int(round(tail * 100)), int(fis)], dtype=np.int64)
        print(name, "m", float(np.abs(mo.numpy() - m).mean()), "z", float(np.abs(zo.numpy() - z).mean()))
    np.savez_compressed(os.path.join(HERE, "evoformer_nn_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "evoformer_nn_golden.npz"))


EXTRA_CASES = [
    # name, seed, no_blocks, n_extra, n_res, mask_tail_frac, fan_in_scaled
    ("x1_s9_r12_pad", 21, 1, 9, 12, 0.17, True),
    ("x2_s7_r10_full", 22, 2, 7, 10, 0.0, True),
    ("x1_s40_r6_std002", 23, 1, 40, 6, 0.34, False),
]


def main_extra():
    from fastfold.model.nn.evoformer import ExtraMSAStack  # the reference

    out = {}
    for name, seed, nb, s, r, tail, fis in EXTRA_CASES:
        torch.manual_seed(0)
        stack = ExtraMSAStack(c_m=64, c_z=128, c_hidden_msa_att=8, c_hidden_opm=32, c_hidden_mul=128,
                              c_hidden_pair_att=32, no_heads_msa=8, no_heads_pair=4, no_blocks=nb,
                              transition_n=4, msa_dropout=0.15, pair_dropout=0.25, inf=1e9, eps=1e-10,
                              ckpt=False).eval()
        sd = synth_extra_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis)
        missing, unexpected = stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
        assert not missing and not unexpected
        m, z, msa_mask, pair_mask = synth_inputs(seed, s, r, c_m=64, mask_tail_frac=tail)
        with torch.no_grad():
            zo = stack(torch.from_numpy(m), torch.from_numpy(z), chunk_size=None,
                       msa_mask=torch.from_numpy(msa_mask), pair_mask=torch.from_numpy(pair_mask))
        out[name + ".z"] = zo.numpy()
        out[name + ".cfg"] = np.array([seed, nb, s, r, int(round(tail * 100)), int(fis)], dtype=np.int64)
        print(name, "z", float(np.abs(zo.numpy() - z).mean()))
    np.savez_compressed(os.path.join(HERE, "extra_msa_nn_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "extra_msa_nn_golden.npz"))


TEMPLATE_CASES = [
    # name, seed, no_blocks, n_templ, n_res, mask_tail_frac, fan_in_scaled
    ("t2_n1_r12_pad", 31, 2, 1, 12, 0.17, True),
    ("t2_n3_r9_full", 32, 2, 3, 9, 0.0, True),
    ("t1_n2_r10_std002", 33, 1, 2, 10, 0.2, False),
]


def main_template():
    from fastfold.model.nn.template import TemplatePairStack  # the reference

    out = {}
    for name, seed, nb, nt, r, tail, fis in TEMPLATE_CASES:
        torch.manual_seed(0)
        stack = TemplatePairStack(c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_blocks=nb, no_heads=4,
                                  pair_transition_n=2, dropout_rate=0.25, blocks_per_ckpt=None, inf=1e9).eval()
        sd = synth_template_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fis)
        missing, unexpected = stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
        assert not missing and not unexpected
        t, pair_mask = synth_template_inputs(seed, nt, r, mask_tail_frac=tail)
        with torch.no_grad():
            to = stack(torch.from_numpy(t), torch.from_numpy(pair_mask)[None], chunk_size=None, _mask_trans=False)
        out[name + ".t"] = to.numpy()
        out[name + ".cfg"] = np.array([seed, nb, nt, r, int(round(tail * 100)), int(fis)], dtype=np.int64)
        print(name, "t", float(np.abs(to.numpy() - t).mean()))
    np.savez_compressed(os.path.join(HERE, "template_pair_nn_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "template_pair_nn_golden.npz"))


POINTWISE_CASES = [
    # name, seed, n_templ, n_res, template_mask
    ("pw_all", 61, 4, 12, (1.0, 1.0, 1.0, 1.0)),
    ("pw_masked", 62, 4, 9, (1.0, 0.0, 1.0, 0.0)),
    ("pw_one", 63, 1, 7, (1.0,)),
    ("pw_none", 64, 2, 5, (0.0, 0.0)),
]


def main_pointwise():
    from fastfold.model.nn.template import TemplatePointwiseAttention  # the reference
    from fastfold_amd.synthetic import synth_pointwise_inputs, synth_pointwise_nn_state

    out = {}
    for name, seed, nt, r, tmask in POINTWISE_CASES:
        mod = TemplatePointwiseAttention(c_t=64, c_z=128, c_hidden=16, no_heads=4, inf=1e5).eval()
        sd = synth_pointwise_nn_state(seed=seed)
        missing, unexpected = mod.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
        assert not missing and not unexpected
        t, z = synth_pointwise_inputs(seed, nt, r)
        with torch.no_grad():
            upd = mod(torch.from_numpy(t), torch.from_numpy(z), template_mask=torch.tensor(tmask), chunk_size=None)
        out[name + ".out"] = upd.numpy()
        out[name + ".cfg"] = np.array([seed, nt, r] + [int(x) for x in tmask], dtype=np.int64)
        print(name, "mean |update|", float(np.abs(upd.numpy()).mean()))
    np.savez_compressed(os.path.join(HERE, "template_pointwise_nn_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "template_pointwise_nn_golden.npz"))


CFG4_CASES = [
    # name, seed, fan_in_scaled
    ("cfg4_fanin", 71, True),
    ("cfg4_std002", 72, False),
]


def cfg4_sample_indices(seed, n_seq, n_valid):
    """Index sets of the stored sample: 16 sequences, 48 row residues, 48 column residues, all un-masked, drawn
    without replacement (random positions inside the kernels' 32- and 256-wide tiles, unlike a strided sample)."""
    rng = np.random.RandomState(seed + 5)
    return (np.sort(rng.choice(n_seq, 16, replace=False)), np.sort(rng.choice(n_valid, 48, replace=False)),
            np.sort(rng.choice(n_valid, 48, replace=False)))


def main_cfg4():
    """The benchmark's headline shape: one block, N_seq = 128, N_res = 1024, last 5 % of the residues masked, inputs
    rounded to bf16 (what the bf16 HIP path receives).  The reference runs in fp32 with its own chunking
    (chunk_size = 64) to bound memory; only a sample of the outputs is stored."""
    from fastfold.model.nn.evoformer import EvoformerStack  # the reference
    from fastfold_amd.synthetic import bf16_round

    s, r, tail = 128, 1024, 0.05
    nv = r - int(round(tail * r))
    out = {}
    for name, seed, fis in CFG4_CASES:
        stack = EvoformerStack(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128,
                               c_hidden_pair_att=32, c_s=384, no_heads_msa=8, no_heads_pair=4, no_blocks=1,
                               transition_n=4, msa_dropout=0.15, pair_dropout=0.25, blocks_per_ckpt=1,
                               inf=1e9, eps=1e-8).eval()
        sd = synth_nn_state(seed=seed, no_blocks=1, fan_in_scaled=fis)
        stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
        m, z, msa_mask, pair_mask = synth_inputs(seed, s, r, mask_tail_frac=tail)
        m, z = bf16_round(m), bf16_round(z)
        with torch.no_grad():
            mo, zo, so = stack(torch.from_numpy(m), torch.from_numpy(z), torch.from_numpy(msa_mask),
                               torch.from_numpy(pair_mask), chunk_size=64, _mask_trans=False)
        S, I, J = cfg4_sample_indices(seed, s, nv)
        out[name + ".S"], out[name + ".I"], out[name + ".J"] = S, I, J
        out[name + ".m"] = mo.numpy()[S][:, J]
        out[name + ".z"] = zo.numpy()[I][:, J]
        out[name + ".s"] = so.numpy()[J]
        out[name + ".cfg"] = np.array([seed, 1, s, r, int(round(tail * 100)), int(fis)], dtype=np.int64)
        print(name, "m", float(np.abs(mo.numpy() - m)[:, :nv].mean()), "z", float(np.abs(zo.numpy() - z)[:nv, :nv].mean()),
              flush=True)
    np.savez_compressed(os.path.join(HERE, "evoformer_cfg4_nn_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "evoformer_cfg4_nn_golden.npz"))


def main_cfg4_deep(no_blocks=48):
    """The headline acceptance: the 48-block stack at N_seq = 128, N_res = 1024, last 5 % of the residues masked, the
    benchmark's N(0, 0.02^2) weights, inputs rounded to bf16.  The reference runs in fp32 with chunk_size = 64 (about
    an hour on eight host cores); a sample of the outputs (random un-masked sequences / residues) and the norms of the
    full outputs and of the accumulated update are stored."""
    import time
    from fastfold.model.nn.evoformer import EvoformerStack  # the reference
    from fastfold_amd.synthetic import bf16_round

    s, r, tail, seed = 128, 1024, 0.05, 73
    nv = r - int(round(tail * r))
    stack = EvoformerStack(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128,
                           c_hidden_pair_att=32, c_s=384, no_heads_msa=8, no_heads_pair=4, no_blocks=no_blocks,
                           transition_n=4, msa_dropout=0.15, pair_dropout=0.25, blocks_per_ckpt=1,
                           inf=1e9, eps=1e-8).eval()
    sd = synth_nn_state(seed=seed, no_blocks=no_blocks, fan_in_scaled=False)
    stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    m, z, msa_mask, pair_mask = synth_inputs(seed, s, r, mask_tail_frac=tail)
    m, z = bf16_round(m), bf16_round(z)
    t0 = time.time()
    with torch.no_grad():
        mo, zo, so = stack(torch.from_numpy(m), torch.from_numpy(z), torch.from_numpy(msa_mask),
                           torch.from_numpy(pair_mask), chunk_size=64, _mask_trans=False)
    print("reference: %d blocks in %.0f s" % (no_blocks, time.time() - t0), flush=True)
    S, I, J = cfg4_sample_indices(seed, s, nv)
    mo, zo, so = mo.numpy(), zo.numpy(), so.numpy()
    name = "cfg4_deep%d" % no_blocks
    out = {name + ".S": S, name + ".I": I, name + ".J": J,
           name + ".m": mo[S][:, J], name + ".z": zo[I][:, J], name + ".s": so[J],
           name + ".cfg": np.array([seed, no_blocks, s, r, int(round(tail * 100)), 0], dtype=np.int64),
           # norms over the un-masked region: of the outputs and of the accumulated update (out - in)
           name + ".norms": np.array([np.linalg.norm(mo[:, :nv]), np.linalg.norm(zo[:nv, :nv]), np.linalg.norm(so[:nv]),
                                      np.linalg.norm((mo - m)[:, :nv]), np.linalg.norm((zo - z)[:nv, :nv])], dtype=np.float64)}
    path = os.path.join(HERE, "evoformer_%s_nn_golden.npz" % name)
    np.savez_compressed(path, **out)
    print("wrote", path)


if __name__ == "__main__":
    if "cfg4_deep" in sys.argv[1:]:
        main_cfg4_deep(int(sys.argv[sys.argv.index("cfg4_deep") + 1]) if len(sys.argv) > sys.argv.index("cfg4_deep") + 1 else 48)
    elif "cfg4" in sys.argv[1:]:
        main_cfg4()
    elif "pointwise" in sys.argv[1:]:
        main_pointwise()
    elif "template" in sys.argv[1:]:
        main_template()
    elif "extra" in sys.argv[1:]:
        main_extra()
    else:
        main()
