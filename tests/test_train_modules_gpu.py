"""The differentiable path of the modules around the Evoformer stack: extra-MSA stack (head-dim-8 row attention,
global column attention), template pair stack, template point-wise attention, input and recycling embedders.

As for the Evoformer stack, a call that autograd has to see runs the reference's operator sequence, and gradients
are checked against autograd through the CPU oracle in float64.  Parameter gradients travel from the oracle's
layout to the fastnn layout through the weight re-layout itself (it only copies and concatenates).

Tolerances: fp32 relative L2 <= 3e-3 per gradient tensor (one ReLU input that changes sign between the float32 run
and the float64 oracle moves every upstream gradient by ~ 1e-3 of its norm).  bf16: the forward values differ from
float64 by ~ 1e-2, so a fraction ~ 1e-2 of the transition's ReLU inputs (|a| below 1e-2 of its spread) sit on the other
side of zero, and a gradient that passes such a layer differs by the square root of that fraction in relative L2:
4e-2 .. 1e-1 is measured on every tensor of the two-block stacks, uniformly.  Bounds: <= 8e-2 on the input gradients of
the stacks, <= 1.5e-1 on their parameter gradients whose float64 norm is above 1 (the others - gradients that are
zero by construction, such as a LayerNorm bias in front of a softmax - must be finite), <= 5e-2 on the single modules
(no ReLU).
"""
import copy

import numpy as np
import pytest
import torch

from fastfold_amd.synthetic import (synth_extra_nn_state, synth_inputs, synth_pointwise_inputs,
                                    synth_pointwise_nn_state, synth_template_inputs, synth_template_nn_state)
from oracle.evoformer_ref import (EvoformerStack as OracleEvoformer, InputEmbedder as OracleInput, OracleModel,
                                  RecyclingEmbedder as OracleRecycling, TemplatePairStack as OracleTemplateStack,
                                  TemplatePointwiseAttention as OraclePointwise)

pytestmark = pytest.mark.gpu


def _rel(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def _grad_holder(ref):
    """A copy of ``ref`` whose parameters hold the gradients of ``ref``'s parameters."""
    holder = copy.deepcopy(ref)
    with torch.no_grad():
        for p, q in zip(holder.parameters(), ref.parameters()):
            p.copy_(q.grad if q.grad is not None else torch.zeros_like(q))
    return holder


def _check_param_grads(fast, want, bound, min_checked):
    checked = 0
    for name, p in fast.named_parameters():
        w = want[name].detach().double().cpu()
        assert p.grad is not None, name
        assert bool(torch.isfinite(p.grad.float()).all()), name
        err = float((p.grad.double().cpu() - w).norm())
        if p.dtype == torch.float32 or float(w.norm()) > 1.0:
            assert err <= bound * float(w.norm()) + 1e-3, (name, err, float(w.norm()))
        checked += float(w.norm()) > 1.0
    assert checked >= min_checked, checked


class _Holder(torch.nn.Module):
    pass


# ------------------------------------------------------------------------------------ extra-MSA stack ----
def _extra(seed, nb):
    model = OracleModel(no_blocks=1, extra_msa_kwargs=dict(no_blocks=nb)).eval()
    sd = synth_extra_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=True)
    model.extra_msa_stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return model


def _extra_fast(model, dev, dtype):
    from fastfold_amd.utils.inject_fastnn import inject_extramsa
    m2 = copy.deepcopy(model)
    inject_extramsa(m2)
    return m2.extra_msa_stack.to(device=dev, dtype=dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nb,s,r,tail", [(2, 24, 40, 0.1), (1, 70, 33, 0.0)])
def test_extra_msa_stack_gradients(dev, dtype, nb, s, r, tail):
    model = _extra(61, nb)
    m, z, mm, pm = synth_inputs(61, s, r, c_m=64, mask_tail_frac=tail)
    if dtype == torch.bfloat16:
        m, z = (torch.from_numpy(x).to(dtype).float().numpy() for x in (m, z))
    nv = r - int(round(tail * r))
    g = torch.Generator().manual_seed(9)
    cot = torch.randn(r, r, 128, generator=g)
    cot[nv:] = 0
    cot[:, nv:] = 0

    ref = copy.deepcopy(model).double()
    mi, zi = (torch.from_numpy(t).double().requires_grad_() for t in (m, z))
    out = ref.extra_msa_stack(mi, zi, msa_mask=torch.from_numpy(mm).double(), pair_mask=torch.from_numpy(pm).double(),
                              _mask_trans=False)
    (out * cot.double()).sum().backward()
    from fastfold_amd.utils.inject_fastnn import inject_extramsa
    holder = _grad_holder(ref)
    inject_extramsa(holder)
    want = dict(holder.extra_msa_stack.named_parameters())

    fast = _extra_fast(model, dev, dtype).eval()
    fm, fz = (torch.from_numpy(t).to(dev, dtype).requires_grad_() for t in (m, z))
    got = fast(fm, fz, chunk_size=None, msa_mask=torch.from_numpy(mm).to(dev, dtype),
               pair_mask=torch.from_numpy(pm).to(dev, dtype))
    assert got.grad_fn is not None
    with torch.no_grad():                                   # the fused forward-only launches agree with it
        fused = fast(fm, fz, chunk_size=None, msa_mask=torch.from_numpy(mm).to(dev, dtype),
                     pair_mask=torch.from_numpy(pm).to(dev, dtype))
    fwd = 2e-5 if dtype == torch.float32 else 2e-2
    assert _rel(got[:nv, :nv], out[:nv, :nv]) <= fwd, _rel(got[:nv, :nv], out[:nv, :nv])
    assert _rel(got[:nv, :nv], fused[:nv, :nv]) <= fwd, _rel(got[:nv, :nv], fused[:nv, :nv])
    (got.float() * cot.to(dev)).sum().backward()
    bound = 3e-3 if dtype == torch.float32 else 8e-2
    assert _rel(fm.grad, mi.grad) <= bound, _rel(fm.grad, mi.grad)
    assert _rel(fz.grad, zi.grad) <= bound, _rel(fz.grad, zi.grad)
    # the MSA stack of the last block feeds nothing that reaches the output pair tensor except through the outer
    # product mean: its column attention and transition still receive gradients, all finite
    _check_param_grads(fast, want, 3e-3 if dtype == torch.float32 else 1.5e-1, 40 * nb)


def test_global_attention_module_gradients(dev):
    """GlobalAttention on its own (already normalised input), with a fully masked column."""
    from fastfold_amd.model.fastnn.ops import GlobalAttention
    from oracle.evoformer_ref import GlobalAttention as OracleGA
    torch.manual_seed(3)
    ref = OracleGA(c_in=64, c_hidden=8, no_heads=8, inf=1e9, eps=1e-10).double()
    with torch.no_grad():
        for p in ref.parameters():
            p.copy_(0.2 * torch.randn_like(p))
    fast = GlobalAttention(qkv_dim=64, c=8, n_head=8, out_dim=64)
    with torch.no_grad():
        fast.to_q.weight.copy_(ref.linear_q.weight)
        fast.to_kv.weight.copy_(torch.cat([ref.linear_k.weight, ref.linear_v.weight], 0))
        fast.gating_linear.weight.copy_(ref.linear_g.weight)
        fast.gating_bias.copy_(ref.linear_g.bias)
        fast.o_linear.weight.copy_(ref.linear_o.weight)
        fast.o_linear.bias.copy_(ref.linear_o.bias)
    fast = fast.to(dev).eval()
    R, S = 7, 45
    x = torch.randn(1, R, S, 64)
    mask = (torch.rand(1, R, S) > 0.3).float()
    mask[0, 2] = 0
    cot = torch.randn(1, R, S, 64)
    xi = x.double().requires_grad_()
    out = ref(xi, mask.double())
    (out * cot.double()).sum().backward()
    fx = x.to(dev).requires_grad_()
    got = fast(fx, mask.to(dev))
    assert _rel(got, out) <= 2e-5, _rel(got, out)
    (got * cot.to(dev)).sum().backward()
    assert _rel(fx.grad, xi.grad) <= 1e-4, _rel(fx.grad, xi.grad)
    assert _rel(fast.to_q.weight.grad, ref.linear_q.weight.grad) <= 1e-4
    assert _rel(fast.to_kv.weight.grad, torch.cat([ref.linear_k.weight.grad, ref.linear_v.weight.grad], 0)) <= 1e-4
    assert _rel(fast.gating_linear.weight.grad, ref.linear_g.weight.grad) <= 1e-4
    assert _rel(fast.gating_bias.grad, ref.linear_g.bias.grad) <= 1e-4
    assert _rel(fast.o_linear.weight.grad, ref.linear_o.weight.grad) <= 1e-4


# ------------------------------------------------------------------------------- template pair stack ----
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_template_pair_stack_gradients(dev, dtype):
    from fastfold_amd.utils.inject_fastnn import inject_template_pair_stack
    nb, nt, r, tail = 2, 2, 40, 0.1
    stack = OracleTemplateStack(no_blocks=nb).eval()
    sd = synth_template_nn_state(seed=71, no_blocks=nb, fan_in_scaled=True)
    stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    t, pm = synth_template_inputs(71, nt, r, mask_tail_frac=tail)
    if dtype == torch.bfloat16:
        t = torch.from_numpy(t).to(dtype).float().numpy()
    nv = r - int(round(tail * r))
    cot = torch.randn(nt, r, r, 64, generator=torch.Generator().manual_seed(4))
    cot[:, nv:] = 0
    cot[:, :, nv:] = 0

    ref = copy.deepcopy(stack).double()
    ti = torch.from_numpy(t).double().requires_grad_()
    out = ref(ti, torch.from_numpy(pm)[None].double(), _mask_trans=False)
    (out * cot.double()).sum().backward()
    e = _Holder()
    e.template_pair_stack = _grad_holder(ref)
    want = dict(inject_template_pair_stack(e).template_pair_stack.named_parameters())

    e = _Holder()
    e.template_pair_stack = copy.deepcopy(stack)
    fast = inject_template_pair_stack(e).template_pair_stack.to(dev, dtype).eval()
    ft = torch.from_numpy(t).to(dev, dtype).requires_grad_()
    keep = ft.detach().clone()
    got = fast(ft, torch.from_numpy(pm)[None].to(dev, dtype), chunk_size=None)
    assert got.grad_fn is not None and torch.equal(ft.detach(), keep)
    assert _rel(got[:, :nv, :nv], out[:, :nv, :nv]) <= (2e-5 if dtype == torch.float32 else 2e-2)
    (got.float() * cot.to(dev)).sum().backward()
    bound = 3e-3 if dtype == torch.float32 else 8e-2
    assert _rel(ft.grad, ti.grad) <= bound, _rel(ft.grad, ti.grad)
    _check_param_grads(fast, want, 3e-3 if dtype == torch.float32 else 1.5e-1, 25 * nb)


# --------------------------------------------------------------------- template point-wise attention ----
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nt,r,tmask", [(4, 12, (1, 0, 1, 1)), (2, 9, (0, 0)), (8, 20, (1, 1, 0, 1, 1, 0, 1, 1))])
def test_template_pointwise_attention_gradients(dev, dtype, nt, r, tmask):
    from fastfold_amd.model.fastnn import TemplatePointwiseAttention
    sd = {k: torch.from_numpy(v) for k, v in synth_pointwise_nn_state(seed=5).items()}
    ref = OraclePointwise().double()
    ref.load_state_dict(sd, strict=True)
    fast = TemplatePointwiseAttention(c_t=64, c_z=128, c_hidden=16, no_heads=4, inf=1e5)
    fast.load_state_dict(sd, strict=True)
    fast = fast.to(dev, dtype).eval()
    t, z = synth_pointwise_inputs(7, nt, r)
    if dtype == torch.bfloat16:
        t, z = (torch.from_numpy(x).to(dtype).float().numpy() for x in (t, z))
    tm = torch.tensor(tmask, dtype=torch.float32)
    cot = torch.randn(r, r, 128, generator=torch.Generator().manual_seed(2))
    ti, zi = (torch.from_numpy(x).double().requires_grad_() for x in (t, z))
    out = ref(ti, zi, template_mask=tm.double()) * float(tm.sum() > 0)
    (out * cot.double()).sum().backward()
    ft, fz = (torch.from_numpy(x).to(dev, dtype).requires_grad_() for x in (t, z))
    got = fast(ft, fz, template_mask=tm.to(dev))
    (got.float() * cot.to(dev)).sum().backward()
    if not any(tmask):
        assert float(got.detach().abs().max()) == 0.0 and float(ft.grad.abs().max()) == 0.0 and float(fz.grad.abs().max()) == 0.0
        return
    bound = 1e-4 if dtype == torch.float32 else 5e-2
    assert _rel(got, out) <= (2e-5 if dtype == torch.float32 else 2e-2)
    assert _rel(ft.grad, ti.grad) <= bound, _rel(ft.grad, ti.grad)
    assert _rel(fz.grad, zi.grad) <= bound, _rel(fz.grad, zi.grad)
    want = dict(ref.named_parameters())
    for name, p in fast.named_parameters():
        assert _rel(p.grad, want[name].grad) <= bound, (name, _rel(p.grad, want[name].grad))


# -------------------------------------------------------------------------------------------- embedders ----
class _EmbModel(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.evoformer = OracleEvoformer(no_blocks=1)
        self.input_embedder = OracleInput(tf_dim=22, msa_dim=49, c_z=128, c_m=256, relpos_k=32)
        self.recycling_embedder = OracleRecycling(c_m=256, c_z=128, min_bin=3.25, max_bin=20.75, no_bins=15, inf=1e8)


def _emb_models(dev, dtype):
    from fastfold_amd.utils.inject_fastnn import inject_embedder
    torch.manual_seed(0)
    ref = _EmbModel()
    with torch.no_grad():
        for mod in (ref.input_embedder, ref.recycling_embedder):
            for n, p in mod.named_parameters():
                p.copy_((1.0 if "layer_norm" in n and n.endswith("weight") else 0.0) + 0.3 * torch.randn_like(p))
    fast = copy.deepcopy(ref)
    inject_embedder(fast)
    return ref.double(), fast.to(dev, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_input_embedder_gradients(dev, dtype):
    ref, fast = _emb_models(dev, dtype)
    s, r = 5, 37
    rng = np.random.RandomState(1)
    tf = torch.from_numpy(rng.standard_normal((r, 22)).astype(np.float32)).to(dtype).float()
    msa = torch.from_numpy(rng.standard_normal((s, r, 49)).astype(np.float32)).to(dtype).float()
    ri = torch.arange(r) + torch.from_numpy((np.arange(r) >= r // 2) * 200)
    cm, cz = torch.randn(s, r, 256), torch.randn(r, r, 128)
    tfi, msai = tf.double().requires_grad_(), msa.double().requires_grad_()
    rm, rz = ref.input_embedder(tfi, ri, msai)
    ((rm * cm.double()).sum() + (rz * cz.double()).sum()).backward()
    ftf, fmsa = tf.to(dev, dtype).requires_grad_(), msa.to(dev, dtype).requires_grad_()
    gm, gz = fast.input_embedder(ftf, ri.to(dev), fmsa)
    assert gm.grad_fn is not None and gz.grad_fn is not None
    fwd = 2e-5 if dtype == torch.float32 else 2e-2
    assert _rel(gm, rm) <= fwd and _rel(gz, rz) <= fwd
    ((gm.float() * cm.to(dev)).sum() + (gz.float() * cz.to(dev)).sum()).backward()
    bound = 1e-4 if dtype == torch.float32 else 5e-2
    assert _rel(ftf.grad, tfi.grad) <= bound and _rel(fmsa.grad, msai.grad) <= bound
    want = dict(ref.input_embedder.named_parameters())
    for name, p in fast.input_embedder.named_parameters():
        assert _rel(p.grad, want[name].grad) <= bound, (name, _rel(p.grad, want[name].grad))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_recycling_embedder_gradients(dev, dtype):
    ref, fast = _emb_models(dev, dtype)
    r = 23
    rng = np.random.RandomState(2)
    m = torch.from_numpy(rng.standard_normal((r, 256)).astype(np.float32)).to(dtype).float()
    z = torch.from_numpy(rng.standard_normal((r, r, 128)).astype(np.float32)).to(dtype).float()
    x = torch.from_numpy((rng.standard_normal((r, 3)) * 9.0).astype(np.float32))
    cm, cz = torch.randn(r, 256), torch.randn(r, r, 128)
    mi, zi = m.double().requires_grad_(), z.double().requires_grad_()
    rm, rz = ref.recycling_embedder(mi, zi, x.double())
    ((rm * cm.double()).sum() + (rz * cz.double()).sum()).backward()
    fm, fz = m.to(dev, dtype).requires_grad_(), z.to(dev, dtype).requires_grad_()
    keep = fz.detach().clone()
    gm, gz = fast.recycling_embedder(fm, fz, x.to(dev))
    assert torch.equal(fz.detach(), keep)
    fwd = 2e-5 if dtype == torch.float32 else 2e-2
    assert _rel(gm, rm) <= fwd and _rel(gz, rz) <= fwd
    ((gm.float() * cm.to(dev)).sum() + (gz.float() * cz.to(dev)).sum()).backward()
    bound = 1e-4 if dtype == torch.float32 else 5e-2
    assert _rel(fm.grad, mi.grad) <= bound and _rel(fz.grad, zi.grad) <= bound
    want = dict(ref.recycling_embedder.named_parameters())
    for name, p in fast.recycling_embedder.named_parameters():
        assert _rel(p.grad, want[name].grad) <= bound, (name, _rel(p.grad, want[name].grad))
