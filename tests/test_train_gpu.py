"""The differentiable path of the fastnn modules (what benchmark/perf.py's forward + backward mode and
tests/test_train.py exercise in the reference): a call that autograd has to see runs the reference's own operator
sequence, with the HIP LayerNorm / attention-core / elementwise kernels and their backward passes.

Gradients are checked against autograd through the CPU oracle in float64 (oracle.evoformer_ref, whose forward is
pinned by the reference's golden vectors).  Parameter gradients are carried from the oracle's layout to the fastnn
layout by the weight re-layout itself: it only copies and concatenates, so applied to a model whose parameters hold
their gradients it yields the gradients of the re-laid-out parameters.

Tolerances: fp32 relative L2 <= 3e-3 per gradient tensor (1e-6 is what is measured when no ReLU input changes sign
between the float32 run and the float64 oracle; one such flip among the 2 M hidden activations of the pair
transition moves every upstream gradient by ~ 1e-3 of its norm, and about one is expected per block at these
sizes); bf16 relative L2 <= 5e-2 on the input gradients and <= 1.5e-1 on the parameter gradients (see
test_stack_gradients_with_checkpointing).
"""
import copy

import numpy as np
import pytest
import torch

from fastfold_amd.synthetic import synth_inputs, synth_nn_state
from oracle.evoformer_ref import OracleModel

pytestmark = pytest.mark.gpu

KW = dict(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128, c_hidden_pair_att=32, c_s=384,
          no_heads_msa=8, no_heads_pair=4, transition_n=4, msa_dropout=0.15, pair_dropout=0.25, blocks_per_ckpt=1,
          inf=1e9, eps=1e-8)


def _oracle(seed, nb):
    model = OracleModel(no_blocks=nb, **KW).eval()
    sd = synth_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=True, std=0.02)
    model.evoformer.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return model


def _fast(model, dev, dtype):
    from fastfold_amd.utils.inject_fastnn import inject_fastnn
    return inject_fastnn(copy.deepcopy(model)).evoformer.to(device=dev, dtype=dtype)


def _rel(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def _oracle_run(model, m, z, mm, pm, cot):
    """Outputs, input gradients and (in the fastnn layout) parameter gradients of the float64 oracle."""
    ref = copy.deepcopy(model).double()
    mi, zi = (torch.from_numpy(t).double().requires_grad_() for t in (m, z))
    out = ref.evoformer(mi, zi, torch.from_numpy(mm).double(), torch.from_numpy(pm).double(), _mask_trans=False)
    sum((o * c.double()).sum() for o, c in zip(out, cot)).backward()
    holder = copy.deepcopy(ref)
    with torch.no_grad():
        for p, q in zip(holder.parameters(), ref.parameters()):
            p.copy_(q.grad if q.grad is not None else torch.zeros_like(q))
    from fastfold_amd.utils.inject_fastnn import inject_fastnn
    pgrads = dict(inject_fastnn(holder).evoformer.named_parameters())
    return [o.detach() for o in out], (mi.grad, zi.grad), pgrads


def _mask_cotangents(cot, r, tail):
    """Zero cotangents at masked residues: what a module leaves there is unspecified (a softmax over keys that are
    all masked is uniform in the reference's kernel and input-dependent in the oracle), and nothing at a valid
    residue reads it."""
    nv = r - int(round(tail * r))
    cot[0][:, nv:] = 0
    cot[1][nv:] = 0
    cot[1][:, nv:] = 0
    cot[2][nv:] = 0
    return nv


@pytest.mark.parametrize("nb,s,r,tail", [(1, 12, 40, 0.2), (2, 33, 64, 0.0)])
def test_stack_gradients_fp32(dev, nb, s, r, tail):
    model = _oracle(31, nb)
    m, z, mm, pm = synth_inputs(31, s, r, mask_tail_frac=tail)
    g = torch.Generator().manual_seed(5)
    cot = [torch.randn(s, r, KW["c_m"], generator=g), torch.randn(r, r, KW["c_z"], generator=g),
           torch.randn(r, KW["c_s"], generator=g)]
    nv = _mask_cotangents(cot, r, tail)
    ref_out, ref_gin, ref_gp = _oracle_run(model, m, z, mm, pm, cot)

    fast = _fast(model, dev, torch.float32).eval()            # eval: no dropout; gradients still flow
    mi, zi = (torch.from_numpy(t).to(dev).requires_grad_() for t in (m, z))
    out = fast(mi, zi, torch.from_numpy(mm).to(dev), torch.from_numpy(pm).to(dev), chunk_size=None)
    assert all(o.grad_fn is not None for o in out)
    with torch.no_grad():                                       # the fused forward-only launches agree with it
        fused = fast(mi, zi, torch.from_numpy(mm).to(dev), torch.from_numpy(pm).to(dev), chunk_size=None)
    for o, f, ref in zip((out[0][:, :nv], out[1][:nv, :nv], out[2][:nv]),
                         (fused[0][:, :nv], fused[1][:nv, :nv], fused[2][:nv]),
                         (ref_out[0][:, :nv], ref_out[1][:nv, :nv], ref_out[2][:nv])):
        assert _rel(o, ref) <= 2e-5, _rel(o, ref)
        assert _rel(o, f) <= 2e-5, _rel(o, f)
    sum((o * c.to(dev)).sum() for o, c in zip(out, cot)).backward()
    assert _rel(mi.grad, ref_gin[0]) <= 3e-3, _rel(mi.grad, ref_gin[0])
    assert _rel(zi.grad, ref_gin[1]) <= 3e-3, _rel(zi.grad, ref_gin[1])
    checked = 0
    for name, p in fast.named_parameters():
        want = ref_gp[name].detach().double()
        assert p.grad is not None, name
        err = float((p.grad.double().cpu() - want).norm())
        # the absolute term covers gradients that are zero by construction (a LayerNorm bias that shifts every logit
        # of a softmax row by the same amount): the others have norms of 30 .. 10 000 here
        assert err <= 3e-3 * float(want.norm()) + 1e-3, (name, err, float(want.norm()))
        checked += float(want.norm()) > 1.0
    assert checked >= 70 * nb, checked


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_stack_gradients_with_checkpointing(dev, dtype):
    """A training step in train() mode with the dropout probabilities forced to zero (so that it is comparable): the
    blocks are re-run in the backward pass (blocks_per_ckpt = 1) and give the gradients of the un-checkpointed run -
    to 1e-4 in fp32 (the pair-bias and LayerNorm parameter gradients are accumulated with floating-point atomics, so
    not bit for bit); in bf16, where a last-bit difference there becomes a rounding step of 4e-3 further up, both runs
    are held to the bf16 bound against the float64 oracle instead."""
    nb, s, r = 2, 16, 48
    model = _oracle(32, nb)
    m, z, mm, pm = synth_inputs(32, s, r, mask_tail_frac=0.1)
    g = torch.Generator().manual_seed(6)
    cot = [torch.randn(s, r, KW["c_m"], generator=g), torch.randn(r, r, KW["c_z"], generator=g),
           torch.randn(r, KW["c_s"], generator=g)]
    _mask_cotangents(cot, r, 0.1)
    _, ref_gin, ref_gp = _oracle_run(model, m, z, mm, pm, cot)
    fast = _fast(model, dev, dtype).train()
    for mod in fast.modules():
        if hasattr(mod, "p_drop"):
            mod.p_drop = 0.0
    grads = []
    for per in (1, None):
        fast.blocks_per_ckpt = per
        mi, zi = (torch.from_numpy(t).to(dev, dtype).requires_grad_() for t in (m, z))
        out = fast(mi, zi, torch.from_numpy(mm).to(dev, dtype), torch.from_numpy(pm).to(dev, dtype), chunk_size=None)
        sum((o.float() * c.to(dev)).sum() for o, c in zip(out, cot)).backward()
        grads.append((mi.grad.clone(), zi.grad.clone()))
        # parameter gradients against the oracle, in both precisions.  bf16: forward values differ from float64 by
        # ~ 1e-2, so about that fraction of the transitions' ReLU inputs sit on the other side of zero and every
        # gradient upstream of one moves by the square root of that fraction (4e-2 .. 1e-1 measured, uniformly)
        pbound = 3e-3 if dtype == torch.float32 else 1.5e-1
        checked = 0
        for name, p in fast.named_parameters():
            want = ref_gp[name].detach().double()
            assert p.grad is not None and bool(torch.isfinite(p.grad.float()).all()), name
            if dtype == torch.float32 or float(want.norm()) > 1.0:
                err = float((p.grad.double().cpu() - want).norm())
                assert err <= pbound * float(want.norm()) + 1e-3, (name, err, float(want.norm()))
                checked += 1
        assert checked >= 70 * nb, checked
        fast.zero_grad()
    if dtype == torch.float32:
        assert _rel(grads[0][0], grads[1][0]) <= 1e-4 and _rel(grads[0][1], grads[1][1]) <= 1e-4
    bound = 3e-3 if dtype == torch.float32 else 5e-2
    for gm, gz in grads:
        assert _rel(gm, ref_gin[0]) <= bound, _rel(gm, ref_gin[0])
        assert _rel(gz, ref_gin[1]) <= bound, _rel(gz, ref_gin[1])


@pytest.mark.parametrize("rows,n,k", [(9216, 128, 128), (16384, 512, 128), (40960, 32, 256)])
def test_linear_weight_gradient_slab_branch(dev, rows, n, k):
    """bf16 projections over 8192 rows or more reduce their weight gradient in row slabs through a batched GEMM whose
    partial sums are added in fp32: against float64 on the bf16 operands, <= 4e-3 relative L2 (one bf16 rounding of the
    slab partial sums and one of the result), with the cotangent and the input sliced from one tensor (the operands
    must reach the library in two allocations)."""
    from fastfold_amd.model.fastnn.ops import Linear
    g = torch.Generator().manual_seed(rows)
    lin = Linear(k, n).to(dev, torch.bfloat16)
    both = torch.randn(rows, n + k, generator=g).to(dev, torch.bfloat16)
    cot, x = both[:, :n], both[:, n:].detach().requires_grad_()
    lin(x).backward(cot)
    want_w = cot.double().t() @ x.detach().double()
    assert _rel(lin.weight.grad, want_w) <= 4e-3, _rel(lin.weight.grad, want_w)
    assert _rel(lin.bias.grad, cot.double().sum(0)) <= 4e-3
    assert _rel(x.grad, cot.double() @ lin.weight.detach().double()) <= 4e-3


def test_block_chain_the_benchmark_way(dev):
    """benchmark/perf.py:141-155: stand-alone first / middle / last blocks in their default (training) mode, inputs
    that require gradients, ``layer_inputs[1].backward(grads)``.  Dropout is active: every triangle update drops
    whole rows (columns for the ending node) of channels with one mask, so only shapes, finiteness and the
    presence of every gradient are checked here."""
    from fastfold_amd.model.fastnn import Evoformer
    torch.manual_seed(0)
    s, r, cm, cz = 16, 40, 256, 128
    layers = [Evoformer(c_m=cm, c_z=cz, first_block=(i == 0), last_block=(i == 2)).to(dev, torch.bfloat16)
              for i in range(3)]
    node = torch.randn(s, r, cm, device=dev, dtype=torch.bfloat16).requires_grad_(True)
    pair = torch.randn(r, r, cz, device=dev, dtype=torch.bfloat16).requires_grad_(True)
    nmask = torch.ones(s, r, device=dev, dtype=torch.bfloat16)
    pmask = torch.ones(r, r, device=dev, dtype=torch.bfloat16)
    x = (node, pair)
    for i, lyr in enumerate(layers):
        x = lyr.forward(*x, nmask, pmask)
        if i < 2:
            assert x[0].shape == (1, s, r + 1, cm) and x[1].shape == (1, r + 1, r + 1, cz)
    assert x[0].shape == (s, r, cm) and x[1].shape == (r, r, cz)
    x[1].backward(torch.randn_like(pair))
    assert node.grad is not None and pair.grad is not None
    assert torch.isfinite(node.grad.float()).all() and torch.isfinite(pair.grad.float()).all()
    assert float(pair.grad.float().abs().max()) > 0


def test_dropout_masks_are_shared_along_rows_and_columns(dev):
    """bias_dropout_add / bias_ele_dropout_residual in training mode: one mask per (column, channel) for the row-wise
    updates, per (row, channel) for the ending node (fastnn/ops.py:405-412, :899-905); kept entries are scaled by
    1 / (1 - p)."""
    from fastfold_amd.model.fastnn.ops import ChunkTriangleAttentionEndingNode, ChunkTriangleAttentionStartingNode
    torch.manual_seed(1)
    r, cz = 32, 128
    z = torch.randn(1, r, r, cz, device=dev)
    mask = torch.ones(1, r, r, device=dev)
    for cls, dim in ((ChunkTriangleAttentionStartingNode, 1), (ChunkTriangleAttentionEndingNode, 2)):
        mod = cls(cz, p_drop=0.25, c=32, n_head=4).to(dev)
        with torch.no_grad():
            mod.attention.o_linear.weight.zero_()        # the update is then the bias alone
            mod.out_bias.fill_(1.0)
        upd = mod(z, mask) - z                           # parameters require gradients -> differentiable path
        assert upd.grad_fn is not None
        vals = torch.unique(upd.detach().round(decimals=4)).tolist()
        assert len(vals) == 2 and vals[0] == 0.0 and abs(vals[1] - 1 / 0.75) < 1e-4, vals
        keep = (upd.detach() != 0)
        assert torch.equal(keep, keep.narrow(dim, 0, 1).expand_as(keep))
        assert 0.5 < float(keep.float().mean()) < 0.95


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_elementwise_ops_backward(dev, dtype):
    from fastfold_amd.model.fastnn.kernel import bias_dropout_add, bias_ele_dropout_residual, bias_sigmod_ele
    g = torch.Generator().manual_seed(3)
    shape = (1, 5, 7, 64)
    tol = 1e-5 if dtype == torch.float32 else 2e-2

    def leaf(*sh):
        return torch.randn(*sh, generator=g).to(dev, dtype).requires_grad_()

    def f64(t):
        return t.detach().double().requires_grad_()
    cot = torch.randn(*shape, generator=g).to(dev)
    dm = (torch.rand(1, 1, 7, 64, generator=g) > 0.3).to(dev, dtype) / 0.7

    y, b, z = leaf(*shape), leaf(64), leaf(*shape)
    out = bias_sigmod_ele(y, b, z)
    (out.float() * cot).sum().backward()
    y2, b2, z2 = f64(y), f64(b), f64(z)
    (torch.sigmoid(y2 + b2) * z2 * cot.double()).sum().backward()
    for a, ref in ((y, y2), (b, b2), (z, z2)):
        assert _rel(a.grad, ref.grad) <= tol, _rel(a.grad, ref.grad)

    x, b, res = leaf(*shape), leaf(64), leaf(*shape)
    out = bias_dropout_add(x, b, dm, res, prob=0.3, training=False)
    (out.float() * cot).sum().backward()
    x2, b2, r2 = f64(x), f64(b), f64(res)
    ((r2 + (x2 + b2) * dm.double()) * cot.double()).sum().backward()
    for a, ref in ((x, x2), (b, b2), (res, r2)):
        assert _rel(a.grad, ref.grad) <= tol, _rel(a.grad, ref.grad)

    ab, b, gt, zr = leaf(*shape), leaf(64), leaf(*shape), leaf(*shape)
    out = bias_ele_dropout_residual(ab, b, gt, dm, zr, prob=0.3, training=False)
    (out.float() * cot).sum().backward()
    ab2, b2, g2, zr2 = f64(ab), f64(b), f64(gt), f64(zr)
    ((zr2 + dm.double() * (g2 * (ab2 + b2))) * cot.double()).sum().backward()
    for a, ref in ((ab, ab2), (b, b2), (gt, g2), (zr, zr2)):
        assert _rel(a.grad, ref.grad) <= tol, _rel(a.grad, ref.grad)


def test_block_forward_backward_at_headline_size(dev):
    """The differentiable block at the headline shape (N_seq = 128, N_res = 1024, last 5 % of the residues masked), bf16:
    outputs against the fused forward-only launches, every gradient finite, and the two input gradients against the
    same path run in fp32 (which the small-shape tests above pin to the float64 oracle) at the bf16 bound.  The
    triangle contraction and its two backward products run on ffk_bgemm_nt at this size (128 x 1024^3), the weight
    gradients of the million-row activations through the guarded slab GEMM."""
    import sys
    print("test_block_forward_backward_at_headline_size: s=128 r=1024 bf16 + fp32", flush=True)
    sys.stdout.flush()
    s, r, tail = 128, 1024, 0.05
    model = _oracle(33, 1)
    m, z, mm, pm = synth_inputs(33, s, r, mask_tail_frac=tail)
    nv = r - int(round(tail * r))
    g = torch.Generator().manual_seed(7)
    cot_z = torch.randn(r, r, KW["c_z"], generator=g)
    cot_z[nv:] = 0
    cot_z[:, nv:] = 0
    grads, outs = {}, {}
    for dtype in (torch.bfloat16, torch.float32):
        fast = _fast(model, dev, dtype).eval()
        mi, zi = (torch.from_numpy(t).to(dev, dtype).requires_grad_() for t in (m, z))
        mk, pk = torch.from_numpy(mm).to(dev, dtype), torch.from_numpy(pm).to(dev, dtype)
        out = fast(mi, zi, mk, pk, chunk_size=None)
        assert out[1].grad_fn is not None
        if dtype == torch.bfloat16:
            with torch.no_grad():
                fused = fast(mi, zi, mk, pk, chunk_size=None)
            assert _rel(out[0][:, :nv], fused[0][:, :nv]) <= 2e-2
            assert _rel(out[1][:nv, :nv], fused[1][:nv, :nv]) <= 2e-2
            del fused
        (out[1].float() * cot_z.to(dev)).sum().backward()
        torch.cuda.synchronize()
        for name, p in fast.named_parameters():
            if name.startswith("linear."):        # the single-representation projection: not on the path to z
                continue
            assert p.grad is not None and bool(torch.isfinite(p.grad.float()).all()), name
        assert bool(torch.isfinite(mi.grad.float()).all()) and bool(torch.isfinite(zi.grad.float()).all())
        grads[dtype] = (mi.grad.float().cpu(), zi.grad.float().cpu())
        outs[dtype] = out[1].detach().float().cpu()
        del fast, out, mi, zi
        torch.cuda.empty_cache()
    assert _rel(outs[torch.bfloat16][:nv, :nv], outs[torch.float32][:nv, :nv]) <= 2e-2
    assert _rel(grads[torch.bfloat16][0], grads[torch.float32][0]) <= 5e-2, _rel(grads[torch.bfloat16][0], grads[torch.float32][0])
    assert _rel(grads[torch.bfloat16][1], grads[torch.float32][1]) <= 5e-2, _rel(grads[torch.bfloat16][1], grads[torch.float32][1])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 2e-2)])
def test_block_recompute_same_dropout_in_both_passes(dev, dtype, tol):
    """A training-mode block under autograd runs the fused launches forward and re-runs itself operator by operator
    in the backward pass (``_BlockRecompute``): with dropout active both passes must apply the SAME multipliers.  The
    multipliers of one call are captured, and the fused forward is compared with the operator-by-operator block run
    on them; the gradients of the call are those of that run."""
    from fastfold_amd.model.fastnn import Evoformer
    torch.manual_seed(4)
    s, r = 12, 40
    blk = Evoformer(c_m=256, c_z=128, first_block=True, last_block=True).to(dev, dtype).train()
    with torch.no_grad():
        for n, p in blk.named_parameters():        # the zero-initialised output layers would hide every update
            if p.dim() >= 2:
                p.copy_(torch.randn_like(p) * p.shape[-1] ** -0.5)
    m = torch.randn(s, r, 256, device=dev).to(dtype).requires_grad_()
    z = torch.randn(r, r, 128, device=dev).to(dtype).requires_grad_()
    mm = torch.ones(s, r, device=dev, dtype=dtype)
    pm = torch.ones(r, r, device=dev, dtype=dtype)
    seen = {}
    draw = blk._draw_drops

    def capture(a, b):
        seen["d"] = draw(a, b)
        return seen["d"]
    blk._draw_drops = capture
    mo, zo = blk(m, z, mm, pm)
    d = seen["d"]
    assert set(d) == {"row", "tmo", "tmi", "tas", "tae"}
    for k, v in d.items():
        assert v.shape == ((1, r, 1, 128) if k == "tae" else (1, 1, r, 256 if k == "row" else 128))
        assert 0.4 < float((v != 0).float().mean()) < 0.99 and float(v.max()) > 1.0
    cot = torch.randn_like(zo)
    (zo.float() * cot.float()).sum().backward()
    got = (m.grad.clone(), z.grad.clone())
    pg = {n: p.grad.clone() for n, p in blk.named_parameters() if p.grad is not None}
    blk.zero_grad()
    m2, z2 = m.detach().clone().requires_grad_(), z.detach().clone().requires_grad_()
    mo2, zo2 = blk._core_train(m2.unsqueeze(0), z2.unsqueeze(0), mm.unsqueeze(0), pm.unsqueeze(0), drops=d)
    assert _rel(mo, mo2.squeeze(0)) <= tol and _rel(zo, zo2.squeeze(0)) <= tol, (_rel(mo, mo2.squeeze(0)), _rel(zo, zo2.squeeze(0)))
    (zo2.squeeze(0).float() * cot.float()).sum().backward()
    gtol = 1e-4 if dtype == torch.float32 else 5e-2      # atomics in the parameter gradients; bf16: one rounding step
    assert _rel(got[0], m2.grad) <= gtol and _rel(got[1], z2.grad) <= gtol
    assert len(pg) >= 70
    for n, p in blk.named_parameters():
        if n in pg and float(p.grad.float().norm()) > 1e-3:
            assert _rel(pg[n], p.grad) <= gtol, n
    # dropped updates really are dropped: with every multiplier zero the pair stack's dropped updates vanish
    zero = {k: torch.zeros_like(v) for k, v in d.items()}
    blk._draw_drops = lambda a, b: zero
    with torch.enable_grad():
        mo3, zo3 = blk(m.detach().requires_grad_(), z.detach().requires_grad_(), mm, pm)
    mo4, zo4 = blk._core_train(m.detach().unsqueeze(0), z.detach().unsqueeze(0), mm.unsqueeze(0), pm.unsqueeze(0), drops=zero)
    assert _rel(zo3, zo4.squeeze(0)) <= tol and _rel(mo3, mo4.squeeze(0)) <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,X,Y", [(3, 64, 64), (2, 70, 33), (5, 1, 9), (1, 129, 200), (4, 40, 128), (2, 8, 8)])
def test_transpose_batched_kernel(dev, dtype, B, X, Y):
    """out[b][y][x] = in[b][x][y] with strides: contiguous operands, views with larger pitches (padding that must stay
    untouched), a batch stride smaller than a row stride (the batch index is the inner one), and pointers off the
    16-byte grid (element-wise branches)."""
    from fastfold_amd import _lib
    g = torch.Generator().manual_seed(B * 100 + X + Y)
    x = torch.randn(B, X, Y, generator=g).to(dev, dtype)
    out = torch.empty(B, Y, X, dtype=dtype, device=dev)
    _lib.transpose_batched(out, x, B=B, X=X, Y=Y, in_bs=X * Y, in_xs=Y, out_bs=X * Y, out_ys=X)
    assert torch.equal(out, x.transpose(1, 2))
    # padded pitches on both sides, element offsets into the buffers
    xp = torch.randn(B, X + 2, Y + 5, generator=g).to(dev, dtype)
    op = torch.full((B, Y + 1, X + 3), 7.0, dtype=dtype, device=dev)
    _lib.transpose_batched(op, xp, B=B, X=X, Y=Y, in_bs=xp.stride(0), in_xs=xp.stride(1), out_bs=op.stride(0),
                           out_ys=op.stride(1), in_off=xp.stride(1) + 3, out_off=op.stride(1) + 2)
    assert torch.equal(op[:, 1:, 2:2 + X], xp[:, 1:1 + X, 3:3 + Y].transpose(1, 2))
    keep = op.clone()
    keep[:, 1:, 2:2 + X] = 7.0
    assert float((keep - 7.0).abs().max()) == 0.0                       # nothing outside the addressed elements
    # the batch index as the inner one: in[x][b][y] -> out[y][b][x]
    xi = torch.randn(X, B, Y, generator=g).to(dev, dtype)
    oi = torch.empty(Y, B, X, dtype=dtype, device=dev)
    _lib.transpose_batched(oi, xi, B=B, X=X, Y=Y, in_bs=Y, in_xs=B * Y, out_bs=X, out_ys=B * X)
    assert torch.equal(oi, xi.permute(2, 1, 0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r,c", [(40, 128), (33, 64), (64, 128)])
@pytest.mark.parametrize("incoming", [False, True])
def test_channel_major_functions_match_the_permutes(dev, dtype, r, c, incoming):
    """_ToChanMajorFn / _FromChanMajorFn / _transpose_cm against the permute + copy they replace, forward and backward."""
    from fastfold_amd.model.fastnn import ops
    g = torch.Generator().manual_seed(r + c)
    lr = torch.randn(1, r, r, 2 * c, generator=g).to(dev, dtype).requires_grad_()
    L, R = ops._ToChanMajorFn.apply(lr, incoming)
    perm = (2, 1, 0) if incoming else (2, 0, 1)
    left, right = lr.chunk(2, dim=-1)
    Lw, Rw = ops._chan_major(left, perm), ops._chan_major(right, perm)
    assert torch.equal(L, Lw) and torch.equal(R, Rw)
    assert L.untyped_storage().data_ptr() != R.untyped_storage().data_ptr()
    cl, cr = torch.randn(L.shape, generator=g).to(dev, dtype), torch.randn(R.shape, generator=g).to(dev, dtype)
    (gl,) = torch.autograd.grad([L, R], [lr], [cl, cr])
    (gw,) = torch.autograd.grad([Lw, Rw], [lr], [cl, cr])
    assert torch.equal(gl, gw)
    assert torch.equal(ops._transpose_cm(L.detach(), r)[..., :r], L.detach()[..., :r].transpose(1, 2))
    p = L.detach().clone().requires_grad_()
    z = ops._FromChanMajorFn.apply(p, r)
    zw = ops.permute_final_dims(p[None, :, :, :r], (1, 2, 0))
    assert z.is_contiguous() and torch.equal(z, zw)
    cz = torch.randn(z.shape, generator=g).to(dev, dtype)
    (gp,) = torch.autograd.grad(z, p, cz)
    (gpw,) = torch.autograd.grad(zw, p, cz)
    assert torch.equal(gp, gpw)
