"""Acceptance runs at the benchmark's own configurations (bf16 HIP path against the fp32 oracle / the reference's
vectors; tolerance of the bf16 mode: relative L2 <= 2e-2 on the MSA, pair and single outputs):

* the 48-block stack at N_seq = 128, N_res = 256 against the fp32 CPU oracle called with ``_mask_trans=False``, on
  the outputs and on the accumulated update (out - in), so that a vanishing update cannot hide in the residual;
* the 48-block stack and one block at N_seq = 128, N_res = 1024 (last 5 % of the residues masked) against a sample of the outputs of the
  reference's own ``fastfold.model.nn.evoformer.EvoformerStack`` (``tests/golden/make_golden.py cfg4``);
* one block at N_seq = 64, N_res = 4096 with ``set_chunk_size(64)`` through ``.inplace``: properties the size does
  not change, and the peak memory;
* the exact operator shapes of the micro-benchmark (fused softmax on [1, 128, 8, 256, 256], LayerNorm over
  65 536 x 128 and 32 768 x 256 rows) against float64 numpy;
* every loop that processes rows in budget-sized pieces, forced to several pieces with a ragged tail.
"""
import copy
import os

import numpy as np
import pytest
import torch

from fastfold_amd.synthetic import bf16_round, synth_extra_nn_state, synth_inputs, synth_nn_state
from oracle import ops_np
from oracle.evoformer_ref import OracleModel

pytestmark = pytest.mark.gpu

KW = dict(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128, c_hidden_pair_att=32, c_s=384,
          no_heads_msa=8, no_heads_pair=4, transition_n=4, msa_dropout=0.15, pair_dropout=0.25, blocks_per_ckpt=1,
          inf=1e9, eps=1e-8)
CFG4_GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "evoformer_cfg4_nn_golden.npz")


def _models(seed, nb, dev, dtype=torch.bfloat16, fan_in_scaled=False, extra=False):
    from fastfold_amd.utils.inject_fastnn import inject_fastnn
    model = OracleModel(no_blocks=nb, extra_msa_kwargs=dict(no_blocks=nb) if extra else None, **KW).eval()
    sd = synth_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fan_in_scaled)
    model.evoformer.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    if extra:
        sd = synth_extra_nn_state(seed=seed, no_blocks=nb, fan_in_scaled=fan_in_scaled)
        model.extra_msa_stack.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    fast = inject_fastnn(copy.deepcopy(model))
    return model, fast.to(dev, dtype).eval()


def _t(x, dev, dtype=torch.bfloat16):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev, dtype)


def _f(t):
    return t.detach().float().cpu().numpy()


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


# ------------------------------------------------------------------ 48 blocks, N_res = 256 ----
@pytest.mark.parametrize("nb,fan_in_scaled", [(48, False), (8, True)])
def test_deep_stack_bf16_against_fp32_oracle(dev, nb, fan_in_scaled):
    """48 blocks with the benchmark's N(0, 0.02^2) weights; and 8 blocks with fan-in scaled weights, whose every
    sub-update is O(1) (deeper, the fan-in scaled stack leaves the range in which fp32 and bf16 runs of a chaotic
    map can be compared at all)."""
    s, r = 128, 256
    model, fast = _models(81, nb, dev, fan_in_scaled=fan_in_scaled)
    m, z, mm, pm = synth_inputs(81, s, r)
    m, z = bf16_round(m), bf16_round(z)
    torch.set_num_threads(max(1, min(16, os.cpu_count() or 1)))
    with torch.no_grad():
        rm, rz, rs = model.evoformer(torch.from_numpy(m), torch.from_numpy(z), torch.from_numpy(mm),
                                     torch.from_numpy(pm), _mask_trans=False)
        gm, gz, gs = fast.evoformer(_t(m, dev), _t(z, dev), _t(mm, dev), _t(pm, dev), chunk_size=None)
    rm, rz, rs, gm, gz, gs = rm.numpy(), rz.numpy(), rs.numpy(), _f(gm), _f(gz), _f(gs)
    assert np.isfinite(gm).all() and np.isfinite(gz).all() and np.isfinite(gs).all()
    em, ez, es = _rel_l2(gm, rm), _rel_l2(gz, rz), _rel_l2(gs, rs)
    um, uz = _rel_l2(gm - m, rm - m), _rel_l2(gz - z, rz - z)
    size_m, size_z = float(np.linalg.norm(rm - m) / np.linalg.norm(m)), float(np.linalg.norm(rz - z) / np.linalg.norm(z))
    print("\n%d blocks (fan-in scaled: %s): rel-L2 m %.3e z %.3e s %.3e | accumulated update: m %.3e z %.3e "
          "(|update| / |input|: m %.2f z %.2f)" % (nb, fan_in_scaled, em, ez, es, um, uz, size_m, size_z))
    assert em <= 2e-2 and ez <= 2e-2 and es <= 2e-2
    # the accumulated update is a large part of the output, and it must be right on its own
    if fan_in_scaled:
        assert size_m > 0.5 and size_z > 0.5
    assert um <= 4e-2 and uz <= 4e-2


# ------------------------------------------------------------------ 48 blocks, N_res = 1024 ----
CFG4_DEEP_GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "evoformer_cfg4_deep48_nn_golden.npz")


def test_cfg4_deep_stack_against_reference_sample(dev):
    """The headline acceptance: the 48-block bf16 stack at N_seq = 128, N_res = 1024 (last 5 % of the residues masked,
    N(0, 0.02^2) weights) against the stored sample of the fp32 outputs of the reference's own ``nn.EvoformerStack``
    (``tests/golden/make_golden.py cfg4_deep 48``): relative L2 <= 2e-2 on the MSA, pair and single outputs, and on the
    accumulated update (out - in), whose size relative to the input is checked against the reference's too."""
    g = np.load(CFG4_DEEP_GOLDEN)
    case = "cfg4_deep48"
    seed, nb, s, r, tail, fis = (int(v) for v in g[case + ".cfg"])
    S, I, J = g[case + ".S"], g[case + ".I"], g[case + ".J"]
    nv = r - int(round(tail / 100.0 * r))
    _, fast = _models(seed, nb, dev, fan_in_scaled=bool(fis))
    m, z, mm, pm = synth_inputs(seed, s, r, mask_tail_frac=tail / 100.0)
    m, z = bf16_round(m), bf16_round(z)
    with torch.no_grad():
        gm, gz, gs = fast.evoformer(_t(m, dev), _t(z, dev), _t(mm, dev), _t(pm, dev), chunk_size=None)
    gm, gz, gs = _f(gm), _f(gz), _f(gs)
    assert np.isfinite(gm).all() and np.isfinite(gz).all() and np.isfinite(gs).all()
    # size of the accumulated update over the whole un-masked region, against the reference's
    rn = g[case + ".norms"]
    um, uz = float(np.linalg.norm((gm - m)[:, :nv])), float(np.linalg.norm((gz - z)[:nv, :nv]))
    assert abs(um / rn[3] - 1) < 2e-2 and abs(uz / rn[4] - 1) < 2e-2
    m0, z0 = m[S][:, J], z[I][:, J]
    gm, gz, gs = gm[S][:, J], gz[I][:, J], gs[J]
    rm, rz, rs = g[case + ".m"], g[case + ".z"], g[case + ".s"]
    em, ez, es = _rel_l2(gm, rm), _rel_l2(gz, rz), _rel_l2(gs, rs)
    dm, dz = _rel_l2(gm - m0, rm - m0), _rel_l2(gz - z0, rz - z0)
    print("\n%s: rel-L2 m %.3e z %.3e s %.3e | accumulated update: m %.3e z %.3e (|update| / |input|: m %.2f z %.2f)"
          % (case, em, ez, es, dm, dz, rn[3] / np.linalg.norm(m[:, :nv]), rn[4] / np.linalg.norm(z[:nv, :nv])))
    assert em <= 2e-2 and ez <= 2e-2 and es <= 2e-2
    assert dm <= 4e-2 and dz <= 4e-2


# ------------------------------------------------------------------ one block, N_res = 1024 ----
@pytest.mark.parametrize("case", ["cfg4_fanin", "cfg4_std002"])
def test_cfg4_block_against_reference_sample(dev, case):
    """Values at the headline shape: the HIP bf16 block against the stored sample of the reference's fp32 outputs
    (random un-masked sequences / residues), on the outputs and on the update alone."""
    g = np.load(CFG4_GOLDEN)
    seed, nb, s, r, tail, fis = (int(v) for v in g[case + ".cfg"])
    S, I, J = g[case + ".S"], g[case + ".I"], g[case + ".J"]
    _, fast = _models(seed, nb, dev, fan_in_scaled=bool(fis))
    m, z, mm, pm = synth_inputs(seed, s, r, mask_tail_frac=tail / 100.0)
    m, z = bf16_round(m), bf16_round(z)
    with torch.no_grad():
        gm, gz, gs = fast.evoformer(_t(m, dev), _t(z, dev), _t(mm, dev), _t(pm, dev), chunk_size=None)
    gm, gz, gs = _f(gm)[S][:, J], _f(gz)[I][:, J], _f(gs)[J]
    rm, rz, rs = g[case + ".m"], g[case + ".z"], g[case + ".s"]
    m0, z0 = m[S][:, J], z[I][:, J]
    em, ez, es = _rel_l2(gm, rm), _rel_l2(gz, rz), _rel_l2(gs, rs)
    um, uz = _rel_l2(gm - m0, rm - m0), _rel_l2(gz - z0, rz - z0)
    print("\n%s: rel-L2 m %.3e z %.3e s %.3e | update: m %.3e z %.3e" % (case, em, ez, es, um, uz))
    assert em <= 2e-2 and ez <= 2e-2 and es <= 2e-2
    # the update alone: inputs are O(1) bf16 values, so a bf16 result carries a rounding error of about
    # 2^-9 |out| per element whatever the size of the update; relative to a small update (N(0, 0.02^2) weights)
    # that is a larger fraction than relative to an O(1) one
    assert um <= (2e-2 if fis else 1e-1) and uz <= (2e-2 if fis else 1e-1)


# ------------------------------------------------------------------ long sequence, chunked, in place ----
def test_long_sequence_block_chunked_inplace(dev):
    """N_seq = 64, N_res = 4096, ``set_chunk_size(64)``, ``.inplace``: finite; bit-identical to ``forward`` on a
    second copy; un-masked outputs bit-identical when masked inputs change; peak memory a small multiple of the
    pair tensor (4.3 GB)."""
    from fastfold_amd.model.fastnn import set_chunk_size
    s, r, tail = 64, 4096, 0.05
    nv = r - int(round(tail * r))
    _, fast = _models(83, 1, dev, fan_in_scaled=True)
    stack = fast.evoformer
    g = torch.Generator(device=dev).manual_seed(83)
    m = torch.randn(s, r, 256, generator=g, device=dev, dtype=torch.bfloat16)
    z = torch.randn(r, r, 128, generator=g, device=dev, dtype=torch.bfloat16)
    seq_mask = torch.ones(r, device=dev, dtype=torch.bfloat16)
    seq_mask[nv:] = 0
    mm = seq_mask[None, :].expand(s, r).contiguous()
    pm = (seq_mask[:, None] * seq_mask[None, :]).contiguous()
    z_bytes = z.numel() * 2
    set_chunk_size(64)
    try:
        with torch.no_grad():
            fm, fz, fs = stack(m, z, mm, pm, chunk_size=64)               # forward: inputs untouched
            torch.cuda.synchronize()
            m1, z1 = [m.clone()], [z.clone()]
            torch.cuda.reset_peak_memory_stats()
            base = torch.cuda.memory_allocated()
            stack.inplace(m1, z1, mm, pm, chunk_size=64)
            torch.cuda.synchronize()
            peak = torch.cuda.max_memory_allocated() - base
            print("\nlong sequence: peak extra memory of the in-place block %.2f GB (pair tensor %.2f GB)"
                  % (peak / 1e9, z_bytes / 1e9))
            assert bool(torch.isfinite(z1[0].float()).all()) and bool(torch.isfinite(m1[0].float()).all())
            assert torch.equal(m1[0], fm) and torch.equal(z1[0], fz)
            # scratch of the chunked path: the triangle-multiplication operands (2 |z|) and contraction result (|z|)
            # are the largest, then the int8 tail of the pair stream (|z| / 2); the rest is bounded by the chunk budget
            assert peak <= 4.0 * z_bytes
            del m1, z1
            # masked residues never reach un-masked outputs
            m2, z2 = m.clone(), z.clone()
            m2[:, nv:] += 3.0
            z2[nv:, :] -= 2.0
            z2[:, nv:] += 1.5
            m2, z2 = [m2], [z2]
            stack.inplace(m2, z2, mm, pm, chunk_size=64)
            assert torch.equal(m2[0][:, :nv], fm[:, :nv]) and torch.equal(z2[0][:nv, :nv], fz[:nv, :nv])
    finally:
        set_chunk_size(None)
    # the update is not vanishing
    assert float((fz.float() - z.float()).norm() / z.float().norm()) > 0.1


# ------------------------------------------------------------------ micro-benchmark shapes ----
def test_softmax_microbench_shape_against_float64(dev):
    """fused_softmax on logits [1, 128, 8, 256, 256] bf16, pair bias [1, 1, 8, 256, 256], key mask with 10 % zeros
    (the grid-stride path of the row kernel: 262 144 rows)."""
    from fastfold_amd.model.fastnn.kernel import fused_softmax
    rng = np.random.RandomState(2)
    B2, H, N = 128, 8, 256
    x = bf16_round(rng.standard_normal((1, B2, H, N, N)).astype(np.float32))
    bias = bf16_round(rng.standard_normal((1, 1, H, N, N)).astype(np.float32))
    mask = (rng.rand(1, B2, N) > 0.1).astype(np.float32)
    mask[..., 0] = 1.0
    out = _f(fused_softmax(_t(x, dev), _t(mask, dev), _t(bias, dev)))
    worst = 0.0
    for b0 in range(0, B2, 16):        # float64 in slabs of 16 batch rows (134 MB each)
        ref = ops_np.fused_softmax(x[:, b0:b0 + 16].astype(np.float64), mask[:, b0:b0 + 16].astype(np.float64),
                                   bias.astype(np.float64))
        got = out[:, b0:b0 + 16]
        assert np.all(got[np.broadcast_to(mask[:, b0:b0 + 16, None, None, :] == 0, got.shape)] == 0.0)
        worst = max(worst, float(np.abs(got - ref).max()))
        assert np.abs(got.sum(-1) - 1.0).max() <= 2e-2
    assert worst <= 4e-3        # half an ulp of bf16 at 1.0 (2^-9) on top of fp32 arithmetic
    print("\nsoftmax [1,128,8,256,256] bf16: max-abs error vs float64 %.2e" % worst)


@pytest.mark.parametrize("rows,cols", [(65536, 128), (32768, 256)])
def test_layernorm_microbench_shape_against_float64(dev, rows, cols):
    from fastfold_amd.model.fastnn.kernel import LayerNorm
    rng = np.random.RandomState(rows + cols)
    x = bf16_round((rng.standard_normal((rows, cols)) * 1.3 + 0.2).astype(np.float32))
    gam = bf16_round((1 + 0.1 * rng.standard_normal(cols)).astype(np.float32))
    bet = bf16_round((0.1 * rng.standard_normal(cols)).astype(np.float32))
    ln = LayerNorm(cols).to(dev, torch.bfloat16)
    with torch.no_grad():
        ln.weight.copy_(_t(gam, dev))
        ln.bias.copy_(_t(bet, dev))
        out = _f(ln(_t(x, dev)))
    ref = ops_np.layer_norm(x.astype(np.float64), gam.astype(np.float64), bet.astype(np.float64))
    err = np.abs(out - ref)
    assert float(err.max()) <= 2 ** -8 * max(1.0, float(np.abs(ref).max()))      # one bf16 ulp at the largest output
    assert _rel_l2(out, ref) <= 4e-3


# ------------------------------------------------------------------ budget loops ----
@pytest.fixture
def tiny_budget(monkeypatch):
    """Chunked mode with a scratch budget of 800 KB: every loop over budget-sized pieces runs several times (at the
    sizes below: triangle attention in slabs of 6 of 88 rows, the MSA transition in 384-row pieces of 3 520, the
    outer product 4 of 88 rows at a time)."""
    from fastfold_amd.model.fastnn import _fused, set_chunk_size
    monkeypatch.setattr(_fused, "_WS_BUDGET_CHUNKED", 800 << 10)
    set_chunk_size(4)
    yield
    set_chunk_size(None)


def _run_both(fn):
    """fn() un-chunked, then chunked; returns the two results."""
    from fastfold_amd.model.fastnn import get_chunk_size, set_chunk_size
    cs = get_chunk_size()
    set_chunk_size(None)
    with torch.no_grad():
        whole = fn()
    set_chunk_size(cs)
    with torch.no_grad():
        pieces = fn()
    return whole, pieces


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_chunked_block_equals_unchunked(dev, dtype, tiny_budget):
    """A whole block (forward and in place) with every sub-module cut into pieces: attention batch-row slabs with a
    ragged last slab (row, column, both triangle attentions), MSA transition rows, outer-product rows (s = 40 is
    outside the fused kernel's 57 .. 64 / 121 .. 128), against the un-chunked run bit for bit and against the oracle."""
    s, r, tail = 40, 88, 0.1
    nv = r - int(round(tail * r))
    model, fast = _models(85, 1, dev, dtype=dtype, fan_in_scaled=True)
    m, z, mm, pm = synth_inputs(85, s, r, mask_tail_frac=tail)
    m, z = bf16_round(m), bf16_round(z)
    args = [_t(a, dev, dtype) for a in (m, z, mm, pm)]
    whole, pieces = _run_both(lambda: fast.evoformer(*args, chunk_size=None))
    for name, a, b in zip("mzs", whole, pieces):
        assert torch.equal(a, b), "%s: chunked run differs by up to %g" % (name, float((a.float() - b.float()).abs().max()))
    def inplace():
        mi, zi = [args[0].clone()], [args[1].clone()]
        _, _, si = fast.evoformer.inplace(mi, zi, args[2], args[3], chunk_size=None)
        return mi[0], zi[0], si
    for a, b in zip(whole, _run_both(inplace)[1]):
        assert torch.equal(a, b)
    with torch.no_grad():
        rm, rz, rs = model.evoformer(*(torch.from_numpy(a) for a in (m, z, mm, pm)), _mask_trans=False)
    gm, gz = _f(pieces[0]), _f(pieces[1])
    if dtype == torch.float32:
        scale = max(1.0, float(rz.abs().max()))
        assert np.abs(gm - rm.numpy())[:, :nv].max() <= 1e-4 * scale and np.abs(gz - rz.numpy())[:nv, :nv].max() <= 1e-4 * scale
    else:
        assert _rel_l2(gm[:, :nv], rm.numpy()[:, :nv]) <= 2e-2 and _rel_l2(gz[:nv, :nv], rz.numpy()[:nv, :nv]) <= 2e-2


def test_attention_slabs_really_iterate(dev, tiny_budget, monkeypatch):
    """The tiny budget cuts a triangle attention over 88 rows into several launches of the core (guards the test above
    against a budget that silently stopped applying)."""
    from fastfold_amd import _lib
    _, fast = _models(86, 1, dev, fan_in_scaled=True)
    m, z, mm, pm = synth_inputs(86, 40, 88)
    calls = []
    real = _lib.attention_fwd
    monkeypatch.setattr(_lib, "attention_fwd", lambda *a, **k: (calls.append(k["B2"]), real(*a, **k))[1])
    with torch.no_grad():
        fast.evoformer.blocks[0].pair.TriangleAttentionStartingNode(_t(z, dev)[None], _t(pm, dev)[None])
    assert len(calls) >= 3 and sum(calls) == 88 and calls[-1] != calls[0], calls


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_chunked_extra_msa_block_equals_unchunked(dev, dtype, tiny_budget, monkeypatch):
    """Extra-MSA block: the gate / output projection of the global column attention (20 or 10 of 72 sequences at a
    time under a 100 KB budget) and the 64-channel transition in pieces, forward and in place."""
    from fastfold_amd.model.fastnn import _fused
    monkeypatch.setattr(_fused, "_WS_BUDGET_CHUNKED", 100 << 10)
    se, r = 72, 40
    _, fast = _models(87, 1, dev, dtype=dtype, fan_in_scaled=True, extra=True)
    m, z, mm, pm = synth_inputs(87, se, r, c_m=64, mask_tail_frac=0.1)
    tm, tz, tmm, tpm = (_t(a, dev, dtype) for a in (m, z, mm, pm))
    stack = fast.extra_msa_stack
    whole, pieces = _run_both(lambda: stack(tm, tz, chunk_size=None, msa_mask=tmm, pair_mask=tpm))
    assert torch.equal(whole, pieces)
    col = stack.blocks[0].msa_stack.MSAColumnAttention
    def inplace():
        mi = [tm[None].clone()]
        col.inplace(mi, tmm[None])
        return mi[0]
    a, b = _run_both(inplace)
    with torch.no_grad():                      # (with gradients enabled the module would take its differentiable path)
        fwd = col(tm[None], tmm[None])
    assert torch.equal(a, b) and torch.equal(a, fwd)
