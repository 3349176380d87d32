"""GPU parity of the input and recycling embedders (pair-embedding kernel + projection kernels) against the
CPU oracle (oracle.evoformer_ref.InputEmbedder / RecyclingEmbedder, pinned by float64 brute force).

Tolerances: fp32 max-abs <= 1e-4; bf16 relative L2 <= 2e-2 against the fp32 oracle."""
import copy

import numpy as np
import pytest
import torch

from oracle.evoformer_ref import (EvoformerStack as OracleEvoformer, InputEmbedder as OracleInput,
                                  RecyclingEmbedder as OracleRecycling)

pytestmark = pytest.mark.gpu


class _Model(torch.nn.Module):
    def __init__(self, c_z=128, c_m=256):
        super().__init__()
        self.evoformer = OracleEvoformer(no_blocks=1)
        self.input_embedder = OracleInput(tf_dim=22, msa_dim=49, c_z=c_z, c_m=c_m, relpos_k=32)
        self.recycling_embedder = OracleRecycling(c_m=c_m, c_z=c_z, min_bin=3.25, max_bin=20.75, no_bins=15, inf=1e8)


def _models(dev, dtype, seed=0):
    from fastfold_amd.utils.inject_fastnn import inject_embedder
    torch.manual_seed(seed)
    ref = _Model().eval()
    with torch.no_grad():
        for mod in (ref.input_embedder, ref.recycling_embedder):
            for n, p in mod.named_parameters():
                p.copy_((1.0 if "layer_norm" in n and n.endswith("weight") else 0.0) + 0.3 * torch.randn_like(p))
    fast = copy.deepcopy(ref)
    inject_embedder(fast)
    return ref, fast.to(dev, dtype).eval()


def _f(t):
    return t.detach().float().cpu().numpy()


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def _check(got, ref, dtype):
    if dtype == torch.float32:
        assert np.abs(got - ref).max() <= 1e-4, np.abs(got - ref).max()
    else:
        assert _rel_l2(got, ref) <= 2e-2, _rel_l2(got, ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("s,r", [(1, 1), (5, 37), (16, 64), (2, 129)])
def test_input_embedder(dev, dtype, s, r):
    from fastfold_amd.model.fastnn.embedders import InputEmbedder
    ref, fast = _models(dev, dtype)
    assert isinstance(fast.input_embedder, InputEmbedder)
    rng = np.random.RandomState(r)
    tf = torch.from_numpy(rng.standard_normal((r, 22)).astype(np.float32))
    msa = torch.from_numpy(rng.standard_normal((s, r, 49)).astype(np.float32))
    ri = torch.arange(r) + torch.from_numpy((np.arange(r) >= r // 2) * 200)      # a chain break beyond the window
    if dtype == torch.bfloat16:
        tf, msa = tf.to(dtype).float(), msa.to(dtype).float()
    with torch.no_grad():
        rm, rz = ref.input_embedder(tf, ri, msa)
        gm, gz = fast.input_embedder(tf.to(dev, dtype), ri.to(dev), msa.to(dev, dtype))
    assert gm.shape == (s, r, 256) and gz.shape == (r, r, 128) and gm.dtype == dtype
    _check(_f(gm), rm.numpy(), dtype)
    _check(_f(gz), rz.numpy(), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r", [5, 23, 64])
def test_recycling_embedder(dev, dtype, r):
    from fastfold_amd.model.fastnn import set_chunk_size
    ref, fast = _models(dev, dtype, seed=1)
    rng = np.random.RandomState(r)
    m = torch.from_numpy(rng.standard_normal((r, 256)).astype(np.float32))
    z = torch.from_numpy(rng.standard_normal((r, r, 128)).astype(np.float32))
    x = torch.from_numpy((rng.standard_normal((r, 3)) * 9.0).astype(np.float32))
    x[1] = x[0] + torch.tensor([3.25, 0.0, 0.0])          # on the first bin edge (up to fp32 rounding of the sum)
    x[3] = x[2]                                           # zero distance: below the first bin
    if dtype == torch.bfloat16:
        m, z = m.to(dtype).float(), z.to(dtype).float()
    with torch.no_grad():
        rm, rz = ref.recycling_embedder(m, z, x)
        tz = z.to(dev, dtype)
        keep = tz.clone()
        gm, gz = fast.recycling_embedder(m.to(dev, dtype), tz, x.to(dev))
    assert torch.equal(tz, keep), "z must be left untouched when no chunk size is set"
    _check(_f(gm), rm.numpy(), dtype)
    # bins are decided in fp32 from the same fp32 coordinates on both sides; a pair within rounding of an
    # edge may still fall on different sides, so allow a handful of pairs to differ by one table row
    diff = np.abs(_f(gz) - rz.numpy()).max(-1)
    tol = 1e-4 if dtype == torch.float32 else 0.25
    assert (diff > tol).sum() <= 4, (diff > tol).sum()
    _check(_f(gz)[diff <= tol], rz.numpy()[diff <= tol], dtype)
    # with a chunk size the update is written into z, as in the reference
    set_chunk_size(4)
    try:
        with torch.no_grad():
            _, gz2 = fast.recycling_embedder(m.to(dev, dtype), tz, x.to(dev))
    finally:
        set_chunk_size(None)
    assert gz2.data_ptr() == tz.data_ptr() and torch.equal(gz2, gz)


def test_pair_embed_rejects_bad_arguments(dev):
    from fastfold_amd import _lib
    out = torch.zeros(4, 4, 128, device=dev)
    table = torch.zeros(4, 128, device=dev)
    pos = torch.zeros(4, device=dev)
    with pytest.raises(RuntimeError, match="odd number"):
        _lib.pair_embed(out, None, None, None, table, None, None, None, mode=_lib.FFK_EMBED_RELPOS, pos=pos, r=4, C=128, nb=4)
    with pytest.raises(RuntimeError, match="bin edges"):
        _lib.pair_embed(out, None, None, None, table, None, None, None, mode=_lib.FFK_EMBED_DISTOGRAM, pos=pos, r=4, C=128, nb=3)
    with pytest.raises(RuntimeError, match="C must be"):
        _lib.pair_embed(torch.zeros(4, 4, 96, device=dev), None, None, None, torch.zeros(3, 96, device=dev), None, None, None,
                        mode=_lib.FFK_EMBED_RELPOS, pos=pos, r=4, C=96, nb=3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_only_embedders(dev, dtype):
    """Template angle / pair and extra-MSA embedders (ragged input widths 57 / 88 / 25) against F.linear."""
    import torch.nn.functional as F
    from fastfold_amd.model.fastnn.ops import ExtraMSAEmbedder, TemplateAngleEmbedder, TemplatePairEmbedder
    torch.manual_seed(3)
    ang = TemplateAngleEmbedder(57, 256).to(dev, dtype).eval()
    pair = TemplatePairEmbedder(88, 64).to(dev, dtype).eval()
    extra = ExtraMSAEmbedder(25, 64).to(dev, dtype).eval()
    with torch.no_grad():
        for mod in (ang, pair, extra):
            for p in mod.parameters():
                p.copy_(torch.randn_like(p.float()) * 0.2)
        x = torch.randn(2, 33, 57, device=dev).to(dtype)
        want = F.linear(F.relu(F.linear(x.float(), ang.linear_1.weight.float(), ang.linear_1.bias.float())),
                        ang.linear_2.weight.float(), ang.linear_2.bias.float())
        _check(_f(ang(x)), want.cpu().numpy(), dtype)
        x = torch.randn(1, 21, 21, 88, device=dev).to(dtype)
        _check(_f(pair(x)), F.linear(x.float(), pair.linear.weight.float(), pair.linear.bias.float()).cpu().numpy(), dtype)
        x = torch.randn(40, 17, 25, device=dev).to(dtype)
        _check(_f(extra(x)), F.linear(x.float(), extra.linear.weight.float(), extra.linear.bias.float()).cpu().numpy(), dtype)
