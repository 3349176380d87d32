"""GPU tests of the module-level API surface that the block / stack tests do not reach: the stand-alone
``SelfAttention`` module, the ``inplace`` variants of the sub-modules, wide ``Linear`` layers, the
default masks of the extra-MSA stack and the forward-only guard.

``SelfAttention`` is checked against a float64 restatement of fastnn/ops.py:296-324 written out here
(projection, scaled logits + bias + 1e9 * (mask - 1), softmax, sigmoid gate, output projection);
tolerances are the north star's: fp32 max-abs <= 1e-4, bf16 relative L2 <= 2e-2."""
import numpy as np
import pytest
import torch

from fastfold_amd.synthetic import synth_inputs, synth_nn_state

pytestmark = pytest.mark.gpu


def _rel_l2(a, b):
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def _self_attention_f64(mod, x, mask, bias_bhqk):
    """x [1, B2, N, C], mask [1, B2, N] or None, bias [1, H, N, N] or None -> [1, B2, N, out_dim]."""
    H, c = mod.n_head, mod.c
    p = {k: v.detach().double().cpu() for k, v in mod.state_dict().items()}
    x = x.double().cpu()
    qkv = x @ p["to_qkv.weight"].T
    q, k, v = (t.unflatten(-1, (H, c)).transpose(-2, -3) for t in qkv.chunk(3, dim=-1))      # [1, B2, H, N, c]
    logits = (q * c ** -0.5) @ k.transpose(-1, -2)
    if bias_bhqk is not None:
        logits = logits + bias_bhqk.double().cpu().unsqueeze(1)
    if mask is not None:
        logits = logits + (1e9 * (mask.double().cpu() - 1))[..., None, None, :]
    w = torch.softmax(logits, -1)
    o = (w @ v).transpose(-2, -3).flatten(-2)
    g = torch.sigmoid(x @ p["gating_linear.weight"].T + p["gating_bias"])
    out = (o * g) @ p["o_linear.weight"].T
    if "o_linear.bias" in p:
        out = out + p["o_linear.bias"]
    return out.numpy()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("qkv_dim,c,H,out_dim,B2,N,bias_form,use_mask,fuse", [
    (256, 32, 8, 256, 5, 40, "bhqk", True, False),
    (128, 32, 4, 128, 7, 33, "bqkh", True, True),
    (64, 16, 4, 64, 3, 72, None, False, False),
    (64, 8, 8, 64, 4, 24, "bhqk", True, True),
])
def test_self_attention_module(dev, dtype, qkv_dim, c, H, out_dim, B2, N, bias_form, use_mask, fuse):
    from fastfold_amd.model.fastnn.ops import SelfAttention
    g = torch.Generator().manual_seed(101 + qkv_dim + c)
    mod = SelfAttention(qkv_dim, c, H, out_dim, gating=True, last_bias_fuse=fuse)
    with torch.no_grad():
        for n, p in mod.named_parameters():
            fan = p.shape[-1] if p.dim() == 2 else 1
            p.copy_(torch.randn(p.shape, generator=g) * (fan ** -0.5 if p.dim() == 2 else 0.3))
    mod = mod.to(dev, dtype).eval()
    x = torch.randn(1, B2, N, qkv_dim, generator=g).to(dev, dtype)
    mask = None
    if use_mask:
        mask = (torch.rand(1, B2, N, generator=g) > 0.2).float()
        mask[..., 0] = 1.0
        mask = mask.to(dev, dtype)
    bias, arg = None, None
    if bias_form is not None:
        bias = torch.randn(1, H, N, N, generator=g).to(dev, dtype)
        arg = (bias, -1) if bias_form == "bhqk" else (bias.permute(0, 2, 3, 1).contiguous(), None)
    with torch.no_grad():
        got = mod(x, mask, arg)
    assert got.shape == (1, B2, N, out_dim) and got.dtype == dtype
    ref = _self_attention_f64(mod, x, mask, bias)
    got = got.float().cpu().numpy()
    if dtype == torch.float32:
        scale = max(1.0, float(np.abs(ref).max()))
        assert np.abs(got - ref).max() <= 1e-4 * scale, np.abs(got - ref).max()
    else:
        assert _rel_l2(got, ref) <= 2e-2, _rel_l2(got, ref)


def test_self_attention_rejects_unsupported(dev):
    from fastfold_amd.model.fastnn.ops import SelfAttention
    x = torch.zeros(1, 2, 8, 64, device=dev)
    with torch.no_grad():
        with pytest.raises(RuntimeError, match="head dim"):
            SelfAttention(64, 64, 4, 64).to(dev)(x, None)
        with pytest.raises(RuntimeError, match="head dim"):
            SelfAttention(64, 16, 4, 64, gating=False).to(dev)(x, None)
        with pytest.raises(RuntimeError, match=r"\[1, B2, N, C\]"):
            SelfAttention(64, 16, 4, 64).to(dev)(x[0], None)


def _block(dev, dtype, cls_name):
    import copy
    from oracle.evoformer_ref import OracleModel
    from fastfold_amd.utils.inject_fastnn import inject_fastnn
    kw = dict(c_m=256, c_z=128, c_hidden_msa_att=32, c_hidden_opm=32, c_hidden_mul=128, c_hidden_pair_att=32,
              c_s=384, no_heads_msa=8, no_heads_pair=4, transition_n=4, msa_dropout=0.15, pair_dropout=0.25,
              blocks_per_ckpt=1, inf=1e9, eps=1e-8)
    model = OracleModel(no_blocks=1, **kw).eval()
    sd = synth_nn_state(seed=33, no_blocks=1, fan_in_scaled=True)
    model.evoformer.load_state_dict({k: torch.from_numpy(v) for k, v in sd.items()}, strict=True)
    return inject_fastnn(copy.deepcopy(model)).evoformer.to(device=dev, dtype=dtype).eval().blocks[0]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_submodule_inplace_equals_forward(dev, dtype):
    """Every ``inplace(...)`` variant (list-wrapped tensor updated in place, fastnn/ops.py:121, 222, 676, 860,
    1010, 1134, 1261) gives bit-for-bit the tensor ``forward`` returns."""
    blk = _block(dev, dtype, "Evoformer")
    m, z, mm, pm = (torch.from_numpy(np.ascontiguousarray(t[None])).to(dev, dtype)
                    for t in synth_inputs(5, 10, 40, mask_tail_frac=0.1))
    msa, pair = blk.msa, blk.pair
    cases = [
        ("opm", lambda: blk.communication(m, mm, z), lambda: blk.communication.inplace(m, mm, [z.clone()])),
        ("tmo", lambda: pair.TriangleMultiplicationOutgoing(z, pm),
         lambda: pair.TriangleMultiplicationOutgoing.inplace([z.clone()], pm)),
        ("tmi", lambda: pair.TriangleMultiplicationIncoming(z, pm),
         lambda: pair.TriangleMultiplicationIncoming.inplace([z.clone()], pm)),
        ("tas", lambda: pair.TriangleAttentionStartingNode(z, pm),
         lambda: pair.TriangleAttentionStartingNode.inplace([z.clone()], pm)),
        ("tae", lambda: pair.TriangleAttentionEndingNode(z, pm),
         lambda: pair.TriangleAttentionEndingNode.inplace([z.clone()], pm)),
        ("ptrans", lambda: pair.PairTransition(z), lambda: pair.PairTransition.inplace([z.clone()])),
        ("msa_core", lambda: msa(m, z, mm), lambda: msa.inplace(m.clone(), z, mm)),
        ("pair_core", lambda: pair(z, pm), lambda: pair.inplace([z.clone()], pm)),
    ]
    # the extra-MSA core holds the chunked row attention and transition, which have the in-place form
    from fastfold_amd.model.fastnn import ExtraMSABlock
    torch.manual_seed(6)
    xb = ExtraMSABlock(64, 128, first_block=True, last_block=True)
    with torch.no_grad():
        for n, p in xb.named_parameters():
            p.copy_((1.0 if ("norm" in n.lower() and n.endswith("weight")) else 0.0) + 0.08 * torch.randn_like(p))
    xb = xb.to(dev, dtype).eval()
    xm = torch.randn(1, 10, 40, 64, device=dev).to(dtype)
    xs = xb.msa_stack
    cases += [
        ("x_row", lambda: xs.MSARowAttentionWithPairBias(xm, z, mm),
         lambda: xs.MSARowAttentionWithPairBias.inplace([xm.clone()], z, mm)),
        ("x_mtrans", lambda: xs.MSATransition(xm), lambda: xs.MSATransition.inplace([xm.clone()])),
        ("x_core", lambda: xs(xm, z, mm), lambda: xs.inplace([xm.clone()], z, mm)),
    ]
    with torch.no_grad():
        for name, fwd, inp in cases:
            a = fwd()
            b = inp()
            b = b[0] if isinstance(b, (list, tuple)) else b
            assert a.shape == b.shape and torch.equal(a, b), name


def test_column_global_attention_inplace_equals_forward(dev):
    from fastfold_amd.model.fastnn.ops import ChunkMSAColumnGlobalAttention
    torch.manual_seed(3)
    mod = ChunkMSAColumnGlobalAttention(64, 8, 8)
    with torch.no_grad():
        for n, p in mod.named_parameters():
            p.copy_((1.0 if ("norm" in n.lower() and n.endswith("weight")) else 0.0) + 0.1 * torch.randn_like(p))
    mod = mod.to(dev).eval()
    m = torch.randn(1, 50, 24, 64, device=dev)
    mask = (torch.rand(1, 50, 24, device=dev) > 0.1).float()
    with torch.no_grad():
        a = mod(m, mask)
        b = mod.inplace([m.clone()], mask)[0]
    assert torch.equal(a, b)


def test_template_block_inplace_equals_forward(dev):
    from fastfold_amd.model.fastnn import TemplatePairBlock
    torch.manual_seed(4)
    blk = TemplatePairBlock(c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_heads=4, pair_transition_n=2,
                            dropout_rate=0.25, inf=1e9, first_block=True, last_block=True)
    with torch.no_grad():
        for n, p in blk.named_parameters():
            p.copy_((1.0 if ("norm" in n.lower() and n.endswith("weight")) else 0.0) + 0.08 * torch.randn_like(p))
    blk = blk.to(dev).eval()
    t = torch.randn(1, 36, 36, 64, device=dev)
    mask = (torch.rand(36, 36, device=dev) > 0.1).float()
    with torch.no_grad():
        a = blk(t, mask)
        b = blk.inplace([t.clone()], mask)[0]
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fin,fout,rows", [(384, 128, 77), (1024, 64, 130), (320, 200, 9)])
def test_linear_wide_input(dev, dtype, fin, fout, rows):
    """in_features above 256 take the batched-GEMM route; same numbers as torch.nn.functional.linear."""
    from fastfold_amd.model.fastnn.ops import Linear
    g = torch.Generator().manual_seed(fin + fout)
    lin = Linear(fin, fout)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(fout, fin, generator=g) * fin ** -0.5)
        lin.bias.copy_(torch.randn(fout, generator=g) * 0.3)
    x = torch.randn(3, rows, fin, generator=g)
    ref = torch.nn.functional.linear(x.double(), lin.weight.detach().double(), lin.bias.detach().double()).numpy()
    lin = lin.to(dev, dtype)
    with torch.no_grad():
        got = lin(x.to(dev, dtype))
    assert got.shape == (3, rows, fout)
    got = got.float().cpu().numpy()
    if dtype == torch.float32:
        assert np.abs(got - ref).max() <= 1e-4 * max(1.0, float(np.abs(ref).max()))
    else:
        assert _rel_l2(got, ref) <= 2e-2


def test_extra_msa_stack_default_masks(dev):
    """msa_mask / pair_mask left out mean all-ones masks (fastnn/msa.py:355-359 call sites pass them; the nn
    stack's signature makes them optional, nn/evoformer.py:604-609)."""
    from fastfold_amd.model.fastnn import ExtraMSAStack
    torch.manual_seed(8)
    st = ExtraMSAStack(c_m=64, c_z=128, no_blocks=2)
    with torch.no_grad():
        for n, p in st.named_parameters():
            p.copy_((1.0 if ("norm" in n.lower() and n.endswith("weight")) else 0.0) + 0.05 * torch.randn_like(p))
    st = st.to(dev).eval()
    m = torch.randn(20, 24, 64, device=dev)
    z = torch.randn(24, 24, 128, device=dev)
    with torch.no_grad():
        a = st(m, z, chunk_size=None)
        b = st(m, z, chunk_size=None, msa_mask=torch.ones(20, 24, device=dev), pair_mask=torch.ones(24, 24, device=dev))
    assert torch.equal(a, b)


def test_forward_only_guard(dev):
    """A call whose input asks for gradients takes the differentiable composition; the in-place variants are
    forward-only launches and raise instead of returning a tensor cut off from the graph."""
    from fastfold_amd.model.fastnn.ops import ChunkTransition, Linear
    lin = Linear(64, 64).to(dev)
    x = torch.randn(4, 64, device=dev, requires_grad=True)
    y = lin(x)
    assert y.grad_fn is not None
    y.sum().backward()
    assert torch.allclose(x.grad, lin.weight.sum(0).expand(4, 64), atol=1e-5)
    from fastfold_amd import _lib
    assert torch.equal(lin(x, act=_lib.FFK_ACT_RELU), torch.relu(y))      # the fused activations, differentiably
    with torch.no_grad():
        assert not lin(x).requires_grad
        assert torch.allclose(lin(x), y, atol=1e-5)
    tr = ChunkTransition(128).to(dev)
    z = torch.randn(1, 8, 8, 128, device=dev, requires_grad=True)
    with pytest.raises(NotImplementedError, match="forward pass only"):
        tr.inplace([z])
    assert tr(z).grad_fn is not None


def test_dropout_modules_are_identity_in_eval(dev):
    """DropoutRowwise / DropoutColumnwise (fastnn/ops.py:33-66) share one mask along a dimension; in eval
    mode they leave the tensor unchanged."""
    from fastfold_amd.model.fastnn.ops import DropoutRowwise, DropoutColumnwise
    x = torch.randn(1, 6, 7, 8, device=dev)
    for cls in (DropoutRowwise, DropoutColumnwise):
        d = cls(0.25).eval()
        assert torch.equal(d(x), x)
        d.train()
        y = d(x)
        keep = (y != 0).float()
        # the mask is shared along rows (dim 1) or columns (dim 2)
        dim = 1 if cls is DropoutRowwise else 2
        assert torch.equal(keep, keep.narrow(dim, 0, 1).expand_as(keep))


def test_side_stream_matches_default_stream(dev):
    """Launches go to the caller's current stream: a block run on a side stream gives the bits of the default stream."""
    blk = _block(dev, torch.bfloat16, "Evoformer")
    m, z, mm, pm = (torch.from_numpy(np.ascontiguousarray(t)).to(dev, torch.bfloat16)
                    for t in synth_inputs(8, 12, 72, mask_tail_frac=0.1))
    with torch.no_grad():
        rm, rz = blk(m, z, mm, pm)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            gm, gz = blk(m, z, mm, pm)
        side.synchronize()
    assert torch.equal(gm, rm) and torch.equal(gz, rz)


def test_block_forward_replays_from_a_captured_graph(dev):
    """One block forward captured in a HIP graph and replayed with new input contents, with eager work and
    synchronisations between the replays: every replay equals the eager result on the same inputs."""
    blk = _block(dev, torch.bfloat16, "Evoformer")
    ins = [[torch.from_numpy(np.ascontiguousarray(t)).to(dev, torch.bfloat16)
            for t in synth_inputs(20 + i, 16, 64, mask_tail_frac=0.1)] for i in range(3)]
    static = [t.clone() for t in ins[0]]
    with torch.no_grad():
        eager = [blk(*x) for x in ins]                      # also warms the weight packs and launch attributes
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            blk(*static)                                    # warm-up on the capture stream
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            gm, gz = blk(*static)
        for i in (1, 2, 0, 1):
            for dst, src in zip(static, ins[i]):
                dst.copy_(src)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(gm, eager[i][0]) and torch.equal(gz, eager[i][1]), "replay with input set %d" % i
            blk(*ins[(i + 1) % 3])                          # eager work between replays
            torch.cuda.synchronize()


def test_empty_inputs_raise(dev):
    """No sequence or no residue is an error of the caller, reported before any launch."""
    blk = _block(dev, torch.float32, "Evoformer")
    for s, r in ((0, 8), (4, 0)):
        m, z = torch.zeros(s, r, 256, device=dev), torch.zeros(r, r, 128, device=dev)
        with torch.no_grad(), pytest.raises(RuntimeError, match="empty input"):
            blk(m, z, torch.ones(s, r, device=dev), torch.ones(r, r, device=dev))


def test_forward_leaves_inputs_untouched_for_a_single_sequence(dev):
    """A middle block's ``forward`` un-pads with a slice that is already contiguous when N_seq = 1; it must still
    work on a private copy (the reference's forward never writes to its inputs)."""
    blk = _block(dev, torch.float32, "Evoformer")
    blk.first_block, blk.last_block = False, False
    s, r = 1, 12
    g = torch.Generator().manual_seed(0)
    m = torch.randn(1, s, r + 1, 256, generator=g).to(dev)
    z = torch.randn(1, r + 1, r + 1, 128, generator=g).to(dev)
    mm, pm = torch.ones(s, r, device=dev), torch.ones(r, r, device=dev)
    m0, z0 = m.clone(), z.clone()
    with torch.no_grad():
        a, b = blk(m, z, mm, pm)
    assert torch.equal(m, m0) and torch.equal(z, z0)
    assert a.shape == m.shape and float((a[:, :, :r] - m0[:, :, :r]).abs().max()) > 1e-3


def test_packed_weights_follow_the_parameters(dev):
    """Kernel-ready weight copies are rebuilt after in-place parameter updates, ``load_state_dict`` and casts; a
    write through ``.data`` needs ``invalidate_packed()``."""
    from fastfold_amd.model.fastnn.ops import Linear
    lin = Linear(64, 32).to(dev)
    x = torch.randn(5, 64, device=dev)
    with torch.no_grad():
        y0 = lin(x)
        lin.weight.mul_(2.0)                                     # in-place op: version counter
        assert torch.allclose(lin(x) - lin.bias, 2 * (y0 - lin.bias), atol=1e-4)
        sd = {k: v.clone() for k, v in lin.state_dict().items()}
        sd["weight"] = sd["weight"] * 0.5
        lin.load_state_dict(sd)                                  # copy_ under no_grad, plus the explicit hook
        assert torch.allclose(lin(x), y0, atol=1e-4)
        lin.weight.data.copy_(sd["weight"] * 3.0)                # invisible to the version counter
        lin.invalidate_packed()
        assert torch.allclose(lin(x) - lin.bias, 3 * (y0 - lin.bias), atol=1e-4)
        lin = lin.to(torch.bfloat16)                             # _apply drops the cache
        assert lin(x.to(torch.bfloat16)).dtype == torch.bfloat16


def test_elementwise_ops_keep_the_graph(dev):
    from fastfold_amd.model.fastnn.kernel import bias_dropout_add, bias_ele_dropout_residual, bias_sigmod_ele
    x = torch.randn(1, 4, 6, 32, device=dev, requires_grad=True)
    b = torch.zeros(32, device=dev)
    dm = torch.ones(1, 1, 6, 32, device=dev)
    assert bias_sigmod_ele(x, b, x.detach()).grad_fn is not None
    assert bias_dropout_add(x, b, dm, x.detach(), prob=0.1, training=False).grad_fn is not None
    assert bias_ele_dropout_residual(x.detach(), b, x, dm, x.detach(), prob=0.1, training=False).grad_fn is not None
    with torch.no_grad():
        assert bias_sigmod_ele(x, b, x).shape == x.shape
