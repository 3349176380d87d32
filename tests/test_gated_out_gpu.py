"""ffk_gated_out_fused (the output stage of a gated attention with the gate computed in place) through the C ABI
against float64:  out = x + Wo (sigmoid(Wg LN(x) + bg) * o) + bo  (fastfold/model/fastnn/ops.py:320-324)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ref(x, gam, bet, wg, bg, o, wo, bo):
    x, gam, bet, wg, bg, o, wo = (t.double().cpu() for t in (x, gam, bet, wg, bg, o, wo))
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    xn = ((x - mu) / torch.sqrt(var + 1e-5) * gam + bet).to(torch.bfloat16).double()     # the kernel multiplies rounded rows
    g = torch.sigmoid(xn @ wg.t() + bg.double().cpu())
    upd = (g * o) @ wo.t()
    if bo is not None:
        upd = upd + bo.double().cpu()
    return x + upd, upd


@pytest.mark.parametrize("C", [128, 256])
@pytest.mark.parametrize("rows,transposed", [(64 * 40, False), (1000, False), (48 * 48, True)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_gated_out_against_float64(dev, C, rows, transposed, with_bias):
    from fastfold_amd import _lib
    g = torch.Generator().manual_seed(C + rows)
    dt = torch.bfloat16
    if transposed:                      # logical row (j, i) lives at x[i, j]: inner = r, s_o = C, s_i = r * C
        r = int(round(rows ** 0.5))
        x = (torch.randn(r, r, C, generator=g) * 1.5 + 0.3).to(dev, dt)
        inner, s_o, s_i = r, C, r * C
        x_log = x.transpose(0, 1).reshape(rows, C)
    else:
        x = (torch.randn(rows, C, generator=g) * 1.5 + 0.3).to(dev, dt)
        inner, s_o, s_i = rows, 0, C
        x_log = x
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dt)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dt)
    wg = (torch.randn(C, C, generator=g) / C ** 0.5).to(dev, dt)
    bg = torch.randn(C, generator=g).to(dev, dt)
    wo = (torch.randn(C, C, generator=g) / C ** 0.5).to(dev, dt)
    bo = torch.randn(C, generator=g).to(dev, dt) if with_bias else None
    o = torch.randn(rows, C, generator=g).to(dev, dt)
    want, upd = _ref(x_log, gam, bet, wg, bg, o, wo, bo)
    out = torch.empty_like(x)
    _lib.gated_out_fused(out, x, gam, bet, wg, bg, o, wo, bo, M=rows, C=C, inner=inner, s_o=s_o, s_i=s_i)
    got = (out.transpose(0, 1).reshape(rows, C) if transposed else out).double().cpu()
    err = float((got - want).norm() / upd.norm())          # measured on the update: the residual would hide it
    assert err < 1.5e-2, err
    # in place, with the residual tail: the 24-bit stream (bf16 + tail byte) moves by the same update
    tail = torch.zeros(x.shape, dtype=torch.int8, device=dev)
    x2 = x.clone()
    _lib.gated_out_fused(x2, x2, gam, bet, wg, bg, o, wo, bo, M=rows, C=C, inner=inner, s_o=s_o, s_i=s_i, xtail=tail)
    # a zero tail on entry: the rounded stream is the plain result up to the tie rule (the stream rounds halves away
    # from zero, the plain store to even; sums of two bf16 numbers are ties one time in ten): one bf16 step at most
    assert float(((x2.float() - out.float()).abs() / out.float().abs().clamp_min(1e-3)).max()) <= 2.0 ** -7
    bits = (x2.view(torch.int16).to(torch.int32) << 16) + (tail.to(torch.int32) << 8)
    val = bits.view(torch.float32)
    val = (val.transpose(0, 1).reshape(rows, C) if transposed else val).double().cpu()
    err24 = float((val - want).norm() / upd.norm())
    assert err24 < err + 1e-4 and err24 < 1.5e-2, (err24, err)


def test_gated_out_rejects_what_it_is_not_built_for(dev):
    from fastfold_amd import _lib
    x = torch.zeros(64, 64, dtype=torch.bfloat16, device=dev)
    v = torch.zeros(64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="128 and 256"):
        _lib.gated_out_fused(x, x, v, v, x, v, x, x, v, M=64, C=64, inner=64, s_o=0, s_i=64)
    xf = torch.zeros(128, 128, device=dev)
    with pytest.raises(RuntimeError, match="bf16"):
        _lib.gated_out_fused(xf, xf, xf[0], xf[0], xf, xf[0], xf, xf, xf[0], M=128, C=128, inner=128, s_o=0, s_i=128)


def test_attention_gate_in_output_stage_matches_gate_tensor_path(dev):
    """The triangle attention and both MSA attentions with the gate computed in the output stage against the same
    modules with the gate as a tensor (written by the projection, read by the core): same results up to the bf16
    rounding of the gate and of the ungated head outputs."""
    from fastfold_amd.model.fastnn import _fused
    from fastfold_amd.model.fastnn.msa import MSAColumnAttention, MSARowAttentionWithPairBias
    from fastfold_amd.model.fastnn.ops import ChunkTriangleAttentionEndingNode, ChunkTriangleAttentionStartingNode
    torch.manual_seed(3)
    r, s = 64, 32
    dt = torch.bfloat16

    def init(mod):
        with torch.no_grad():
            for n, p in mod.named_parameters():
                if "layernorm" in n and n.endswith("weight"):
                    p.copy_(1 + 0.1 * torch.randn_like(p))
                else:
                    p.copy_(torch.randn_like(p) * (0.3 if p.dim() == 1 else p.shape[-1] ** -0.5))
        return mod.to(dev, dt).eval()
    z = torch.randn(1, r, r, 128, device=dev).to(dt)
    m = torch.randn(1, s, r, 256, device=dev).to(dt)
    zm = torch.ones(1, r, r, device=dev, dtype=dt)
    zm[:, :, -5:] = 0
    zm[:, -5:] = 0
    mm = torch.ones(1, s, r, device=dev, dtype=dt)
    mm[:, :, -5:] = 0
    cases = [(init(ChunkTriangleAttentionStartingNode(128, 0.25, c=32, n_head=4)), (z, zm)),
             (init(ChunkTriangleAttentionEndingNode(128, 0.25, c=32, n_head=4)), (z, zm)),
             (init(MSARowAttentionWithPairBias(256, 128)), (m, z, mm)),
             (init(MSAColumnAttention(256)), (m, mm))]
    for mod, args in cases:
        outs = []
        for on in (True, False):
            _fused._GATE_IN_OUT_STAGE = on
            keep = (_fused._GATE_IN_OUT_MIN_N, _fused._GATE_IN_OUT_WIDTHS)
            _fused._GATE_IN_OUT_MIN_N, _fused._GATE_IN_OUT_WIDTHS = 0, (128, 256)      # small shapes and the MSA width too
            try:
                with torch.no_grad():
                    outs.append(mod(*args).float())
            finally:
                _fused._GATE_IN_OUT_STAGE = True
                _fused._GATE_IN_OUT_MIN_N, _fused._GATE_IN_OUT_WIDTHS = keep
        upd = outs[1] - args[0].float()
        assert float(upd.norm()) > 1.0
        err = float((outs[0] - outs[1]).norm() / upd.norm())
        assert err < 2e-2, (type(mod).__name__, err)
