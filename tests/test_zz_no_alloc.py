"""ffk_pair_bias_static, the entry point that allocates nothing (its scratch is a static device array of the
library): bit-identical to ffk_pair_bias on two calls in a row, the second on a smaller input."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(dev, r, H, C, seed):
    g = torch.Generator().manual_seed(seed)
    dt = torch.bfloat16
    z = (torch.randn(r, r, C, generator=g) * 1.5 + 0.4).to(dev, dt)
    wb = (torch.randn(H, C, generator=g) / C ** 0.5).to(dev, dt)
    gam = (1 + 0.1 * torch.randn(C, generator=g)).to(dev, dt)
    bet = (0.1 * torch.randn(C, generator=g)).to(dev, dt)
    return z, wb, gam, bet


def test_pair_bias_static_matches_pair_bias(dev):
    from fastfold_amd import _lib
    lib = _lib.load()
    st = _lib.stream_ptr()
    # (residues, heads, channels): the second call is smaller in every dimension, the third uses the transposed traversal
    cases = [(96, 8, 128, False), (45, 4, 64, False), (64, 4, 128, True)]
    for i, (r, H, C, transposed) in enumerate(cases):
        z, wb, gam, bet = _inputs(dev, r, H, C, seed=100 + i)
        T = (r + 31) // 32
        amap = (r, C, r * C) if transposed else (r * r, 0, C)
        want = torch.zeros(H, T, T, 1024, dtype=torch.bfloat16, device=dev)
        scratch = torch.empty(16 * C + 16, dtype=torch.float32, device=dev)
        rc = lib.ffk_pair_bias(want.data_ptr(), z.data_ptr(), gam.data_ptr(), bet.data_ptr(), wb.data_ptr(),
                               scratch.data_ptr(), r, C, H, amap[0], amap[1], amap[2], _lib.LOG2E, 1e-5, _lib.FFK_BF16, st)
        assert rc == 0, lib.ffk_last_error_string()
        got = torch.zeros_like(want)
        args = (got.data_ptr(), z.data_ptr(), gam.data_ptr(), bet.data_ptr(), wb.data_ptr(),
                r, C, H, amap[0], amap[1], amap[2], _lib.LOG2E, 1e-5, _lib.FFK_BF16, st)
        if i == 0:
            # one untimed call first: the code object load and the one-time symbol lookup of a device are not
            # what "allocates nothing" is about
            assert lib.ffk_pair_bias_static(*args) == 0, lib.ffk_last_error_string()
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        free_before = torch.cuda.mem_get_info()[0]        # the driver's view: sees a hipMalloc made by the library too
        rc = lib.ffk_pair_bias_static(*args)
        assert rc == 0, lib.ffk_last_error_string()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] == free_before, "free device memory changed across the call"
        assert float(want.float().abs().max()) > 0.5
        assert torch.equal(got, want), "case %d: static-scratch result differs" % i


def test_pair_bias_static_rejects_what_does_not_fit(dev):
    from fastfold_amd import _lib
    lib = _lib.load()
    buf = torch.zeros(4096, dtype=torch.bfloat16, device=dev)
    p = buf.data_ptr()
    args = lambda C, H: (p, p, p, p, p, 32, C, H, 1024, 0, C, 1.0, 1e-5, _lib.FFK_BF16, None)
    assert lib.ffk_pair_bias_static(*args(256, 4)) == 2 and b"static scratch" in lib.ffk_last_error_string()
    assert lib.ffk_pair_bias_static(*args(128, 9)) == 2
    # the weight operand is rebuilt by every call: w / gamma / beta may not be omitted
    assert lib.ffk_pair_bias_static(p, p, None, None, None, 32, 128, 4, 1024, 0, 128, 1.0, 1e-5, _lib.FFK_BF16, None) == 3
