"""Evoformer hot-path benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4|cfg3] [--no-cpu]

One step = one forward pass of the 48-block Evoformer stack (bf16, N_seq=128, random-init
weights ~N(0, 0.02^2), inputs ~N(0,1)) with inputs and weights resident in HBM.  The metric is
the Evoformer-block latency (ms per block = step time / 48).  The same JSON line carries
  roofline      the dominant kernel (flash attention core with bias: triangle + MSA-row attention),
                algorithmic FLOPs / HIP-event time of its launches inside the timed region,
  cpu_baseline  the CPU oracle (plain-PyTorch restatement of the reference's nn Evoformer block)
                timed on this box's host cores on a bounded sample,
and the op micro-benchmarks of benchmark configuration 2 (fused softmax, LayerNorm: HBM GB/s).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0

WORKLOADS = {
    "cfg3": dict(n_seq=128, n_res=256, tail=0.0, name="configs[2]: 48-block stack bf16 N_seq=128 N_res=256",
                 traffic_profile=None),
    "cfg4": dict(n_seq=128, n_res=1024, tail=0.05,
                 name="configs[3]: 48-block stack bf16 N_seq=128 N_res=1024, last 5% of residues masked",
                 traffic_profile="profiles/evoformer_blocks_cfg4_hbm_traffic.txt"),
}


def attention_traffic(profile):
    """HBM bytes per launch of the biased attention kernel, averaged over the launches the roofline object covers
    (triangle and MSA-row attention, weighted by their launch counts).  Hardware counters cannot be read inside a
    timed run: the figure is taken from the committed summary of the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
    of this script (rows ``attention_kernel<bf16, true>  workgroups  n  read MB  written MB`` of its table, already
    scaled by the calibration the file states); None when the file or its rows are missing."""
    if profile is None:
        return None
    try:
        lines = open(os.path.join(ROOT, profile)).read().splitlines()
    except OSError:
        return None
    tot, n = 0.0, 0
    for ln in lines:
        if not ln.startswith("attention_kernel<bf16, true>"):
            continue
        f = ln.split(">", 1)[1].split()
        try:
            launches, rd, wr = int(f[1]), float(f[2]), float(f[3])
        except (IndexError, ValueError):
            continue
        tot += launches * (rd + wr) * 1e6
        n += launches
    return round(tot / n) if n else None


def block_gflop(s, r, c_m=256, c_z=128, hm=8, hz=4, d=32, c_opm=32, c_mul=128, n=4):
    """Algorithmic GFLOP of one block: 2*M*N*K per contraction, un-padded shapes."""
    row_proj = 2 * s * r * c_m * (3 * hm * d) + 2 * (2 * s * r * c_m * hm * d) + 2 * r * r * c_z * hm
    row_core = 4 * s * hm * r * r * d
    col_proj = row_proj - 2 * r * r * c_z * hm
    col_core = 4 * r * hm * s * s * d
    mtrans = 4 * s * r * c_m * (n * c_m)
    opm = 4 * s * r * c_m * c_opm + 2 * r * r * s * c_opm ** 2 + 2 * r * r * c_opm ** 2 * c_z
    trimul = (2 * (2 * r * r * c_z * 2 * c_mul) + 2 * r * r * c_z * c_z + 2 * r * r * c_mul * c_z) + 2 * c_mul * r ** 3
    triatt = (2 * r * r * c_z * (3 * hz * d) + 2 * (2 * r * r * c_z * hz * d) + 2 * r * r * c_z * hz) + 4 * r * hz * r * r * d
    ptrans = 4 * r * r * c_z * (n * c_z)
    return (row_proj + row_core + col_proj + col_core + mtrans + opm + 2 * trimul + 2 * triatt + ptrans) / 1e9


def build_stack(no_blocks, dev, dtype, seed=0):
    import torch
    from fastfold_amd.model.fastnn import EvoformerStack
    from fastfold_amd.synthetic import synth_nn_state
    from fastfold_amd.utils.inject_fastnn import convert_nn_state_dict
    st = EvoformerStack(c_m=256, c_z=128, c_s=384, no_blocks=no_blocks, blocks_per_ckpt=1)
    st.load_state_dict(convert_nn_state_dict(synth_nn_state(seed=seed, no_blocks=no_blocks, std=0.02)), strict=True)
    return st.to(device=dev, dtype=dtype).eval()


def micro_ops(dev):
    """benchmark configuration 2: fused softmax [1,128,8,256,256] bf16 with pair bias and 10% masked keys;
    LayerNorm over [65536,128] and [32768,256] bf16; plus two plain copies of the same bytes as the practical
    HBM ceiling of this box: torch's copy_ and the library's streaming copy (ffk_stream_copy: the row kernels' own
    access pattern without their arithmetic).  Each op runs over rotating buffers (> 512 MB in
    total, so nothing is served from cache) as N launches recorded into one HIP graph; the time is
    the graph replay divided by N (no host launch overhead, no per-launch events)."""
    import torch
    from fastfold_amd import _lib
    from fastfold_amd.model.fastnn.kernel.softmax import _softmax_forward
    res = {}
    g = torch.Generator().manual_seed(0)

    def run(fn, n, nbytes, reps=5):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(n):
                fn(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(n):
                fn(i)
        graph.replay()
        torch.cuda.synchronize()
        us = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            us.append(e0.elapsed_time(e1) * 1e3 / n)
        med = sorted(us)[len(us) // 2]
        return {"us": round(med, 2), "GB/s": round(nbytes / med / 1e3, 1),
                "frac_of_8TBps": round(nbytes / med / 1e3 / PEAK_HBM_GBPS, 3)}

    nb = 4
    xs = [torch.randn(1, 128, 8, 256, 256, device=dev, dtype=torch.bfloat16) for _ in range(nb)]
    outs = [torch.empty_like(xs[0]) for _ in range(nb)]
    bias = torch.randn(1, 1, 8, 256, 256, device=dev, dtype=torch.bfloat16)
    mask = (torch.rand(1, 128, 256, generator=g) > 0.1).to(dev, torch.bfloat16)
    mask[..., 0] = 1
    nbytes = 2 * xs[0].numel() * 2
    res["softmax_bf16_1x128x8x256x256"] = run(
        lambda i: _softmax_forward(xs[i % nb], mask, bias, out=outs[i % nb]), 20, nbytes)
    # the form the reference's forward kernel has (softmax_cuda_kernel.cu:438-440, :521: probabilities overwrite the
    # logits): same bytes moved, half the footprint
    res["softmax_inplace_bf16_1x128x8x256x256"] = run(
        lambda i: _softmax_forward(xs[i % nb], mask, bias, out=xs[i % nb]), 20, nbytes)
    res["device_copy_same_bytes_as_softmax"] = run(lambda i: outs[i % nb].copy_(xs[i % nb]), 20, nbytes)
    res["stream_copy_same_bytes_as_softmax"] = run(
        lambda i: _lib.call("ffk_stream_copy", outs[i % nb].data_ptr(), xs[i % nb].data_ptr(), nbytes // 2, _lib.stream_ptr()),
        20, nbytes)
    del xs, outs
    for rows, cols in ((65536, 128), (32768, 256)):
        nb = 20
        xs = [torch.randn(rows, cols, device=dev, dtype=torch.bfloat16) for _ in range(nb)]
        os_ = [torch.empty_like(xs[0]) for _ in range(nb)]
        gam = (1 + 0.1 * torch.randn(cols, generator=g)).to(dev, torch.bfloat16)
        bet = (0.1 * torch.randn(cols, generator=g)).to(dev, torch.bfloat16)

        def f(i):
            _lib.call("ffk_layernorm_fwd", os_[i % nb].data_ptr(), None, None, xs[i % nb].data_ptr(), gam.data_ptr(),
                      bet.data_ptr(), rows, cols, 1e-5, _lib.FFK_BF16, _lib.stream_ptr())
        res["layernorm_bf16_%dx%d" % (rows, cols)] = run(f, 60, 2 * rows * cols * 2)
        if cols == 128:
            res["device_copy_same_bytes_as_layernorm"] = run(lambda i: os_[i % nb].copy_(xs[i % nb]), 60, 2 * rows * cols * 2)
            res["stream_copy_same_bytes_as_layernorm"] = run(
                lambda i: _lib.call("ffk_stream_copy", os_[i % nb].data_ptr(), xs[i % nb].data_ptr(), rows * cols * 2,
                                    _lib.stream_ptr()), 60, 2 * rows * cols * 2)
        del xs, os_
    return res


def feeder_stacks(dev, r):
    """The two stacks that run before the Evoformer (hub/alphafold.py:262-362) at their own widths, random
    weights: the 4-block extra-MSA stack on 1024 extra sequences and the 2-block template pair stack on one
    template, milliseconds per block; and the point-wise attention over four templates, milliseconds."""
    import torch
    from fastfold_amd.model.fastnn import ExtraMSAStack, TemplatePairStack

    def init(mod):
        g = torch.Generator().manual_seed(0)
        with torch.no_grad():
            for n, p in mod.named_parameters():
                ln_w = ("norm" in n) and n.endswith("weight")
                p.copy_((1.0 if ln_w else 0.0) + 0.02 * torch.randn(p.shape, generator=g))
        return mod.to(dev, torch.bfloat16).eval()

    def timed(fn, blocks, reps=3):
        # two untimed passes: the first packs the weights, the second lets the caching allocator settle on the
        # multi-GB intermediates (a pass that still has to ask the driver for memory is host-bound)
        with torch.no_grad():
            fn()
            fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                out = fn()
            torch.cuda.synchronize()
        assert bool(torch.isfinite(out.float()).all())
        return round((time.perf_counter() - t0) * 1e3 / reps / blocks, 4)

    res = {}
    se = 1024
    g = torch.Generator().manual_seed(1)
    ex = init(ExtraMSAStack(c_m=64, c_z=128, no_blocks=4))
    m = torch.randn(se, r, 64, generator=g).to(dev, torch.bfloat16)
    z = torch.randn(r, r, 128, generator=g).to(dev, torch.bfloat16)
    mm = torch.ones(se, r, device=dev, dtype=torch.bfloat16)
    pm = torch.ones(r, r, device=dev, dtype=torch.bfloat16)
    res["extra_msa_stack"] = {"workload": "4 blocks, N_extra=%d, N_res=%d, c_e=64" % (se, r),
                              "ms_per_block": timed(lambda: ex(m, z, chunk_size=None, msa_mask=mm, pair_mask=pm), 4)}
    del ex, m, z, mm
    tp = init(TemplatePairStack(c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_blocks=2, no_heads=4,
                                pair_transition_n=2, dropout_rate=0.25, blocks_per_ckpt=None))
    t = torch.randn(1, r, r, 64, generator=g).to(dev, torch.bfloat16)
    res["template_pair_stack"] = {"workload": "2 blocks, 1 template, N_res=%d, c_t=64" % r,
                                  "ms_per_block": timed(lambda: tp(t, pm[None], chunk_size=None), 2)}
    del tp, t
    from fastfold_amd.model.fastnn import TemplatePointwiseAttention
    pw = init(TemplatePointwiseAttention(c_t=64, c_z=128, c_hidden=16, no_heads=4, inf=1e5))
    t4 = torch.randn(4, r, r, 64, generator=g).to(dev, torch.bfloat16)
    z = torch.randn(r, r, 128, generator=g).to(dev, torch.bfloat16)
    tm = torch.ones(4, device=dev, dtype=torch.bfloat16)
    res["template_pointwise_attention"] = {"workload": "4 templates, N_res=%d" % r,
                                           "ms": timed(lambda: pw(t4, z, template_mask=tm), 1)}
    return res


def long_sequence(dev):
    """Benchmark configuration 5: one block at N_seq = 64, N_res = 4096 (z = 4.3 GB), chunk size 64, in place; latency
    and peak device memory."""
    import torch
    from fastfold_amd.model.fastnn import set_chunk_size
    s, r = 64, 4096
    stack = build_stack(1, dev, torch.bfloat16)
    g = torch.Generator().manual_seed(2)
    m = [torch.randn(s, r, 256, generator=g).to(dev, torch.bfloat16)]
    z = [torch.randn(r, r, 128, generator=g).to(dev, torch.bfloat16)]
    mm = torch.ones(s, r, device=dev, dtype=torch.bfloat16)
    pm = torch.ones(r, r, device=dev, dtype=torch.bfloat16)
    set_chunk_size(64)
    try:
        torch.cuda.reset_peak_memory_stats()
        with torch.no_grad():
            stack.inplace(m, z, mm, pm, chunk_size=64)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            stack.inplace(m, z, mm, pm, chunk_size=64)
            torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3
    finally:
        set_chunk_size(None)
    assert bool(torch.isfinite(z[0].float()).all())
    return {"workload": "configs[4]: 1 block bf16 N_seq=64 N_res=4096, chunk_size=64, in place",
            "ms_per_block": round(ms, 2), "block_tflop": round(block_gflop(s, r) / 1e3, 1),
            "tflops": round(block_gflop(s, r) / ms, 1), "peak_device_GB": round(torch.cuda.max_memory_allocated() / 1e9, 1)}


def forward_backward(dev, layers=4, trials=5, warm=2, r=256):
    """The reference's own harness shape (benchmark/perf.py:83-183): stand-alone blocks in training mode (dropout
    active), bf16, N_seq = 128, N_res = 256 (``r``), inputs that require gradients, ``layer_inputs[1].backward(grads)``;
    HIP-event times of the forward and of the backward pass per layer."""
    import torch
    from fastfold_amd.model.fastnn import Evoformer
    s = 128
    torch.manual_seed(0)
    blocks = [Evoformer(c_m=256, c_z=128, first_block=(i == 0), last_block=(i == layers - 1)).to(dev, torch.bfloat16)
              for i in range(layers)]
    node = torch.randn(s, r, 256, device=dev, dtype=torch.bfloat16).requires_grad_(True)
    pair = torch.randn(r, r, 128, device=dev, dtype=torch.bfloat16).requires_grad_(True)
    nm = torch.ones(s, r, device=dev, dtype=torch.bfloat16)
    pm = torch.ones(r, r, device=dev, dtype=torch.bfloat16)
    grads = torch.randn_like(pair)
    fwd = bwd = 0.0
    for t in range(trials + warm):
        e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        torch.cuda.synchronize()
        e0.record()
        x = (node, pair)
        for blk in blocks:
            x = blk(*x, nm, pm)
        e1.record()
        x[1].backward(grads)
        e2.record()
        torch.cuda.synchronize()
        if t >= warm:
            fwd += e0.elapsed_time(e1)
            bwd += e1.elapsed_time(e2)
    return {"workload": "benchmark/perf.py shape: %d stand-alone block(s), training mode, bf16, N_seq=128, N_res=%d" % (layers, r),
            "fwd_ms_per_block": round(fwd / trials / layers, 3), "bwd_ms_per_block": round(bwd / trials / layers, 3)}


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(threads):
    """The CPU oracle (plain-PyTorch fp32 restatement of the reference's nn Evoformer block, ``_mask_trans=False``)
    timed on the host cores: benchmark configuration 1 (one block, N_seq = 32, N_res = 64; 3 warm-up + 10 timed
    passes, median) and, as a second point, one block at N_seq = 128, N_res = 256 (1 + 5 passes)."""
    import numpy as np
    import torch
    from fastfold_amd.synthetic import synth_inputs, synth_nn_state
    from oracle.evoformer_ref import EvoformerStack as OracleStack
    torch.set_num_threads(threads)
    st = OracleStack(no_blocks=1).eval()
    st.load_state_dict({k: torch.from_numpy(v) for k, v in synth_nn_state(seed=0, no_blocks=1).items()})

    def timed(s, r, warm, n, budget_s):
        m, z, mm, pm = (torch.from_numpy(t) for t in synth_inputs(0, s, r))
        ts = []
        with torch.no_grad():
            for _ in range(warm):
                st(m, z, mm, pm, _mask_trans=False)
            t_end = time.time() + budget_s
            while len(ts) < n and (time.time() < t_end or len(ts) < 2):
                t0 = time.time()
                st(m, z, mm, pm, _mask_trans=False)
                ts.append((time.time() - t0) * 1e3)
        return ts

    t1 = timed(32, 64, 3, 10, 10.0)
    t3 = timed(128, 256, 1, 5, 20.0)
    return {"value": round(float(np.median(t1)), 2), "unit": "ms/block", "cores": torch.get_num_threads(),
            "kind": "port", "min": round(float(np.min(t1)), 2), "os_cpu_count": os.cpu_count(), "cpu_model": _cpu_model(),
            "sample": "configs[0]: 1 Evoformer block, fp32, N_seq=32 N_res=64 (10.9 GFLOP), oracle/evoformer_ref.py, "
                      "median of %d runs after 3 warm-ups; threads = the box's CPU share (OMP_NUM_THREADS), not "
                      "os.cpu_count()" % len(t1),
            "second_sample": {"workload": "1 block, fp32, N_seq=128 N_res=256 (configs[2] shape, 216.1 GFLOP)",
                              "value": round(float(np.median(t3)), 2), "unit": "ms/block", "runs": len(t3)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="cfg4", choices=sorted(WORKLOADS))
    ap.add_argument("--blocks", type=int, default=48)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-micro", action="store_true")
    ap.add_argument("--only-micro", action="store_true",
                    help="run only the operator micro-benchmarks of benchmark configuration 2 (for profiling them)")
    ap.add_argument("--only-feeders", action="store_true",
                    help="time only the extra-MSA and template pair stacks (for profiling them on their own)")
    ap.add_argument("--no-long-sequence", action="store_true",
                    help="skip the block at N_res = 4096 (a few seconds and about 30 GB of device memory)")
    ap.add_argument("--no-forward-backward", action="store_true",
                    help="skip the differentiable path timed the way benchmark/perf.py does (training-mode blocks, N_res = 256)")
    ap.add_argument("--plain-residual", action="store_true",
                    help="A/B switch: the reference's plain bf16 residual stream instead of the extended one")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the Evoformer on ONE GPU (DAP size 1, no collectives); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from fastfold_amd import _lib
    from fastfold_amd.synthetic import synth_inputs
    _lib.load()
    dev = torch.device("cuda:0")
    wl = WORKLOADS[args.workload]
    s, r = wl["n_seq"], wl["n_res"]
    if args.only_micro:
        print(json.dumps({"ops": micro_ops(dev)}))
        return
    if args.only_feeders:
        print(json.dumps({"feeders": feeder_stacks(dev, r)}))
        return
    stack = build_stack(args.blocks, dev, torch.bfloat16)
    if args.plain_residual:
        stack.extended_residual = False
    m, z, mm, pm = (torch.from_numpy(t).to(dev, torch.bfloat16) for t in synth_inputs(0, s, r, mask_tail_frac=wl["tail"]))

    def step():
        with torch.no_grad():
            return stack(m, z, mm, pm, chunk_size=None)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # HIP events bracket every attention launch of the first timed step only: an event pair costs the
    # stream about 10 us per launch, which the other steps do not have to carry
    rec = _lib.time_kernel("ffk_attention_fwd")
    others = {name: _lib.time_kernel(name) for name in ("ffk_bgemm_nt", "ffk_transition_fused", "ffk_opm_fused")}
    t0 = time.perf_counter()
    for i in range(args.steps):
        out = step()
        if i == 0:
            _lib.time_kernel("ffk_attention_fwd", enable=False)
            for name in others:
                _lib.time_kernel(name, enable=False)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    assert all(bool(torch.isfinite(t.float()).all()) for t in out), "non-finite output"

    # dominant kernel: attention core launches that carry a bias (MSA row + triangle start/end)
    flops, ms, n = 0.0, 0.0, 0
    for e0, e1, a in rec:
        if a[4] is None:       # bias_t == NULL: column attention (other kernel instantiation)
            continue
        B2, H, Nq, Nk = a[8], a[9], a[10], a[11]
        flops += 4.0 * B2 * H * Nq * Nk * 32
        ms += e0.elapsed_time(e1)
        n += 1
    ach = flops / (ms * 1e-3) / 1e12 if ms > 0 else 0.0
    roofline = {"bound": "mfma", "kernel": "attention_kernel<bf16, bias> (ffk_attention_fwd)",
                "achieved": round(ach, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(ach / PEAK_BF16_TFLOPS, 4), "traffic": attention_traffic(wl["traffic_profile"]),
                "traffic_unit": "bytes/launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, see profiles/)",
                "launches": n, "avg_launch_ms": round(ms / max(n, 1), 4),
                "flops_per_launch_avg": round(flops / max(n, 1) / 1e9, 2)}

    # the other matrix-pipe kernels of the block, timed the same way (HIP events around their launches in the
    # first timed step): algorithmic flops of the launch / its duration, against the dense bf16 peak
    def summarise(records, gflop_of):
        acc = {}
        for e0, e1, a in records:
            k = gflop_of(a)
            if k is None:
                continue
            name, gf = k
            t = acc.setdefault(name, [0, 0.0, gf])
            t[0] += 1
            t[1] += e0.elapsed_time(e1)
        return {name: {"launches": n_, "avg_ms": round(ms_ / n_, 4), "gflop": round(gf, 1),
                       "TFLOP/s": round(gf / (ms_ / n_), 1), "frac_of_peak": round(gf / (ms_ / n_) / PEAK_BF16_TFLOPS, 3)}
                for name, (n_, ms_, gf) in acc.items()}

    def bgemm_kind(a):
        d = a[0]._obj
        if d.batch == 128 and d.M == r and d.N == r:
            return "trimul_contraction_bgemm_big", 2.0 * d.batch * d.M * d.N * d.K / 1e9
        return None
    kernels = {}
    kernels.update(summarise(others["ffk_bgemm_nt"], bgemm_kind))
    kernels.update(summarise(others["ffk_transition_fused"],
                             lambda a: ("transition_fused_C%d" % a[10], 4.0 * a[9] * a[10] * a[11] / 1e9)))
    kernels.update(summarise(others["ffk_opm_fused"],
                             lambda a: ("opm_fused", 2.0 * r * r * (32 * 32 * s + 1024 * 128) / 1e9)))

    line = {
        "metric": "Evoformer-block latency, bf16, N_seq=%d, N_res=%d (stack of %d blocks)" % (s, r, args.blocks),
        "value": round(ms_per_step / args.blocks, 4), "unit": "ms/block",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": wl["name"], "blocks": args.blocks, "n_seq": s, "n_res": r,
                   "block_gflop": round(block_gflop(s, r), 1),
                   "stack_tflops": round(block_gflop(s, r) * args.blocks / ms_per_step, 1),
                   "residual_stream": "bf16" if args.plain_residual else "bf16 + int8 tail (24-bit)"},
        "roofline": roofline,
        "kernels": kernels,
    }
    if args.workload == "cfg4" and not args.no_micro:
        # the same stack at benchmark configuration 3 (N_res = 256), reported beside the headline number
        w3 = WORKLOADS["cfg3"]
        m3, z3, mm3, pm3 = (torch.from_numpy(t).to(dev, torch.bfloat16)
                            for t in synth_inputs(0, w3["n_seq"], w3["n_res"], mask_tail_frac=w3["tail"]))
        with torch.no_grad():
            stack(m3, z3, mm3, pm3, chunk_size=None)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(3):
                stack(m3, z3, mm3, pm3, chunk_size=None)
            torch.cuda.synchronize()
        line["secondary"] = {"workload": w3["name"], "ms_per_block": round((time.perf_counter() - t0) * 1e3 / 3 / args.blocks, 4)}
        del m3, z3, mm3, pm3
    del stack, out
    torch.cuda.empty_cache()
    if not args.no_long_sequence and args.workload == "cfg4":
        line["long_sequence"] = long_sequence(dev)
        torch.cuda.empty_cache()
    if not args.no_forward_backward and not args.no_micro:
        line["forward_backward"] = forward_backward(dev)
        if args.workload == "cfg4":         # the same at the headline size: one block, forward + backward
            line["forward_backward_n_res_1024"] = forward_backward(dev, layers=1, trials=2, warm=1, r=1024)
        torch.cuda.empty_cache()
    if not args.no_micro:
        line["feeders"] = feeder_stacks(dev, r)
        line["ops"] = micro_ops(dev)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
