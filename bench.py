#!/usr/bin/env python3
"""Benchmark of the D2Conv3D operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload c3|c1|c2_f32|c2_bf16|c3_f32|c4|c5a|c5b|c2_sizemap|dwconv|c3_norm|c3_layer]
                    [--shape N,Cin,Cout,T,H,W,kd,kh,kw,G,dtype[,groups]]

One step = one forward (+ one backward with all five gradients, except for
the forward-only workload c1) of the modulated deformable convolution through
the C ABI of libd2conv.so, inputs resident in HBM, outputs and workspace
pre-allocated.  Default workload: the headline configuration c3 (N=2,
Cin=Cout=512, 8x30x54, 3x3x3, pad 1, 8 offset groups, offsets ~N(0,2),
bfloat16 in / fp32 accumulate).

Prints ONE JSON line: whole-job effective TFLOP/s (GEMM-equivalent flops
2*N*P*Cout*(Cin/groups)*K forward, twice that backward), ms per step (and the
forward / backward split), a `roofline` object for the kernel that takes the
most time (its algorithmic flops or bytes over its average duration, measured
with HIP events on the launch stream inside the library) and a `cpu_baseline`
object (the CPU oracle, i.e. the reference's algorithm restated in C, timed
on the host cores on a bounded sample of the same workload).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# name: nd, N, Cin, Cout, spatial dims, weight groups, offset groups, dtype, offsets, seed, backward, roofline bound
#   offsets: ("normal", sigma) or ("dilation", lo, hi) = per-location, per-axis dilation map expanded to tap offsets
WORKLOADS = {
    "c1": dict(nd=3, N=1, C=64, dims=(8, 32, 32), groups=1, G=1, dt="f32", off=("normal", 1.0), seed=1001,
               backward=False, bound="mfma"),
    "c2_f32": dict(nd=3, N=2, C=256, dims=(8, 30, 54), groups=1, G=1, dt="f32", off=("dilation", 0.5, 4.0), seed=1002,
                   backward=True, bound="mfma"),
    "c2_bf16": dict(nd=3, N=2, C=256, dims=(8, 30, 54), groups=1, G=1, dt="bf16", off=("dilation", 0.5, 4.0),
                    seed=1002, backward=True, bound="mfma"),
    "c3": dict(nd=3, N=2, C=512, dims=(8, 30, 54), groups=1, G=8, dt="bf16", off=("normal", 2.0), seed=1003,
               backward=True, bound="mfma"),
    # the headline shape in float32 (the reference's default precision): weight groups of 512 output channels, two
    # passes of the float32 grad-column product
    "c3_f32": dict(nd=3, N=2, C=512, dims=(8, 30, 54), groups=1, G=8, dt="f32", off=("normal", 2.0), seed=1003,
                   backward=True, bound="mfma"),
    "c4": dict(nd=3, N=2, C=1024, dims=(8, 15, 27), groups=1024, G=1, dt="f32", off=("normal", 1.5), seed=1004,
               backward=True, bound="hbm"),
    "c5a": dict(nd=1, N=4, C=512, dims=(64,), groups=1, G=1, dt="f32", off=("normal", 1.5), seed=1005,
                backward=True, bound="hbm"),
    "c5b": dict(nd=3, N=1, C=256, dims=(32, 60, 108), groups=1, G=1, dt="bf16", off=("normal", 1.0), seed=1005,
                backward=True, bound="mfma"),
}
PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}
PEAK_GBS = 8000.0
# largest sample the CPU leg runs (the oracle does ~0.09 TFLOP/s on 16 cores): N and leading dim cut down to this
CPU_CROP = {"c3": (1, (8, 30, 54)), "c3_f32": (1, (8, 30, 54)), "c5b": (1, (8, 60, 108))}


def make_inputs(name, torch, crop=None, want_size=False):
    """Seeded synthetic tensors of the workload (generated on the CPU so that the CPU leg and the GPU see the
    same numbers).  `crop` = (N, dims) replaces the batch and spatial size for the CPU sample.  `want_size`
    appends the dilation map that the offsets were expanded from (None for workloads with free offsets)."""
    from d2conv3d_amd.grid import offsets_from_size_map
    c = WORKLOADS[name]
    N, dims = (c["N"], c["dims"]) if crop is None else crop
    C, nd, G, groups = c["C"], c["nd"], c["G"], c["groups"]
    g = torch.Generator().manual_seed(c["seed"])
    ks = (3,) * nd
    K = 3 ** nd
    x = torch.randn(N, C, *dims, generator=g)
    bound = 1.0 / (C // groups * K) ** 0.5
    w = (torch.rand(C, C // groups, *ks, generator=g) * 2 - 1) * bound
    b = (torch.rand(C, generator=g) * 2 - 1) * bound
    size = None
    if c["off"][0] == "dilation":
        _, lo, hi = c["off"]
        size = torch.rand(N, 3, *dims, generator=g) * (hi - lo) + lo
        off = offsets_from_size_map(size, "xyz", (3, 3, 3), (1, 1, 1))
    else:
        off = torch.randn(N, G * nd * K, *dims, generator=g) * c["off"][1]
    m = torch.sigmoid(torch.randn(N, G * K, *dims, generator=g))
    gout = torch.randn(N, C, *dims, generator=g)
    return (x, off, m, w, b, gout, size) if want_size else (x, off, m, w, b, gout)


def algorithmic(name, N=None, dims=None):
    """GEMM-equivalent flops (forward) and bytes with every tensor counted once (forward, backward)."""
    c = WORKLOADS[name]
    N = c["N"] if N is None else N
    dims = c["dims"] if dims is None else dims
    C, nd, G, groups = c["C"], c["nd"], c["G"], c["groups"]
    K = 3 ** nd
    P = 1
    for d in dims:
        P *= d
    es = 2 if c["dt"] == "bf16" else 4
    f_fwd = 2.0 * N * P * C * (C // groups) * K
    sz_x = N * C * P * es
    sz_off, sz_m = N * G * nd * K * P * es, N * G * K * P * es
    sz_w, sz_b = C * (C // groups) * K * es, C * es
    b_fwd = sz_x + sz_off + sz_m + sz_w + sz_b + sz_x
    b_bwd = 2 * (sz_x + sz_off + sz_m + sz_w) + sz_x + sz_b
    return f_fwd, b_fwd, b_bwd


def hbm_traffic_bytes(workload, kernel):
    """(HBM bytes per launch of `kernel`, where the figure comes from): read from the committed rocprofv3 --pmc
    summary of the workload (FETCH_SIZE + WRITE_SIZE, calibrated on a plain copy kernel), i.e. NOT measured in this
    run; (None, None) if not recorded."""
    import glob
    import subprocess
    stem = kernel[:-len("_kernel")] if kernel.endswith("_kernel") else kernel
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", f"{workload}_*.md"))):
        try:
            for row in open(path):
                cells = [c.strip().strip("`") for c in row.split("|")]
                # the traffic table: | kernel | fetch MB | write MB | total MB |
                if len(cells) == 6 and cells[1].startswith(stem):
                    rel = os.path.relpath(path, ROOT)
                    src = f"{rel} (committed rocprofv3 --pmc summary, not measured in this run)"
                    try:
                        h = subprocess.run(["git", "-C", ROOT, "log", "-1", "--format=%h", "--", rel],
                                           capture_output=True, text=True, timeout=10).stdout.strip()
                        if h:
                            src = f"{rel} @ {h} (committed rocprofv3 --pmc summary, not measured in this run)"
                    except (OSError, subprocess.SubprocessError):
                        pass
                    return int(float(cells[4]) * 1e6), src
        except (OSError, ValueError):
            pass
    return None, None


def cpu_baseline(name, torch):
    """The oracle (reference algorithm restated in C, OpenMP) on a bounded sample of the workload."""
    from oracle import cpu
    c = WORKLOADS[name]
    crop = CPU_CROP.get(name)
    x, off, m, w, b, gout = make_inputs(name, torch, crop)
    if c["dt"] == "bf16":
        x, w, b, gout, off, m = (t.bfloat16().float() for t in (x, w, b, gout, off, m))
    fwd, bwd = (cpu.conv3d_forward, cpu.conv3d_backward) if c["nd"] == 3 else (cpu.conv1d_forward, cpu.conv1d_backward)
    # one untimed warm-up iteration, then timed iterations until at least three are done and 5 s have passed (at
    # most 200); the figure is their median
    def once():
        fwd(x, off, m, w, b, 1, 1, 1, c["groups"], c["G"])
        if c["backward"]:
            bwd(gout, x, off, m, w, True, 1, 1, 1, c["groups"], c["G"])
    t_start = time.perf_counter()
    once()
    t_warm = time.perf_counter() - t_start
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < 5.0 and len(times) < 200):
        t0 = time.perf_counter()
        once()
        times.append(time.perf_counter() - t0)
    timed = sorted(times)
    per_iter, stat = timed[len(timed) // 2], "median"
    f_fwd, _, _ = algorithmic(name, x.shape[0], tuple(x.shape[2:]))
    flops = (3 if c["backward"] else 1) * f_fwd
    what = "full workload" if crop is None else f"same layer on N={crop[0]}, {'x'.join(map(str, crop[1]))} positions"
    return {
        "value": flops / per_iter / 1e12, "unit": "TFLOP/s", "cores": cpu.num_threads(), "kind": "port",
        "sample": f"{what}, fp32, {'forward+backward' if c['backward'] else 'forward'}: {stat} of {len(timed)} "
                  f"iterations after one warm-up = {per_iter * 1e3:.2f} ms ({sum(times) + t_warm:.2f} s of CPU work)",
    }


def bench_size_map(args):
    """The deformation producer in front of workload c2: predicted size map [2, 3, 8, 30, 54] -> ELU + 1 -> tap
    offsets [2, 81, 8, 30, 54] and back (d2c_size_map_offsets_forward / _backward), against the torch formulation
    of the reference (network/layers.py:171-181 + utils/grid.py:72-98) on the same GPU."""
    import torch
    from d2conv3d_amd.grid import offsets_from_size_map, size_map_offsets
    from d2conv3d_amd.modules import _apply_size_activation
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    g = torch.Generator().manual_seed(1002)
    raw = torch.randn(2, 3, 8, 30, 54, generator=g).to(dev).requires_grad_(True)
    gout = torch.randn(2, 81, 8, 30, 54, generator=g).to(dev)

    def fused():
        raw.grad = None
        size_map_offsets(raw, "xyz", (3, 3, 3), (1, 1, 1), "elu").backward(gout)

    def stock():
        raw.grad = None
        offsets_from_size_map(_apply_size_activation("elu", raw), "xyz", (3, 3, 3), (1, 1, 1)).backward(gout)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms, ms_torch = timed(fused), timed(stock)
    nbytes = 2 * (raw.numel() + gout.numel()) * 4          # each tensor once per direction
    gbs = nbytes / (ms * 1e-3) / 1e9
    line = {
        "metric": "size map -> offsets fwd+bwd GB/s (c2_sizemap) on 1 GPU", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c2_sizemap: size map [2,3,8,30,54] -> ELU+1 -> offsets [2,81,8,30,54], forward + "
                               "backward, through the autograd function (launch overhead included)",
                   "torch_formulation_ms_per_step": round(ms_torch, 4), "algorithmic_mbytes": round(nbytes / 1e6, 2)},
        "roofline": {"bound": "hbm", "kernel": "size_map_fwd_kernel + size_map_bwd_kernel", "achieved": round(gbs, 1),
                     "peak": PEAK_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_GBS, 4), "traffic": None},
    }
    print(json.dumps(line))


def bench_conv_act_norm(args):
    """The `_conv` block of the reference's refinement modules (network/modules/refinement.py:38-43) at the size of
    workload c3: Sequential(MDConv3d-style operator, ReLU, GroupNorm(32)), forward + backward, as the fused block
    of util.fuse_conv_act_norm (activation and per-channel sums in the convolution's forward kernel, GroupNorm in one
    pass from them) against the plain sequence (the same operator, then torch's relu and group_norm)."""
    import copy
    import torch
    import torch.nn as nn
    from d2conv3d_amd import util
    from d2conv3d_amd.deform_conv import DeformConv3d
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    x, off, m, w, b, gout = (t.to(dev, torch.bfloat16) for t in make_inputs("c3", torch))

    class Block(nn.Module):          # offsets / mask given (the deformation branch is not part of this measurement)
        def __init__(self):
            super().__init__()
            self.deform_conv = DeformConv3d(512, 512, 3, padding=1, offset_groups=8)
            self.norm = nn.GroupNorm(32, 512)
            self.fused = False

        def forward(self, x, off, m):
            dc = self.deform_conv
            if not self.fused:
                return self.norm(torch.relu(dc(x, off, m)))
            from d2conv3d_amd import _ops
            dc.output_relu_scale, dc.keep_output_stats = 1.0, True
            out = dc(x, off, m)
            return _ops.group_norm_from_stats(out, dc.last_output_stats, self.norm.weight, self.norm.bias, 32, self.norm.eps)

    net = Block().to(dev, torch.bfloat16)
    with torch.no_grad():
        net.deform_conv.weight.copy_(w)
        net.deform_conv.bias.copy_(b)
    xs = x.clone().requires_grad_(True)
    offs, ms = off.clone().requires_grad_(True), m.clone().requires_grad_(True)

    def step():
        net.zero_grad(set_to_none=True)
        xs.grad = offs.grad = ms.grad = None
        net(xs, offs, ms).backward(gout)

    def timed():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    net.fused = False
    ms_plain = timed()
    y_plain = net(xs, offs, ms).detach().float()
    net.fused = True
    ms_fused = timed()
    y_fused = net(xs, offs, ms).detach().float()
    err = float((y_fused - y_plain).norm() / y_plain.norm())
    f_fwd, _, _ = algorithmic("c3")
    value = 3 * f_fwd / (ms_fused * 1e-3) / 1e12
    line = {
        "metric": "mdconv3d + ReLU + GroupNorm block fwd+bwd effective TFLOP/s (c3_norm) on 1 GPU", "value": round(value, 3),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_fused, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "c3_norm: Sequential(modulated deformable conv3d of workload c3, ReLU, GroupNorm(32)) "
                               "forward + backward through the autograd functions (allocations included), fused block",
                   "plain_sequence_ms_per_step": round(ms_plain, 4), "relative_l2_fused_vs_plain": err},
        "roofline": None,
    }
    print(json.dumps(line))


def bench_layer(args):
    """A whole self-deforming layer at the size of workload c3: MDConv3d(512, 512, 3, padding=1, offset_groups=8) in
    bfloat16 -- the Conv3d that predicts the deformation (network/layers.py:51-60), then the operator --
    forward + backward through autograd.  Timed twice on the same GPU: with the deformation tensor handed to the
    operator as it is (the sampler reads offsets and modulation inside it and applies the sigmoid; the default), and
    with the reference's split + sigmoid in front of the operator (network/layers.py:107-120)."""
    import torch
    from d2conv3d_amd import modules
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    c = WORKLOADS["c3"]
    torch.manual_seed(c["seed"])
    layer = modules.MDConv3d(c["C"], c["C"], 3, padding=1, offset_groups=c["G"]).to(dev)
    with torch.no_grad():     # offsets ~ N(0, 2) like the operator workload: a branch that predicts something
        layer.deform_params.weight.normal_(0, 2.0 / (c["C"] * 27) ** 0.5)
    layer = layer.to(torch.bfloat16)
    g = torch.Generator().manual_seed(c["seed"])
    x = torch.randn(c["N"], c["C"], *c["dims"], generator=g).to(dev, torch.bfloat16).requires_grad_(True)
    gout = torch.randn(c["N"], c["C"], *c["dims"], generator=g).to(dev, torch.bfloat16)

    def step():
        layer.zero_grad(set_to_none=True)
        x.grad = None
        layer(x).backward(gout)

    def timed():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    res, outs = {}, {}
    for fused in (False, True):
        layer.fused_deformation = fused
        res[fused] = timed()
        outs[fused] = layer(x).detach().float()
    err = float((outs[True] - outs[False]).norm() / outs[False].norm())
    # ... and with the branch's convolution on the vendor library (what the reference runs) instead of on the operator
    # at zero offsets (modules._branch_conv, the default)
    layer.branch_on_operator = False
    stock_branch_ms = timed()
    stock_out = layer(x).detach().float()
    layer.branch_on_operator = True
    err_branch = float((outs[True] - stock_out).norm() / stock_out.norm())
    # the operator's GEMM-equivalent flops plus those of the deformation branch's convolution (864 output channels)
    f_op, _, _ = algorithmic("c3")
    P = c["dims"][0] * c["dims"][1] * c["dims"][2]
    f_branch = 2.0 * c["N"] * P * (4 * c["G"] * 27) * c["C"] * 27
    value = 3 * (f_op + f_branch) / (res[True] * 1e-3) / 1e12
    line = {
        "metric": "MDConv3d layer fwd+bwd effective TFLOP/s (c3_layer) on 1 GPU", "value": round(value, 3),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(res[True], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "c3_layer: MDConv3d(512, 512, 3, padding=1, offset_groups=8) on [2, 512, 8, 30, 54], bf16, "
                               "forward + backward through autograd (allocations included), the deformation branch's "
                               "stock Conv3d (512 -> 864 channels) included",
                   "deformation": "read by the operator inside the branch's output tensor, sigmoid in the sampler",
                   "split_and_sigmoid_in_front_ms_per_step": round(res[False], 4),
                   "relative_l2_fused_vs_split": err,
                   "branch": "the layer's Conv3d 512 -> 864 evaluated by the operator at zero offsets",
                   "branch_on_the_vendor_library_ms_per_step": round(stock_branch_ms, 4),
                   "relative_l2_branch_on_operator_vs_vendor": err_branch,
                   "algorithmic_gflop": round(3 * (f_op + f_branch) / 1e9, 2)},
        "roofline": None,
    }
    print(json.dumps(line))


def bench_shape(args):
    """`--shape N,Cin,Cout,T,H,W,kd,kh,kw,G,dtype[,groups]`: modulated deformable conv3d of any size (stride 1,
    "same" padding, offsets ~N(0,1.5), sigmoid mask, bias) through d2conv3d_amd.deform_conv3d, forward and backward timed
    apart with HIP events.  For the layer shapes of the reference's own networks, e.g. the refinement blocks of
    network/segmentation/encoder_decoder.py:112-131 (`--shape 1,1024,256,8,30,54,3,3,3,1,bf16`) or its global-convolution
    bridge (network/modules/bridging.py:14-22: `--shape 1,2048,256,8,30,54,1,7,1,1,bf16`)."""
    import torch
    import d2conv3d_amd as d2c
    from d2conv3d_amd import _ops
    f = args.shape.split(",")
    N, Cin, Cout, T, H, W, kd, kh, kw, G = (int(v) for v in f[:10])
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32}[f[10]]
    groups = int(f[11]) if len(f) > 11 else 1
    dev = torch.device("cuda:0")
    dims, ks, pad, K = (T, H, W), (kd, kh, kw), (kd // 2, kh // 2, kw // 2), kd * kh * kw
    g = torch.Generator().manual_seed(4242)
    bound = 1.0 / (Cin // groups * K) ** 0.5
    x = torch.randn(N, Cin, *dims, generator=g).to(dtype).to(dev).requires_grad_(True)
    w = ((torch.rand(Cout, Cin // groups, *ks, generator=g) * 2 - 1) * bound).to(dtype).to(dev).requires_grad_(True)
    b = ((torch.rand(Cout, generator=g) * 2 - 1) * bound).to(dtype).to(dev).requires_grad_(True)
    off = (torch.randn(N, 3 * K * G, *dims, generator=g) * 1.5).to(dev).requires_grad_(True)
    m = torch.sigmoid(torch.randn(N, K * G, *dims, generator=g)).to(dev).requires_grad_(True)
    gout = torch.randn(N, Cout, *dims, generator=g).to(dtype).to(dev)
    algo = _ops.conv3d_algo(x, off, m, w, (1, 1, 1), pad, (1, 1, 1), groups, G)
    if algo == "generic" and dtype == torch.bfloat16 and \
            _ops.conv3d_algo(x, off, m, w, (1, 1, 1), pad, (1, 1, 1), groups, G, as_dtype=torch.float32) == "mfma":
        algo = "mfma, in float32 and rounded (channel counts the bfloat16 kernels cannot chunk)"
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    t_f = t_b = 0.0
    for it in range(args.warmup + args.steps):
        for t in (x, w, b, off, m):
            t.grad = None
        ev[0].record()
        out = d2c.deform_conv3d(x, off, m, w, b, 1, pad, 1, groups, G)
        ev[1].record()
        out.backward(gout)
        ev[2].record()
        torch.cuda.synchronize()
        if it >= args.warmup:
            t_f += ev[0].elapsed_time(ev[1]) / args.steps
            t_b += ev[1].elapsed_time(ev[2]) / args.steps
    flop = 2.0 * N * T * H * W * Cout * (Cin // groups) * K
    print(json.dumps({
        "metric": "modulated deformable conv3d fwd+bwd effective TFLOP/s (--shape) on 1 GPU",
        "value": round(3 * flop / ((t_f + t_b) * 1e-3) / 1e12, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(t_f + t_b, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": f[10], "data": "synthetic",
        "config": {"workload": f"--shape {args.shape}: N={N}, {Cin}->{Cout} channels, {T}x{H}x{W}, kernel {kd}x{kh}x{kw}, "
                               f"{G} offset group(s), {groups} weight group(s), through d2conv3d_amd.deform_conv3d",
                   "kernel_family": algo, "forward_ms": round(t_f, 4), "backward_ms": round(t_b, 4),
                   "forward_tflops": round(flop / (t_f * 1e-3) / 1e12, 1),
                   "backward_tflops": round(2 * flop / (t_b * 1e-3) / 1e12, 1)}}))


def bench_dwconv(args):
    """Plain depthwise conv3d (the reference's fast-depthwise-conv3d operator; backbone shape: 256 channels,
    8x56x56, 3x3x3, stride 1, padding 1, float32), forward + backward through the C ABI with pre-allocated
    buffers; torch's own grouped convolution (MIOpen) is timed beside it on the same GPU."""
    import ctypes
    import numpy as np
    import torch
    import torch.nn.functional as F
    from d2conv3d_amd import _lib
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.load()
    N, C, dims = 2, 256, (8, 56, 56)
    g = torch.Generator().manual_seed(1006)
    x = torch.randn(N, C, *dims, generator=g)
    w = (torch.rand(C, 1, 3, 3, 3, generator=g) * 2 - 1) / 27 ** 0.5
    b = (torch.rand(C, generator=g) * 2 - 1) / 27 ** 0.5
    gout = torch.randn(N, C, *dims, generator=g)
    xd, wd, bd, gd = (t.to(dev) for t in (x, w, b, gout))
    desc = _lib.DwConv3dDesc(N, C, C, *dims, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, *dims, _lib.D2C_F32)
    _lib.check(lib.d2c_dwconv3d_check(ctypes.byref(desc)), "check")
    out, gx, gw, gb = torch.empty_like(xd), torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(bd)
    nws = lib.d2c_dwconv3d_backward_workspace_bytes(ctypes.byref(desc))
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device=dev)
    st = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def forward():
        _lib.check(lib.d2c_dwconv3d_forward(ctypes.byref(desc), p(xd), p(wd), p(bd), p(out), st), "forward")

    def backward():
        _lib.check(lib.d2c_dwconv3d_backward(ctypes.byref(desc), p(gd), p(xd), p(wd), p(gx), p(gw), p(gb), p(ws), nws, st),
                   "backward")

    def step():
        forward()
        backward()

    xt, wt, bt = (t.clone().requires_grad_(True) for t in (xd, wd, bd))

    def stock():
        xt.grad = wt.grad = bt.grad = None
        F.conv3d(xt, wt, bt, 1, 1, 1, groups=C).backward(gd)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms, ms_f, ms_b, ms_torch = timed(step), timed(forward), timed(backward), timed(stock)
    # parity of what was just timed, against torch's result on the same tensors (the reference's own check)
    stock()
    err = max(float((out - F.conv3d(xd, wd, bd, 1, 1, 1, groups=C)).abs().max()), float((gx - xt.grad).abs().max()),
              float((gw - wt.grad).abs().max() / wt.grad.abs().max()), float((gb - bt.grad).abs().max() / bt.grad.abs().max()))
    n_el = x.numel()
    nbytes = 4 * (2 * n_el + 3 * n_el + 3 * w.numel() + 2 * b.numel())   # fwd: x, out; bwd: gout, x, gx; w, gw, b, gb
    gbs = nbytes / (ms * 1e-3) / 1e9
    line = {
        "metric": "plain depthwise conv3d fwd+bwd GB/s (dwconv) on 1 GPU", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "dwconv: depthwise conv3d fwd+bwd, N=2, C=256, 8x56x56, k3 s1 p1, bias, fp32",
                   "forward_ms": round(ms_f, 4), "backward_ms": round(ms_b, 4),
                   "torch_grouped_conv_ms_per_step": round(ms_torch, 4), "max_error_vs_torch": err,
                   "algorithmic_mbytes": round(nbytes / 1e6, 1)},
        "roofline": {"bound": "hbm", "kernel": "dwc_fwd_kernel + dwc_bwd_input_kernel + dwc_bwd_weight_kernel",
                     "achieved": round(gbs, 1), "peak": PEAK_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_GBS, 4),
                     "traffic": None},
    }
    if not args.no_cpu:
        from oracle import dwconv
        cx, cw, cb, cg = x[:1, :32].numpy(), w[:32].numpy(), b[:32].numpy(), gout[:1, :32].numpy()
        t0 = time.perf_counter()
        dwconv.forward(cx, cw, cb, (1, 1, 1), (1, 1, 1), (1, 1, 1))
        dwconv.backward(cg, cx, cw, (1, 1, 1), (1, 1, 1), (1, 1, 1))
        dt = time.perf_counter() - t0
        line["cpu_baseline"] = {"value": round(nbytes / 16 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                                "sample": f"1 of 2 samples, 32 of 256 channels (1/16 of the workload), numpy float64: {dt:.2f} s"}
    print(json.dumps(line))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + ["c2_sizemap", "dwconv", "c3_norm", "c3_layer"])
    ap.add_argument("--shape", default=None,
                    help="instead of a named workload: N,Cin,Cout,T,H,W,kd,kh,kw,G,dtype[,groups] (dtype bf16 | f32), "
                         "timed through the Python layer (see bench_shape)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--offset-axes", type=int, default=7,
                    help="mask of the axes the offsets displace along (1 z, 2 y, 4 x): 6 = the Spatial layers, 1 = the "
                         "Temporal layers of the reference (3-D matrix-core workloads only; default all three)")
    ap.add_argument("--grad-weight-mode", type=int, default=1, choices=[0, 1, 2],
                    help="matrix-core backward of bfloat16 problems: 1 (default) grad_weight as a matrix product over "
                         "the sampled columns that the offset / mask gradient kernel writes; 2 the same with the columns "
                         "written over the grad-column rows (no buffer of their own); 0 the grad-weight kernel "
                         "samples the input again")
    ap.add_argument("--backward-slices", type=int, default=0,
                    help="matrix-core backward of bfloat16 problems with several offset groups: number of slices over "
                         "the offset groups (0 or 1: one pass over all groups; the description's backward_flags)")
    ap.add_argument("--grad-input-mode", type=int, default=1, choices=[0, 1],
                    help="matrix-core backward: 1 (default) grad-column rows through device memory, offset / mask "
                         "gradient and grad_input (from sample lists) as kernels of their own; 0 everything inside "
                         "the grad-column kernel, grad_input scattered with atomics (the reference's formulation; for "
                         "comparison)")
    ap.add_argument("--prepared", choices=["off", "train", "infer"], default="off",
                    help="3-D matrix-core workloads: keep a prepared region (d2c_conv3d_*_prepared) the way a layer would: "
                         "'train' = the backward call reuses the input copy its forward call made (weights change every "
                         "step); 'infer' = forward calls also reuse the re-ordered weights")
    ap.add_argument("--columns", choices=["on", "off"], default="on",
                    help="keep the forward call's sampled columns for the backward call of the step where the "
                         "description is served (d2c_conv3d_forward_columns / _backward_columns; the Python layer's "
                         "default), or let the backward pass sample again")
    ap.add_argument("--f32-split-backward", action="store_true",
                    help="float32 matrix-core workloads: the backward matrix kernels on two-term bfloat16 operands too "
                         "(D2C_BWD_F32_SPLIT; gradients with ~4e-6 relative error of their scale)")
    ap.add_argument("--expanded-offsets", action="store_true",
                    help="dynamic-dilation workloads (c2_*): expand the dilation map to an offsets tensor first "
                         "and time the ordinary operator on it, instead of handing the map to the operator")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this operator path is measured on ONE GPU only (--gpus 1); "
                 "no multi-GPU run exists or is meaningful for it")

    import torch
    from d2conv3d_amd import _lib
    lib = _lib.load()  # raises if the HIP library is missing: there is no fallback
    lib.d2c_set_grad_input_mode(args.grad_input_mode)
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    if args.shape:
        return bench_shape(args)
    if args.workload == "c2_sizemap":
        return bench_size_map(args)
    if args.workload == "dwconv":
        return bench_dwconv(args)
    if args.workload == "c3_norm":
        return bench_conv_act_norm(args)
    if args.workload == "c3_layer":
        return bench_layer(args)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    name = args.workload
    c = WORKLOADS[name]
    N, C, dims, G, groups, dt, nd = c["N"], c["C"], c["dims"], c["G"], c["groups"], c["dt"], c["nd"]
    x, off, m, w, b, gout, size = make_inputs(name, torch, want_size=True)
    tdt = torch.bfloat16 if dt == "bf16" else torch.float32
    x, w, b, gout, off, m = (t.to(dev, tdt).contiguous() for t in (x, w, b, gout, off, m))
    code = _lib.D2C_BF16 if dt == "bf16" else _lib.D2C_F32
    # Dynamic-dilation workloads hand the dilation map itself to the operator (d2c_conv3d_sized_*: the sampler
    # forms the tap offsets, no [N, 81, ...] tensor exists) unless --expanded-offsets asks for the two-step form.
    sized = size is not None and not args.expanded_offsets
    if sized:
        from d2conv3d_amd.grid import size_map_desc
        size = size.to(dev, tdt).contiguous()
        sdesc = size_map_desc(size, "xyz", (3, 3, 3), (1, 1, 1), "linear")
        gsize = torch.empty_like(size)
    if nd == 3:
        T_, H_, W_ = dims
        desc = _lib.Conv3dDesc(N, C, C, T_, H_, W_, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, groups, G, T_, H_, W_,
                               code, code, 0, 1.0, args.offset_axes,
                               {1: _lib.BWD_GW_COLUMNS, 2: _lib.BWD_GW_IN_PLACE, 0: _lib.BWD_GW_RESAMPLE}[args.grad_weight_mode]
                               | _lib.bwd_slices(args.backward_slices)
                               | (_lib.BWD_F32_SPLIT if args.f32_split_backward else 0))
        kind = "conv3d"
        algo = _lib.ALGO_NAMES[lib.d2c_conv3d_algo(ctypes.byref(desc))]
    else:
        desc = _lib.Conv1dDesc(N, C, C, dims[0], 3, 1, 1, 1, groups, G, dims[0], code, code, 1)
        kind = "conv1d"
        algo = _lib.ALGO_NAMES[lib.d2c_conv1d_algo(ctypes.byref(desc))]
    f_check = getattr(lib, f"d2c_{kind}_check")
    f_fwd_ws, f_bwd_ws = (getattr(lib, f"d2c_{kind}_{d}_workspace_bytes") for d in ("forward", "backward"))
    f_fwd, f_bwd = getattr(lib, f"d2c_{kind}_forward"), getattr(lib, f"d2c_{kind}_backward")
    _lib.check(f_check(ctypes.byref(desc)), "check")
    out = torch.empty(N, C, *dims, device=dev, dtype=tdt)
    gx, goff, gm, gw, gb = (torch.empty_like(t) for t in (x, off, m, w, b))
    nf = f_fwd_ws(ctypes.byref(desc))
    nb = f_bwd_ws(ctypes.byref(desc)) if c["backward"] else 0
    ws = torch.empty(max(nf, nb, 256), dtype=torch.uint8, device=dev)
    cur = [ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)]   # the stream the library launches on
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    if sized:
        nf = lib.d2c_conv3d_sized_forward_workspace_bytes(ctypes.byref(desc), ctypes.byref(sdesc))
        nb = lib.d2c_conv3d_sized_backward_workspace_bytes(ctypes.byref(desc), ctypes.byref(sdesc))
        ws = torch.empty(max(nf, nb, 256), dtype=torch.uint8, device=dev)

    # The sampled columns of the forward call, kept for the backward call of the step (what the Python layer does by
    # default where the description is served): d2c_conv3d_forward_columns / _backward_columns.
    kept_cols = None
    if args.columns == "on" and nd == 3 and c["backward"] and args.prepared == "off" and args.grad_weight_mode == 1 \
            and not args.backward_slices:
        zdesc = ctypes.byref(sdesc) if sized else None
        ncol = lib.d2c_conv3d_columns_bytes(ctypes.byref(desc), zdesc)
        if ncol:
            kept_cols = torch.empty(ncol, dtype=torch.uint8, device=dev)
            nb = lib.d2c_conv3d_backward_columns_workspace_bytes(ctypes.byref(desc), zdesc)

    prep = None
    if args.prepared != "off" and nd == 3 and not sized:
        npre = lib.d2c_conv3d_prepared_bytes(ctypes.byref(desc))
        if npre:
            prep = torch.empty(npre, dtype=torch.uint8, device=dev)
    fwd_reuse = [0]

    def forward():
        if kept_cols is not None:
            _lib.check(lib.d2c_conv3d_forward_columns(ctypes.byref(desc), zdesc, p(x), p(size if sized else off), p(m), p(w),
                                                      p(b), p(out), p(kept_cols), kept_cols.numel(), p(ws), nf, cur[0]), "forward")
            return
        if prep is not None:
            _lib.check(lib.d2c_conv3d_forward_prepared(ctypes.byref(desc), p(x), p(off), p(m), p(w), p(b), p(out), p(prep),
                                                       prep.numel(), fwd_reuse[0], p(ws), nf, cur[0]), "forward")
            if args.prepared == "infer":
                fwd_reuse[0] = _lib.REUSE_FORWARD_WEIGHTS
            return
        if sized:
            _lib.check(lib.d2c_conv3d_sized_forward(ctypes.byref(desc), ctypes.byref(sdesc), p(x), p(size), p(m), p(w),
                                                    p(b), p(out), p(ws), nf, cur[0]), "forward")
            return
        _lib.check(f_fwd(ctypes.byref(desc), p(x), p(off), p(m), p(w), p(b), p(out), p(ws), nf, cur[0]), "forward")

    def backward():
        if kept_cols is not None:
            _lib.check(lib.d2c_conv3d_backward_columns(ctypes.byref(desc), zdesc, p(gout), p(x), p(size if sized else off),
                                                       p(m), p(w), p(kept_cols), kept_cols.numel(), p(gx),
                                                       p(gsize if sized else goff), p(gm), p(gw), p(gb), p(ws), nb,
                                                       cur[0]), "backward")
            return
        if prep is not None:
            _lib.check(lib.d2c_conv3d_backward_prepared(ctypes.byref(desc), p(gout), p(x), p(off), p(m), p(w), p(gx), p(goff),
                                                        p(gm), p(gw), p(gb), p(prep), prep.numel(), _lib.REUSE_INPUT, p(ws),
                                                        nb, cur[0]), "backward")
            return
        if sized:
            _lib.check(lib.d2c_conv3d_sized_backward(ctypes.byref(desc), ctypes.byref(sdesc), p(gout), p(x), p(size),
                                                     p(m), p(w), p(gx), p(gsize), p(gm), p(gw), p(gb), p(ws), nb,
                                                     cur[0]), "backward")
            return
        _lib.check(f_bwd(ctypes.byref(desc), p(gout), p(x), p(off), p(m), p(w), p(gx), p(goff), p(gm), p(gw), p(gb),
                         p(ws), nb, cur[0]), "backward")

    def step():
        forward()
        if c["backward"]:
            backward()

    taps = None
    if nd == 3:
        # how much of the offset field leaves the volume (outside the timed region)
        from d2conv3d_amd.util import tap_statistics
        st = tap_statistics((N, C, *dims), off, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), G)
        taps = {k: round(st[k], 4) for k in ("dead", "partial", "corners_read")}

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # The same step captured once into a HIP graph and replayed (the library only enqueues kernels: no allocation,
    # no memset node, no synchronisation).  Informational: what a launch-bound caller gains; `value` stays eager.
    graph_ms = None
    try:
        graph = torch.cuda.CUDAGraph()
        default_stream = cur[0]
        with torch.cuda.graph(graph):
            cur[0] = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            step()
        cur[0] = default_stream
        for _ in range(2):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    except Exception as e:  # noqa: BLE001  (reported, never fatal: the eager figures above stand)
        cur[0] = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        sys.stderr.write(f"bench.py: graph replay not measured: {e}\n")

    f_fwd_flops, b_fwd, b_bwd = algorithmic(name)
    nflops = (3 if c["backward"] else 1) * f_fwd_flops
    value = nflops / (ms * 1e-3) / 1e12

    # forward and backward separately (events on the launch stream), then per-kernel durations recorded by
    # the library with HIP events around each launch
    nprof = max(3, min(args.steps, 10))
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    t_f = t_b = 0.0
    for _ in range(nprof):
        ev[0].record()
        forward()
        ev[1].record()
        if c["backward"]:
            backward()
        ev[2].record()
        torch.cuda.synchronize()
        t_f += ev[0].elapsed_time(ev[1]) / nprof
        t_b += ev[1].elapsed_time(ev[2]) / nprof
    # With the columns kept, the forward kernel also writes them (work of the backward pass moved into it): its
    # duration in a plain forward call is measured as well, so that its GEMM rate can be read both ways.
    plain_fwd_ms = None
    if kept_cols is not None:
        lib.d2c_profile_reset()
        lib.d2c_profile_enable(1)
        for _ in range(nprof):
            if sized:
                _lib.check(lib.d2c_conv3d_sized_forward(ctypes.byref(desc), ctypes.byref(sdesc), p(x), p(size), p(m), p(w),
                                                        p(b), p(out), p(ws), nf, cur[0]), "forward")
            else:
                _lib.check(f_fwd(ctypes.byref(desc), p(x), p(off), p(m), p(w), p(b), p(out), p(ws), nf, cur[0]), "forward")
        torch.cuda.synchronize()
        lib.d2c_profile_enable(0)
        tot, cnt = ctypes.c_double(0), ctypes.c_int(0)
        lib.d2c_profile_read(_lib.PROF_FWD, ctypes.byref(tot), ctypes.byref(cnt))
        if cnt.value:
            plain_fwd_ms = tot.value / nprof
    lib.d2c_profile_reset()
    lib.d2c_profile_enable(1)
    for _ in range(nprof):
        step()
    torch.cuda.synchronize()
    lib.d2c_profile_enable(0)
    fam = {"mfma": "tiled", "depthwise": "dw", "generic": "generic"}[algo]
    # per-kernel time under the name a profiler trace shows (the library reports which kernel it launched)
    ids = {_lib.PROF_FWD: "fwd", _lib.PROF_BWD_DATA: "bwd_data", _lib.PROF_BWD_WEIGHT: "bwd_weight",
           _lib.PROF_GX_OWNER: "gx_owner", _lib.PROF_BWD_AUX: "bwd_aux", _lib.PROF_PACK: "pack"}
    kern, role = {}, {}
    for kid, r in ids.items():
        tot, cnt = ctypes.c_double(0), ctypes.c_int(0)
        lib.d2c_profile_read(kid, ctypes.byref(tot), ctypes.byref(cnt))
        if cnt.value:
            kname = "pack/clear/convert/lists" if r == "pack" else (lib.d2c_profile_kernel_name(kid).decode() or r)
            kern[kname] = tot.value / nprof  # ms per step spent in this kernel (all launches of it)
            role[kname] = r

    es = 2 if dt == "bf16" else 4
    P = 1
    for d in dims:
        P *= d
    K = 3 ** nd
    kms = {k: round(v, 4) for k, v in kern.items()}
    roofline = None
    gemm_k = {k: v for k, v in kern.items() if role[k] in ("fwd", "bwd_data", "bwd_weight")}
    main_k = {k: v for k, v in kern.items() if role[k] != "pack"}
    if c["bound"] == "mfma" and gemm_k:
        # the longest kernel that carries one of the three GEMMs (2*N*P*Cout*(Cin/groups)*K flop each)
        dom = max(gemm_k, key=gemm_k.get)
        ach = f_fwd_flops / (gemm_k[dom] * 1e-3) / 1e12
        traffic, traffic_source = hbm_traffic_bytes(name, dom)
        roofline = {"bound": "mfma", "kernel": dom, "achieved": round(ach, 2), "peak": PEAK_TFLOPS[dt],
                    "unit": "TFLOP/s", "frac": round(ach / PEAK_TFLOPS[dt], 4), "traffic": traffic,
                    "traffic_source": traffic_source, "algorithmic_gflop_per_launch": round(f_fwd_flops / 1e9, 2),
                    "whole_step_frac": round(value / PEAK_TFLOPS[dt], 4), "kernel_ms": kms}
        # float32 workloads: most matrix kernels run on the bfloat16 instruction with every float operand taken apart
        # into two or three bfloat16 terms, so `frac` (against the float32 instruction's peak) can pass 1; the
        # instructions executed are the partial products
        if dt == "f32":
            terms = {"tiled_fwd_dma_kernel": 4, "tiled_fwd_kernel": 4, "tiled_bwd_weight_col3_kernel": 6,
                     "tiled_bwd_col_kernel": 4, "tiled_bwd_col32f_kernel": 3}
            if args.f32_split_backward:
                terms.update({"tiled_bwd_weight_dma_kernel": 4, "tiled_bwd_data_kernel": 4})
            if dom in terms:
                ex = terms[dom] * ach
                roofline["on_bf16_instructions"] = {
                    "partial_products_per_product": terms[dom], "executed_tflops": round(ex, 1),
                    "frac_of_bf16_peak": round(ex / PEAK_TFLOPS["bf16"], 4),
                    "note": "float operands as sums of bfloat16 terms on v_mfma_f32_32x32x16_bf16; `peak` above is "
                            "the float32 instruction's"}
        if plain_fwd_ms and role[dom] == "fwd":
            ach0 = f_fwd_flops / (plain_fwd_ms * 1e-3) / 1e12
            roofline["note"] = ("this launch also writes the sampled columns that the backward call of the step "
                                "multiplies over (config.columns_kept_for_backward_mbytes); `in_a_plain_forward_call` "
                                "is the same kernel without that store")
            roofline["in_a_plain_forward_call"] = {"kernel_ms": round(plain_fwd_ms, 4), "achieved": round(ach0, 2),
                                                   "frac": round(ach0 / PEAK_TFLOPS[dt], 4)}
    elif main_k:
        # bandwidth-bound workloads: the longest kernel against every tensor of its direction once
        dom = max(main_k, key=main_k.get)
        nbytes = b_fwd if role[dom] == "fwd" else b_bwd
        ach = nbytes / (main_k[dom] * 1e-3) / 1e9
        traffic, traffic_source = hbm_traffic_bytes(name, dom)
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(ach, 2), "peak": PEAK_GBS, "unit": "GB/s",
                    "frac": round(ach / PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                    "algorithmic_mbytes_per_launch": round(nbytes / 1e6, 1),
                    "whole_step_frac": round((b_fwd + (b_bwd if c["backward"] else 0)) / (ms * 1e-3) / 1e9 / PEAK_GBS, 4),
                    "kernel_ms": kms}

    # The gather kernels of the matrix-core backward carry no GEMM; what they move is mostly the library's own
    # intermediates (grad-column rows, sampled columns, sample lists), i.e. internal traffic, not tensors of the
    # operator: reported apart from `roofline`, never as a fraction of a peak over algorithmic bytes.
    internal = None
    if fam == "tiled":
        rows = N * P * K * C * es
        per = {}
        for kname, r in role.items():
            if r == "bwd_aux":
                # (the sampled columns it writes -- unless the forward call kept them)
                cols = rows if (dt == "bf16" and nd == 3 and args.grad_weight_mode >= 1 and (C // groups) % 128 == 0
                                and kept_cols is None) else 0
                aux = N * P * K * G * (nd + 1) * es
                per[kname] = rows + cols + N * P * C * es + 2 * aux + N * P * K * G * (16 if dt == "bf16" else 32)
            elif r == "gx_owner":
                per[kname] = rows + N * P * K * G * (16 if dt == "bf16" else 32) + N * C * P * 4
        if per:
            internal = {"note": "internal traffic: grad-column rows, sampled columns and sample lists of the library "
                                "plus the operator's tensors these kernels touch, each counted once",
                        "kernels": {k: {"ms": round(kern[k], 4), "internal_mbytes": round(v / 1e6, 1),
                                        "gbytes_per_s": round(v / (kern[k] * 1e-3) / 1e9, 1)} for k, v in per.items()}}

    # Depthwise kernels: the corner rows they pull through the vector-memory path of the compute units (L1), which
    # is what bounds them (64 bytes per clock and compute unit; 256 units at 2.4 GHz), beside the HBM figure above.
    roofline_l1 = None
    if fam == "dw" and nd == 3:
        peak_l1 = 64 * 256 * 2.4  # GB/s
        npos, esz = dims[0] * dims[1] * dims[2], (2 if dt == "bf16" else 4)
        rows = N * npos * 27 * 8 * C * esz          # 8 corner values per tap and channel
        # (the backward kernel stages the grad_out rows of a tile in LDS once for all its taps: they pass through the
        #  vector-memory path once, not once per tap)
        per = {"dw_fwd_kernel": rows, "dw_bwd_kernel": rows + N * npos * C * esz,
               "dw_gx_owner_kernel": N * npos * 27 * (32 + C * esz) + N * npos * C * 4}  # list entry + grad_out row per sample, grad_input once
        roofline_l1 = {"bound": "l1", "peak": round(peak_l1, 1), "unit": "GB/s",
                       "peak_source": "64 B/clk/CU x 256 CUs x 2.4 GHz (vector-memory path)", "kernels": {}}
        for kname, nbytes in per.items():
            if kname in kern:
                gbs = nbytes / (kern[kname] * 1e-3) / 1e9
                roofline_l1["kernels"][kname] = {"bytes": nbytes, "ms": round(kern[kname], 4),
                                                 "achieved": round(gbs, 1), "frac": round(gbs / peak_l1, 4)}

    what = "modulated deformable conv%dd %s" % (nd, "fwd+bwd" if c["backward"] else "fwd")
    line = {
        "metric": "mdconv3d fwd+bwd effective TFLOP/s (C=512, 8x30x54, k3) on 1 GPU" if name == "c3"
                  else f"{what} effective TFLOP/s ({name}) on 1 GPU",
        "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{name}: {what}, N={N}, Cin=Cout={C}, {'x'.join(map(str, dims))}, k3 p1, "
                               f"groups={groups}, offset_groups={G}, bias, "
                               + ("bf16 in / fp32 accumulate" if dt == "bf16" else "fp32"),
                   "offsets": ("formed in the sampler from the dilation map [N,3,T,H,W] (d2c_conv3d_sized_*)" if sized
                               else "offsets tensor [N,3*K*G,T,H,W]"),
                   "offset_axes": args.offset_axes,
                   "grad_input_mode": args.grad_input_mode, "grad_weight_mode": args.grad_weight_mode,
                   "backward_slices": args.backward_slices, "prepared_region": args.prepared if prep is not None else "off",
                   "columns_kept_for_backward_mbytes": round(kept_cols.numel() / 1e6, 1) if kept_cols is not None else 0,
                   "f32_split_backward": bool(args.f32_split_backward),
                   "kernel_family": algo, "forward_ms": round(t_f, 4), "backward_ms": round(t_b, 4),
                   "graph_replay_ms_per_step": round(graph_ms, 4) if graph_ms is not None else None,
                   "taps_outside_volume": taps,
                   "algorithmic_gflop": round(nflops / 1e9, 2),
                   "algorithmic_mbytes": round((b_fwd + (b_bwd if c["backward"] else 0)) / 1e6, 1),
                   "backward_workspace_mbytes": round(nb / 1e6, 1), "forward_workspace_mbytes": round(nf / 1e6, 1),
                   "frac_of_mfma_peak_whole_step": round(value / PEAK_TFLOPS[dt], 4),
                   "frac_of_hbm_peak_whole_step": round((b_fwd + (b_bwd if c["backward"] else 0))
                                                        / (ms * 1e-3) / 1e9 / PEAK_GBS, 4)},
        "roofline": roofline,
    }
    if roofline_l1:
        line["roofline_l1"] = roofline_l1
    if internal:
        line["gather_kernels"] = internal
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(name, torch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
