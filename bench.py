#!/usr/bin/env python3
"""Benchmark of the D2Conv3D operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2_bf16|c2_f32|c5b]

One step = one forward + one backward (all five gradients) of the modulated
deformable conv3d through the C ABI of libd2conv.so, inputs resident in HBM,
outputs and workspace pre-allocated.  Default workload: the headline
configuration (N=2, Cin=Cout=512, 8x30x54, 3x3x3, pad 1, 8 offset groups,
offsets ~N(0,2), bfloat16 in / fp32 accumulate).

Prints ONE JSON line: whole-job effective TFLOP/s (GEMM-equivalent flops
2*N*P*Cout*Cin*K forward, twice that backward), ms per step, a `roofline`
object for the kernel that takes the most time (its own flops over its average
duration, measured with HIP events on the launch stream, against the 2.5
PFLOP/s dense bf16 MFMA peak) and a `cpu_baseline` object (the CPU oracle,
i.e. the reference's algorithm restated in C, timed on the host cores on a
cropped sample of the same workload).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (N, C, (T,H,W), offset groups, dtype, offset sigma, seed)
    "c3": (2, 512, (8, 30, 54), 8, "bf16", 2.0, 1003),
    "c2_bf16": (2, 256, (8, 30, 54), 1, "bf16", None, 1002),
    "c2_f32": (2, 256, (8, 30, 54), 1, "f32", None, 1002),
    "c5b": (1, 256, (32, 60, 108), 1, "bf16", 1.0, 1005),
}
PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}


def make_inputs(name, torch, crop=None):
    """Seeded synthetic tensors of the workload (generated on the CPU).  `crop`
    replaces (T,H,W) for the CPU sample."""
    from d2conv3d_amd.grid import offsets_from_size_map
    N, C, dims, G, dt, sig, seed = WORKLOADS[name]
    if crop is not None:
        N, dims = 1, crop
    g = torch.Generator().manual_seed(seed)
    K = 27
    x = torch.randn(N, C, *dims, generator=g)
    bound = 1.0 / (C * K) ** 0.5
    w = (torch.rand(C, C, 3, 3, 3, generator=g) * 2 - 1) * bound
    b = (torch.rand(C, generator=g) * 2 - 1) * bound
    if sig is None:  # dynamic dilation: per-location, per-axis dilation ~U(0.5, 4) expanded to tap offsets
        size = torch.rand(N, 3, *dims, generator=g) * 3.5 + 0.5
        off = offsets_from_size_map(size, "xyz", (3, 3, 3), (1, 1, 1))
    else:
        off = torch.randn(N, G * 3 * K, *dims, generator=g) * sig
    m = torch.sigmoid(torch.randn(N, G * K, *dims, generator=g))
    gout = torch.randn(N, C, *dims, generator=g)
    return x, off, m, w, b, gout, G


def hbm_traffic_bytes(kernel):
    """HBM bytes per launch of `kernel` on the headline workload, from the committed rocprofv3 --pmc
    summary (FETCH_SIZE + WRITE_SIZE, calibrated on a plain copy kernel); None if not recorded."""
    path = os.path.join(ROOT, "profiles", "c3_hbm_traffic.md")
    try:
        for row in open(path):
            cells = [c.strip().strip("`") for c in row.split("|")]
            if len(cells) > 4 and cells[1].startswith(kernel):
                return int(float(cells[4]) * 1e6)
    except (OSError, ValueError):
        pass
    return None


def cpu_baseline(name, torch):
    """The oracle (reference algorithm restated in C, OpenMP) on a cropped sample."""
    from oracle import cpu
    crop = (8, 15, 27) if WORKLOADS[name][1] >= 512 else (8, 30, 27)
    x, off, m, w, b, gout, G = make_inputs(name, torch, crop)
    if WORKLOADS[name][4] == "bf16":
        x, w, b, gout = (t.bfloat16().float() for t in (x, w, b, gout))
    t0 = time.perf_counter()
    cpu.conv3d_forward(x, off, m, w, b, 1, 1, 1, 1, G)
    cpu.conv3d_backward(gout, x, off, m, w, True, 1, 1, 1, 1, G)
    dt = time.perf_counter() - t0
    C = x.shape[1]
    P = crop[0] * crop[1] * crop[2]
    flops = 3 * 2 * P * C * C * 27
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cpu.num_threads(), "kind": "port",
        "sample": f"same layer (C={C}, k3, G={G}) on N=1, {crop[0]}x{crop[1]}x{crop[2]} positions, fp32, "
                  f"forward+backward once: {dt:.2f} s",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this operator path is measured on ONE GPU only (--gpus 1); "
                 "no multi-GPU run exists or is meaningful for it")

    import torch
    from d2conv3d_amd import _lib
    lib = _lib.load()  # raises if the HIP library is missing: there is no fallback
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    name = args.workload
    N, C, dims, G, dt, sig, seed = WORKLOADS[name]
    x, off, m, w, b, gout, G = make_inputs(name, torch)
    tdt = torch.bfloat16 if dt == "bf16" else torch.float32
    x, w, b, gout = (t.to(dev, tdt).contiguous() for t in (x, w, b, gout))
    off, m = (t.to(dev, tdt).contiguous() for t in (off, m))
    code = _lib.D2C_BF16 if dt == "bf16" else _lib.D2C_F32
    T_, H_, W_ = dims
    desc = _lib.Conv3dDesc(N, C, C, T_, H_, W_, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, G, T_, H_, W_, code, code)
    _lib.check(lib.d2c_conv3d_check(ctypes.byref(desc)), "check")
    algo = _lib.ALGO_NAMES[lib.d2c_conv3d_algo(ctypes.byref(desc))]
    out = torch.empty(N, C, *dims, device=dev, dtype=tdt)
    gx, goff, gm, gw, gb = (torch.empty_like(t) for t in (x, off, m, w, b))
    nf = lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(desc))
    nb = lib.d2c_conv3d_backward_workspace_bytes(ctypes.byref(desc))
    ws = torch.empty(max(nf, nb, 256), dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def step():
        rc = lib.d2c_conv3d_forward(ctypes.byref(desc), p(x), p(off), p(m), p(w), p(b), p(out), p(ws), nf, stream)
        _lib.check(rc, "forward")
        rc = lib.d2c_conv3d_backward(ctypes.byref(desc), p(gout), p(x), p(off), p(m), p(w), p(gx), p(goff), p(gm),
                                     p(gw), p(gb), p(ws), nb, stream)
        _lib.check(rc, "backward")

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps

    P = T_ * H_ * W_
    f_fwd = 2.0 * N * P * C * C * 27
    value = 3 * f_fwd / (ms * 1e-3) / 1e12

    # per-kernel durations: HIP events on the launch stream, recorded inside the library
    lib.d2c_profile_reset()
    lib.d2c_profile_enable(1)
    nprof = max(3, min(args.steps, 10))
    for _ in range(nprof):
        step()
    torch.cuda.synchronize()
    lib.d2c_profile_enable(0)
    kern = {}
    for kid, kname in ((_lib.PROF_FWD, "tiled_fwd_kernel"), (_lib.PROF_BWD_DATA, "tiled_bwd_data_kernel"),
                       (_lib.PROF_BWD_WEIGHT, "tiled_bwd_weight_kernel"), (_lib.PROF_GX_OWNER, "gx_owner_kernel"),
                       (_lib.PROF_PACK, "pack/clear/convert/lists")):
        tot, cnt = ctypes.c_double(0), ctypes.c_int(0)
        lib.d2c_profile_read(kid, ctypes.byref(tot), ctypes.byref(cnt))
        if cnt.value:
            kern[kname] = tot.value / nprof  # ms per step spent in this kernel (all launches of it)
    # the kernel that takes the most time, against the roofline that bounds it
    main_k = {k: v for k, v in kern.items() if not k.startswith("pack")}
    dom = max(main_k, key=main_k.get) if main_k else None
    roofline = None
    if dom:
        traffic = hbm_traffic_bytes(dom)
        kms = {k: round(v, 4) for k, v in kern.items()}
        if dom == "gx_owner_kernel":
            # memory-bound: every grad-column row (N*P*K*Cin elements), every list entry (32 B per live
            # sample) and every grad_input element (fp32 accumulator) once
            es = 2 if dt == "bf16" else 4
            nbytes = N * P * 27 * C * es + N * P * 27 * G * 32 + N * C * P * 4
            ach = nbytes / (main_k[dom] * 1e-3) / 1e9
            roofline = {"bound": "hbm", "kernel": dom, "achieved": round(ach, 1), "peak": 8000.0, "unit": "GB/s",
                        "frac": round(ach / 8000.0, 4), "traffic": traffic, "kernel_ms": kms}
        else:
            ach = f_fwd / (main_k[dom] * 1e-3) / 1e12  # each of the three tiled kernels carries one GEMM of f_fwd flops
            roofline = {"bound": "mfma", "kernel": dom, "achieved": round(ach, 2), "peak": PEAK_TFLOPS[dt],
                        "unit": "TFLOP/s", "frac": round(ach / PEAK_TFLOPS[dt], 4), "traffic": traffic,
                        "kernel_ms": kms}

    line = {
        "metric": "mdconv3d fwd+bwd effective TFLOP/s (C=512, 8x30x54, k3) on 1 GPU" if name == "c3"
                  else f"mdconv3d fwd+bwd effective TFLOP/s ({name})",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{name}: modulated deformable conv3d fwd+bwd, N={N}, Cin=Cout={C}, "
                               f"{T_}x{H_}x{W_}, k3 p1, offset_groups={G}, bias, {dt} in / fp32 accumulate",
                   "kernel_family": algo, "frac_of_peak_whole_step": round(value / PEAK_TFLOPS[dt], 4)},
        "roofline": roofline,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(name, torch)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
