#!/usr/bin/env python3
"""Headline benchmark: RandomHingeForest fp32 forward+backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c1|c4] [--mode atomic|deterministic]
                    [--path train|stateless]

One step = one forward plus one backward (all three gradients requested, atomic mode) over one batch of synthetic input
that is already resident in HBM, called through the C ABI on torch's current stream. `--path train` (default) is what
the autograd functions run in training: the forward keeps its walk records and the backward consumes them
(tree_forward_records / tree_backward_records); `--path stateless` is the reference's operator pair (tree_forward /
tree_backward), whose backward walks the trees again. The other path is timed too and reported under `other_path`.
The default workload is the configuration the metric is quoted on: x ~ N(0,1) [65536, 1024], 1000 trees, depth 10,
extra_outputs = 10 (out [65536, 1000, 10]); thresholds ~ U(-3,3) made consistent like the module constructor does,
ordinals ~ U{0..1023}, leaf weights ~ N(0,1), upstream gradient ~ N(0,1).

`--workload c4` times the convolutional operator instead (tree_conv2d_forward / tree_conv2d_backward on images
[32,16,128,128], 64 out channels, depth 6, 3x3 taps: 64 x 16 trees over the 9 taps of one channel each, summed over
the channels); it is bound by LDS reads and vector instructions, not by HBM, so its line reports images/s and vertex
visits/s with the HBM fraction for information only.

`--workload c5` times the README model's dense front plus forest (linear_bn_forward -> tree_forward ->
tree_backward -> linear_bn_backward); its roofline object prices the projection against the fp32 matrix-core peak.

Prints ONE JSON line. `value` is samples/s over the timed steps (wall clock between device synchronisations);
`roofline` prices the whole step (forward + backward, the metric's own scope) against the 8 TB/s HBM peak using its
algorithmic bytes (every input read once, every output written once) and its duration measured with events on the
launch stream, with the forward and backward fractions beside it; it names the step's largest kernel and the measured
HBM traffic per step from the rocprofv3 summaries under profiles/ -- only where those were measured on the kernel
sources the library is built from, else null; `cpu_baseline` is the reference's single-threaded CPU path (its own sources
compiled into oracle/_ref, else the oracle's restatement of them) timed on a bounded slice of the same workload on this
host.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

PROFILES = os.path.join(ROOT, "profiles")
STEP_KERNELS = ("forward_rows_kernel", "pad_rows", "pack_quads_kernel", "pack_nodes_kernel", "tree_lean_kernel",
                "tree_kernel", "dx_kernel", "dthr_kernel", "zero_kernel")


def kernel_sources_digest():
    """Digest of the HIP sources the library is built from. The rocprofv3 summaries under profiles/ carry the digest of
    the sources they were measured on; figures are only quoted from a summary whose digest equals the current one."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "hingetreefortorch_amd", "csrc")
    for name in sorted(os.listdir(src)):
        if name.endswith((".hip", ".hpp")):
            h.update(name.encode())
            h.update(open(os.path.join(src, name), "rb").read())
    return h.hexdigest()[:16]


def profiled_step(workload):
    """What the committed rocprofv3 summaries of this workload say about one step of the training path: the kernel with
    the largest average duration and the HBM bytes per step (FETCH_SIZE + WRITE_SIZE over the step's kernels, scaled as
    the summary states). (None, None, reason) where the summaries are missing or were measured on other sources."""
    import re
    digest = kernel_sources_digest()
    prefix = {"c3": "forest_c3", "c2": "fern_c2"}.get(workload)
    if prefix is None:
        return None, None, "no profile for this workload"
    out = {}
    for what in ("kernel_stats", "hbm_traffic"):
        path = os.path.join(PROFILES, f"{prefix}_{what}.txt")
        if not os.path.exists(path):
            return None, None, f"profiles/{prefix}_{what}.txt is missing"
        text = open(path).read()
        m = re.search(r"kernel sources digest: ([0-9a-f]{16})", text)
        if m is None or m.group(1) != digest:
            return None, None, (f"profiles/{prefix}_{what}.txt was measured on other kernel sources "
                                f"({m.group(1) if m else 'no digest'} vs {digest})")
        out[what] = text
    best, total = None, 0.0
    for line in out["kernel_stats"].splitlines():
        cols = line.split()
        if len(cols) >= 6 and cols[0].startswith(STEP_KERNELS):
            try:
                avg = float(cols[-4])
            except ValueError:
                continue
            if best is None or avg > best[1]:
                best = (cols[0].split("<")[0], avg)
    for line in out["hbm_traffic"].splitlines():
        cols = line.split()
        if len(cols) >= 4 and (cols[0].startswith(STEP_KERNELS) or cols[0].startswith("ht::pad_rows")):
            try:
                total += float(cols[-1]) * 1e6
            except ValueError:
                continue
    return (best[0] if best else None), (int(total) if total else None), f"profiles/{prefix}_*.txt, kernel sources digest {digest}"


WORKLOADS = {
    # name: (B, F, T, depth, M, kind, x distribution, description)
    "c3": (65536, 1024, 1000, 10, 10, "tree", "normal",
           "forest fp32 fwd+bwd, x~N(0,1) [65536,1024], T=1000, depth=10, extra_outputs=10"),
    "c2": (65536, 1024, 1000, 10, 1, "fern", "normal",
           "fern fp32 fwd+bwd, x~N(0,1) [65536,1024], T=1000, depth=10, extra_outputs=1"),
    "c1": (100, 1000, 100, 7, 1, "tree", "uniform",
           "forest fp32 fwd+bwd, x~U[0,1) [100,1000], T=100, depth=7, extra_outputs=1"),
}


def algorithmic_bytes(B, F, T, depth, M, kind):
    """Compulsory traffic: every input read once, every output written once; ordinals at their int64 API width."""
    V = depth if kind == "fern" else 2 ** depth - 1
    L = 2 ** depth
    x, thr, ordn, w, out = 4 * B * F, 4 * T * V, 8 * T * V, 4 * T * L * M, 4 * B * T * M
    fwd = x + thr + ordn + w + out
    bwd = x + thr + ordn + w + out + x + thr + w   # + gout read, dX, dThr, dW written
    return fwd, bwd


def make_inputs(torch, name, dev):
    import hingetree_cpp as ops
    B, F, T, depth, M, kind, dist, _ = WORKLOADS[name]
    g = torch.Generator().manual_seed(6112)
    V = depth if kind == "fern" else 2 ** depth - 1
    thr = 6.0 * torch.rand([T, V], generator=g) - 3.0
    ordn = torch.randint(0, F, [T, V], generator=g, dtype=torch.int64)
    w = torch.randn([T, 2 ** depth, M], generator=g)
    if kind == "tree":
        ops.tree_fix_thresholds(thr, ordn, w)   # as the module constructor does (host side)
    gg = torch.Generator(device=dev).manual_seed(6113)
    if dist == "normal":
        x = torch.randn([B, F], generator=gg, device=dev)
    else:
        x = torch.rand([B, F], generator=gg, device=dev)
    gout = torch.randn([B, T, M], generator=gg, device=dev)
    return x, thr.to(dev), ordn.to(dev), w.to(dev), gout


def cpu_baseline(torch, name, x, thr, ordn, w, gout, budget_rows):
    """The reference's CPU path on the first rows of the same batch, one thread: its own sources as compiled into
    oracle/_ref where that build is present (kind "reference"), else the oracle's restatement of them (kind "port");
    with the reference build present the port is timed on half the slice as well, to show the two agree."""
    from oracle import hinge_oracle as ho
    B, F, T, depth, M, kind, _, _ = WORKLOADS[name]
    rows = min(B, budget_rows)
    xs, gs = x[:rows].cpu().contiguous(), gout[:rows].cpu().contiguous()
    tc, oc, wc = thr.cpu(), ordn.cpu(), w.cpu()
    fern = kind == "fern"
    pre = "fern_" if fern else "tree_"
    ho.lib()
    try:
        ref = ho.reference_module()
    except Exception:  # a build for another torch: fall back to the port
        ref = None

    def port(n):
        t0 = time.perf_counter()
        ho.forward(xs[:n], tc, oc, wc, fern)
        t1 = time.perf_counter()
        ho.backward(xs[:n], tc, oc, wc, gs[:n], fern=fern)
        return t1 - t0, time.perf_counter() - t0

    if ref is None:
        fwd_s, all_s = port(rows)
        extra = {}
    else:
        threads = torch.get_num_threads()
        torch.set_num_threads(1)
        try:
            t0 = time.perf_counter()
            getattr(ref, pre + "forward")(xs, tc, oc, wc)
            t1 = time.perf_counter()
            getattr(ref, pre + "backward")(xs, True, tc, True, oc, False, wc, True, gs)
            fwd_s, all_s = t1 - t0, time.perf_counter() - t0
        finally:
            torch.set_num_threads(threads)
        half = max(1, rows // 2)
        extra = {"port_value": half / port(half)[1], "port_sample": f"the oracle's restatement on the first {half} rows"}
    return {"value": rows / all_s, "unit": "samples/s", "cores": 1, "kind": "port" if ref is None else "reference",
            "sample": f"first {rows} of {B} rows of the same batch, all {T} trees; 1 forward + 1 backward "
                      f"(3 gradients) = {all_s:.2f} s (forward {fwd_s:.2f} s), single thread",
            "host_cores": os.cpu_count(), **extra}


def bench_conv(torch, ops, dev, args):
    """HingeTreeConv2d forward+backward on the convolutional benchmark shape."""
    B, C, Cout, H, W, depth = 32, 16, 64, 128, 128, 6
    V, L = 2 ** depth - 1, 2 ** depth
    g = torch.Generator().manual_seed(6112)
    thr = (6.0 * torch.rand([Cout, C, V], generator=g) - 3.0).to(dev)
    ordn = torch.randint(0, 9, [Cout, C, V], generator=g, dtype=torch.int64).to(dev)
    w = torch.randn([Cout, C, L], generator=g).to(dev)
    gg = torch.Generator(device=dev).manual_seed(6113)
    x = torch.randn([B, C, H, W], generator=gg, device=dev)
    gout = torch.randn([B, Cout, H, W], generator=gg, device=dev)
    geo = ([3, 3], [1, 1], [1, 1], [1, 1])

    def step(ev=None):
        if ev: ev[0].record()
        ops.tree_conv2d_forward(x, thr, ordn, w, *geo)
        if ev: ev[1].record()
        ops.tree_conv2d_backward(x, True, thr, True, ordn, False, w, True, gout, *geo)
        if ev: ev[2].record()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(ev[i])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    walks = B * Cout * C * H * W
    fwd_bytes = 4 * (x.numel() + thr.numel() + w.numel() + gout.numel()) + 8 * ordn.numel()
    bwd_bytes = fwd_bytes + 4 * (x.numel() + thr.numel() + w.numel())
    return {
        "metric": "conv fwd+bwd images/s (HingeTreeConv2d [32,16,128,128] -> 64 channels, depth 6, 3x3)",
        "value": B / (ms * 1e-3), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "c4: 64 x 16 trees of depth 6 over the 9 taps of one input channel each, summed over "
                               "the 16 channels; stride 1, padding 1, dilation 1", "B": B, "C": C, "Cout": Cout,
                   "H": H, "W": W, "depth": depth},
        "forward": {"ms": fwd_ms, "vertex_visits_per_s": walks * depth / (fwd_ms * 1e-3),
                    "hbm_frac": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "backward": {"ms": bwd_ms, "hbm_frac": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "roofline": {"bound": "hbm", "kernel": "conv_tiled_forward_kernel",
                     "achieved": fwd_bytes / (fwd_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "traffic": None,
                     "note": "informational: the kernel is bound by LDS reads and vector instructions "
                             "(3.2e9 vertex visits per pass), not by HBM"},
    }


MFMA_FP32_PEAK_TFLOPS = 157.3


def bench_projection(torch, ops, dev, args):
    """Linear(784 -> 12700, no bias) -> BatchNorm1d(affine=False) -> forest (100 trees, depth 7, sequential ordinals,
    10 outputs per leaf), forward+backward with gradients for the projection, the thresholds and the leaf weights."""
    B, K, T, depth, M = 16384, 784, 100, 7, 10
    V, L = 2 ** depth - 1, 2 ** depth
    N = T * V
    g = torch.Generator().manual_seed(6112)
    x = torch.rand([B, K], generator=g).to(dev)
    lin = (torch.randn([N, K], generator=g) / K ** 0.5).to(dev)
    thr = 6.0 * torch.rand([T, V], generator=g) - 3.0
    ordn = torch.arange(N, dtype=torch.int64).reshape(T, V)
    w = torch.randn([T, L, M], generator=g)
    ops.tree_fix_thresholds(thr, ordn, w)
    thr, ordn, w = thr.to(dev), ordn.to(dev), w.to(dev)
    gout = torch.randn([B, T, M], generator=torch.Generator(device=dev).manual_seed(6113), device=dev)

    dense = bool(getattr(args, "dense_backward", False))

    def step(ev=None):
        if ev: ev[0].record()
        if dense:
            zhat, mean, rstd, var = ops.linear_bn_forward(x, lin, 1e-5)
            if ev: ev[1].record()
            # the training path of the autograd function: the forward keeps its walk records for the backward
            out, rec = ops.tree_forward_records(zhat, thr, ordn, w)
        else:
            # one call: product + statistics, then the forest normalising the product as it reads it
            if ev: ev[1].record()
            out, rec, z, mean, rstd, var = ops.tree_linear_bn_forward_records(x, lin, 1e-5, thr, ordn, w)
        if ev: ev[2].record()
        if dense:
            # dense route: the forest's input gradient as a [B, N] matrix, batch-norm backward, dLin = dz^T x
            dz, dthr, _, dw = ops.tree_backward_records(rec, False, zhat, True, thr, True, ordn, False, w, True, gout)
            if ev: ev[3].record()
            ops.linear_bn_backward(x, False, lin, True, zhat, rstd, dz)
        else:
            # all three gradients from the walk records; the forest's input gradient (one non-zero per sample and
            # tree) is never formed
            if ev: ev[3].record()
            got = ops.tree_linear_bn_backward_records(rec, x, lin, True, z, rstd, thr, True, ordn, w, True, gout,
                                                      mean=mean)
            assert got is not None
        if ev: ev[4].record()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(ev[i])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    seg = [sum(e[i].elapsed_time(e[i + 1]) for e in ev) / args.steps for i in range(4)]
    flops = 2.0 * B * K * N
    # the projection's product by itself, for the matrix-core roofline: the separate operator (product with batch sums,
    # statistics, normalisation pass), timed apart from the step
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        ops.linear_bn_forward(x, lin, 1e-5)
    e1.record()
    torch.cuda.synchronize()
    proj_ms = e0.elapsed_time(e1) / 5
    tf_proj = flops / (proj_ms * 1e-3) / 1e12
    if dense:
        parts = {
            "projection_forward": {"ms": seg[0], "tflops": flops / (seg[0] * 1e-3) / 1e12,
                                   "note": "GEMM with fused batch sums + statistics + in-place normalisation"},
            "forest_forward_ms": seg[1], "forest_backward_ms": seg[2],
            "projection_backward": {"ms": seg[3], "tflops": flops / (seg[3] * 1e-3) / 1e12,
                                    "note": "batch-norm backward sums + dLin = dz^T x GEMM with the normalisation's "
                                            "backward in its operand loader"},
        }
    else:
        parts = {
            "forward": {"ms": seg[0] + seg[1],
                        "note": "one call: GEMM with fused batch sums, statistics, forest forward with walk records "
                                "that normalises the product as it reads it (no normalised copy is written)"},
            "backward": {"ms": seg[2] + seg[3],
                         "note": "one call: forest backward (dThr, dW) + dLin from the walk records -- segment sums of "
                                 "centred inputs per (tree, vertex), xc^T xc and lin * (xc^T xc) on the matrix cores; no "
                                 "dense gradient [B, N] is formed (--dense-backward times the dense route)"},
        }
    out = {
        "metric": "fwd+bwd samples/s (Linear 784->12700 + BatchNorm + forest T=100,D=7,M=10, B=16384)",
        "value": B / (ms * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "c5: x~U[0,1) [16384,784], bias-free linear to 12700 = 100 x 127 private vertex features, "
                               "batch norm without affine, forest 100 trees depth 7 sequential ordinals, 10 outputs "
                               "per leaf; gradients: linear weights, thresholds, leaf weights", "B": B, "K": K, "N": N,
                   "T": T, "depth": depth, "extra_outputs": M, "route": "dense" if dense else "records"},
        "projection_operator": {"ms": proj_ms, "tflops": tf_proj,
                                "note": "linear_bn_forward alone, outside the timed step: GEMM with fused batch sums + "
                                        "statistics + normalisation pass"},
        "roofline": {"bound": "mfma", "kernel": "gemm_kernel (projection forward)", "achieved": tf_proj,
                     "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf_proj / MFMA_FP32_PEAK_TFLOPS,
                     "traffic": None, "flops": flops,
                     "note": "the timed span also holds the statistics and normalisation kernels"},
    }
    out.update(parts)
    return out


def _timed(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def bench_mix(torch, ops, dev, args):
    """The forest -> linear operators (tree_fused_linear_forward / backward) at the headline forest shape with a
    10-class linear head: 65536 x 1024 inputs, 1000 trees of depth 10 with one output per leaf, mixed down to 10
    channels."""
    B, F, T, depth, O = 65536, 1024, 1000, 10, 10
    V, L = 2 ** depth - 1, 2 ** depth
    g = torch.Generator().manual_seed(6112)
    thr = 6.0 * torch.rand([T, V], generator=g) - 3.0
    ordn = torch.randint(0, F, [T, V], generator=g, dtype=torch.int64)
    w = torch.randn([T, L], generator=g)
    ops.tree_fix_thresholds(thr, ordn, w)
    lin = (torch.randn([O, T], generator=g) / T ** 0.5).to(dev)
    bias = torch.randn([O], generator=g).to(dev)
    thr, ordn, w = thr.to(dev), ordn.to(dev), w.to(dev)
    gg = torch.Generator(device=dev).manual_seed(6113)
    x = torch.randn([B, F], generator=gg, device=dev)
    gout = torch.randn([B, O], generator=gg, device=dev)
    # the training path of the autograd function: the forward keeps the forest output and the walk records
    fwd_ms = _timed(torch, lambda: ops.tree_fused_linear_forward_records(x, thr, ordn, w, lin, bias), args.steps,
                    args.warmup)
    _, f, records = ops.tree_fused_linear_forward_records(x, thr, ordn, w, lin, bias)
    bwd_ms = _timed(torch, lambda: ops.tree_fused_linear_backward_records((f, records), False, x, True, thr, True, ordn,
                                                                           False, w, True, lin, True, bias, True, gout),
                    args.steps, args.warmup)
    # ... and the reference's stateless operator pair, whose backward computes the forest again
    s_fwd = _timed(torch, lambda: ops.tree_fused_linear_forward(x, thr, ordn, w, lin, bias), args.steps, args.warmup)
    s_bwd = _timed(torch, lambda: ops.tree_fused_linear_backward(x, True, thr, True, ordn, False, w, True, lin, True,
                                                                  bias, True, gout), args.steps, args.warmup)
    plain_fwd = _timed(torch, lambda: ops.tree_forward(x, thr, ordn, w), args.steps, args.warmup)
    ms = fwd_ms + bwd_ms
    # every input read once, every output written once (the forest's [B, T] intermediate is not part of the interface)
    fwd_bytes = 4 * (B * F + T * V + T * L + O * T + O + B * O) + 8 * T * V
    bwd_bytes = fwd_bytes + 4 * (B * F + T * V + T * L + O * T + O)
    return {
        "metric": "fwd+bwd samples/s (forest -> linear: B=65536,F=1024,T=1000,D=10 -> 10 channels)",
        "value": B / (ms * 1e-3), "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "f1: forest -> linear forward + backward (all five gradients) as HingeTreeFusedLinear runs them, "
                               "x~N(0,1) [65536,1024], 1000 trees of depth 10, one output per leaf, linear head "
                               "[10,1000] with bias", "B": B, "F": F, "T": T, "depth": depth, "out_channels": O},
        "forward": {"ms": fwd_ms, "of_which_forest_ms": plain_fwd}, "backward": {"ms": bwd_ms},
        "other_path": {"path": "stateless", "forward_ms": s_fwd, "backward_ms": s_bwd},
        "roofline": {"bound": "hbm", "kernel": "forward_rows_kernel + gemm_kernel (forest, then the mix over trees)",
                     "achieved": fwd_bytes / (fwd_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "traffic": None,
                     "algorithmic_bytes": fwd_bytes,
                     "note": "interface bytes only; the operator also writes and re-reads the 262 MB forest output"},
        "backward_hbm_frac": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
    }


def bench_tiles(torch, ops, dev, args):
    """contract / expand on the segmentation shape: leaf patches [8,100,64,64,8,8] <-> images [8,100,512,512]."""
    B, C, H, W, P = 8, 100, 512, 512, 8
    gg = torch.Generator(device=dev).manual_seed(6113)
    image = torch.randn([B, C, H, W], generator=gg, device=dev)
    tiles = ops.contract(image, [P, P], [0, 0])
    c_ms = _timed(torch, lambda: ops.contract(image, [P, P], [0, 0]), args.steps, args.warmup)
    e_ms = _timed(torch, lambda: ops.expand(tiles, [0, 0]), args.steps, args.warmup)
    nbytes = 2 * image.numel() * 4   # read once, written once
    ms = c_ms + e_ms
    # the head of the segmentation model: forest with 8 x 8 outputs per leaf on [8, 100, 64, 64], then expand
    F, T, D = 100, 100, 6
    cg = torch.Generator().manual_seed(6114)
    x = torch.randn([B, F, H // P, W // P], generator=cg).to(dev)
    thr = (6 * torch.rand([T, 2 ** D - 1], generator=cg) - 3).to(dev)
    ordn = torch.randint(0, F, [T, 2 ** D - 1], generator=cg, dtype=torch.int64).to(dev)
    wts = torch.randn([T, 2 ** D, P, P], generator=cg).to(dev)
    assert torch.equal(ops.tree_forward_expanded(x, thr, ordn, wts, [0, 0]),
                       ops.expand(ops.tree_forward(x, thr, ordn, wts), [0, 0]))
    two_ms = _timed(torch, lambda: ops.expand(ops.tree_forward(x, thr, ordn, wts), [0, 0]), args.steps, args.warmup)
    one_ms = _timed(torch, lambda: ops.tree_forward_expanded(x, thr, ordn, wts, [0, 0]), args.steps, args.warmup)
    # ... and its backward from the gradient of the image: contract + backward against the one call that reads the image
    gimg = torch.randn([B, T, H, W], generator=gg, device=dev)
    bwd_two_ms = _timed(torch, lambda: ops.tree_backward(x, True, thr, True, ordn, False, wts, True,
                                                         ops.contract(gimg, [P, P], [0, 0])), args.steps, args.warmup)
    bwd_one_ms = _timed(torch, lambda: ops.tree_backward_expanded(False, [0, 0], x, True, thr, True, ordn, False, wts,
                                                                  True, gimg), args.steps, args.warmup)
    return {
        "metric": "contract + expand GB/s (tiles [8,100,64,64,8,8] <-> images [8,100,512,512])",
        "value": 2 * nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "f3: one contract and one expand of an 839 MB float32 image batch, window 8 x 8, no padding"},
        "contract": {"ms": c_ms, "gbps": nbytes / (c_ms * 1e-3) / 1e9}, "expand": {"ms": e_ms, "gbps": nbytes / (e_ms * 1e-3) / 1e9},
        "forest_then_expand": {"ms": two_ms, "what": "tree_forward [8,100,64,64] x 100 trees of depth 6 x [8,8] outputs, then expand"},
        "forest_expanded": {"ms": one_ms, "what": "the same image from one pass (tree_forward_expanded)",
                            "gbps": (nbytes // 2 + x.numel() * 4) / (one_ms * 1e-3) / 1e9},
        "contract_then_backward": {"ms": bwd_two_ms, "what": "contract of the image gradient, then tree_backward (x, thresholds, leaf weights)"},
        "backward_expanded": {"ms": bwd_one_ms, "what": "the same gradients from one call that reads the image gradient (tree_backward_expanded)",
                              "gbps": (nbytes // 2) / (bwd_one_ms * 1e-3) / 1e9},
        "roofline": {"bound": "hbm", "kernel": "tile_permute_kernel", "achieved": 2 * nbytes / (ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": 2 * nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     "traffic": None, "algorithmic_bytes": nbytes},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--dense-backward", action="store_true",
                    help="c5: backward through a dense dL/dzhat (forest dX, batch-norm backward, dz^T x) instead of "
                         "the records form")
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + ["c4", "c5", "f1", "f3"])
    ap.add_argument("--mode", default="atomic", choices=["atomic", "deterministic"])
    ap.add_argument("--path", default="train", choices=["train", "stateless"])
    ap.add_argument("--other-steps", type=int, default=-1,
                    help="timed steps of the path not selected by --path (-1: a quarter of --steps, 0: skip)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run three 1 GiB device-to-device copies (what the HBM counters are scaled against)")
    ap.add_argument("--graph", action="store_true",
                    help="also time the step replayed from a HIP graph (always done for the launch-bound c1)")
    ap.add_argument("--cpu-rows", type=int, default=32768, help="rows of the batch timed on the CPU (0 = skip)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the path needs no exchange between GPUs and nothing "
                 "here shards it); use --gpus 1.")

    import torch
    import hingetree_cpp as ops

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP library is the only back-end.")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        src = torch.ones(256 * 1024 * 1024, dtype=torch.float32, device=dev)   # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "3 x copy of 1 GiB (reads 1073741824 B, writes 1073741824 B per launch)"}))
        return
    name = args.workload
    if name == "c4":
        print(json.dumps(bench_conv(torch, ops, dev, args)), flush=True)
        return
    if name == "c5":
        print(json.dumps(bench_projection(torch, ops, dev, args)), flush=True)
        return
    if name == "f1":
        print(json.dumps(bench_mix(torch, ops, dev, args)), flush=True)
        return
    if name == "f3":
        print(json.dumps(bench_tiles(torch, ops, dev, args)), flush=True)
        return
    B, F, T, depth, M, kind, _, desc = WORKLOADS[name]
    x, thr, ordn, w, gout = make_inputs(torch, name, dev)
    pre = "fern_" if kind == "fern" else "tree_"
    det = args.mode == "deterministic"

    def make_step(path):
        if path == "train":
            fwd_op, bwd_op = getattr(ops, pre + "forward_records"), getattr(ops, pre + "backward_records")

            def fwd():
                return fwd_op(x, thr, ordn, w)

            stateless_bwd = getattr(ops, pre + ("backward_deterministic" if det else "backward"))

            def bwd(state):
                if state[1] is None:   # shape for which the library keeps no records: the autograd function re-walks
                    return stateless_bwd(x, True, thr, True, ordn, False, w, True, gout)
                return bwd_op(state[1], det, x, True, thr, True, ordn, False, w, True, gout)
        else:
            fwd_op = getattr(ops, pre + "forward")
            bwd_op = getattr(ops, pre + ("backward_deterministic" if det else "backward"))

            def fwd():
                return fwd_op(x, thr, ordn, w)

            def bwd(state):
                return bwd_op(x, True, thr, True, ordn, False, w, True, gout)
        return fwd, bwd

    def run(path, steps, warmup):
        fwd, bwd = make_step(path)
        for _ in range(warmup):
            bwd(fwd())
        torch.cuda.synchronize()
        # events on torch's current stream, which is the stream the library launches on
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
        t0 = time.perf_counter()
        for i in range(steps):
            ev[i][0].record()
            state = fwd()
            ev[i][1].record()
            grads = bwd(state)
            ev[i][2].record()
            del state, grads
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return ((t1 - t0) * 1e3 / steps, sum(e[0].elapsed_time(e[1]) for e in ev) / steps,
                sum(e[1].elapsed_time(e[2]) for e in ev) / steps)

    def run_graph(path, steps):
        """The same step captured once into a HIP graph and replayed: what a launch-bound shape costs without the
        per-launch host work (the library allocates nothing and clears memory with kernels, so it can be captured)."""
        fwd, bwd = make_step(path)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                bwd(fwd())
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            held = bwd(fwd())
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        del held
        return (time.perf_counter() - t0) * 1e3 / steps

    other = "stateless" if args.path == "train" else "train"
    other_steps = max(3, args.steps // 4) if args.other_steps < 0 else args.other_steps
    o_ms = o_fwd = o_bwd = None
    if other_steps > 0:
        o_ms, o_fwd, o_bwd = run(other, other_steps, 2)
    ms_per_step, fwd_ms, bwd_ms = run(args.path, args.steps, args.warmup)

    fwd_bytes, bwd_bytes = algorithmic_bytes(B, F, T, depth, M, kind)
    # The roofline object prices the whole step -- the metric is forward + backward -- on its event-timed duration
    # (forward span + backward span on the launch stream); `kernel` names the step's largest kernel by the committed
    # rocprofv3 summary, and `traffic` is the measured HBM bytes per step from the same summaries: both only where
    # those summaries were taken on the kernel sources this library is built from.
    dominant, traffic, source = (None, None, "deterministic mode has its own summary") if det else profiled_step(name)
    if args.path != "train":
        traffic = None
    span_ms = fwd_ms + bwd_ms
    achieved = (fwd_bytes + bwd_bytes) / (span_ms * 1e-3) / 1e9
    result = {
        "metric": "fwd+bwd samples/s (forest B=65536,F=1024,T=1000,D=10) + % of HBM peak BW",
        "value": B / (ms_per_step * 1e-3),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{name}: {desc}", "backward_mode": args.mode, "path": args.path, "host": ops.host, "B": B, "F": F, "T": T, "depth": depth,
                   "extra_outputs": M},
        "roofline": {"bound": "hbm",
                     "kernel": dominant or "forward kernel + tree kernel (the step's two large kernels; no current profile names the larger)",
                     "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": traffic, "traffic_source": source,
                     "algorithmic_bytes": fwd_bytes + bwd_bytes, "ms": span_ms,
                     "scope": "one step = forward pass + backward pass (all kernels), events on the launch stream",
                     "forward": {"ms": fwd_ms, "algorithmic_bytes": fwd_bytes, "samples_per_s": B / (fwd_ms * 1e-3),
                                 "frac": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
                     "backward": {"ms": bwd_ms, "algorithmic_bytes": bwd_bytes, "samples_per_s": B / (bwd_ms * 1e-3),
                                  "frac": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}},
        "backward": {"mode": args.mode, "ms": bwd_ms, "samples_per_s": B / (bwd_ms * 1e-3),
                     "algorithmic_bytes": bwd_bytes, "hbm_frac": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "forward": {"ms": fwd_ms, "samples_per_s": B / (fwd_ms * 1e-3), "algorithmic_bytes": fwd_bytes,
                    "hbm_frac": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "step_hbm_frac": (fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
    }
    if args.graph or name == "c1":
        g_ms = run_graph(args.path, max(args.steps, 50))
        result["hip_graph"] = {"ms_per_step": g_ms, "samples_per_s": B / (g_ms * 1e-3),
                               "note": "the same step captured once with torch.cuda.CUDAGraph and replayed"}
    if o_ms is not None:
        result["other_path"] = {"path": other, "ms_per_step": o_ms, "forward_ms": o_fwd, "backward_ms": o_bwd,
                                "samples_per_s": B / (o_ms * 1e-3)}
    if args.cpu_rows > 0:
        result["cpu_baseline"] = cpu_baseline(torch, name, x, thr, ordn, w, gout, args.cpu_rows)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
