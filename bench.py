#!/usr/bin/env python3
"""Benchmark of the DiffLUT hot path on one MI355X.

A step is one forward + EFD backward of a single RandomLayer + DWN layer through the C ABI
(dl_dwn_layer_fwd / dl_dwn_layer_bwd), on synthetic data already resident in HBM:
  bits Bernoulli(0.5) [4096,16384] stored fp32, 8192 nodes with k=6 (64-entry fp32 tables
  U[-1,1]), seeded RandomLayer mapping, upstream gradient N(0,1), input gradient produced.
Outputs, gradients and workspaces are allocated once before the timed region.

Prints ONE JSON line (metric = LUT-node evals/sec, forward+backward) that also carries
  roofline     - the dominant kernel: algorithmic bytes per launch / its average duration, measured
                 with HIP events on the launch stream (the library's per-kernel timing hook)
  roofline_step- the whole step against the 1 080 229 888 algorithmic bytes of forward+backward
  cpu_baseline - the C restatement of the reference's CPU loops (oracle/dwn_oracle.c, OpenMP) timed
                 on the host cores on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
PROFILE_DIR = os.path.join(ROOT, "profiles")
KERNEL_SOURCE = os.path.join(ROOT, "difflut_amd", "csrc", "dwn_kernels.hip")


def source_hash(path=KERNEL_SOURCE):
    import hashlib
    with open(path, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from the rocprofv3 counter summary committed under profiles/ (FETCH_SIZE scaled
    by the copy calibration written there, plus WRITE_SIZE).  The summary names the hash of the kernel source it was
    measured on; when the source has changed since, the figure is stale and None is reported instead."""
    import re
    path = os.path.join(PROFILE_DIR, f"{workload}_kernels.md")
    if not os.path.exists(path):
        return None
    text = open(path).read()
    m = re.search(r"kernel_source_sha256_16:\s*([0-9a-f]{16})", text)
    t = re.search(rf"traffic_bytes_per_launch:\s*{re.escape(kernel)}\s+(\d+)", text)
    if not m or not t or m.group(1) != source_hash():
        return None
    return int(t.group(1))


WORKLOADS = {
    # name: (B, I, N, k, O)
    "dwn_k6_b4096_i16384_n8192": (4096, 16384, 8192, 6, 1),   # the configuration the metric is quoted on
    "dwn_small": (256, 3136, 2000, 6, 1),
    # secondary workloads of the same path, reported with their own metric names (see run_secondary)
    "prob_k4_b1024_i4096_n4096": (1024, 4096, 4096, 4, 1),
    "softmap_b512_i3136_m48000": (512, 3136, 8000, 6, 1),
    # the whole layer of that configuration through the layer API: soft connectivity feeding 8000 DWN nodes
    "learnable_layer_b512_i3136_n8000": (512, 3136, 8000, 6, 1),
    # the headline layer shape with the two other table-lookup node types
    "stable_k6_b4096_i16384_n8192": (4096, 16384, 8192, 6, 1),
    "hybrid_k6_b4096_i16384_n8192": (4096, 16384, 8192, 6, 1),
    # convolutional LUT layer through the layer API: (images, in_channels, out_channels, k, O); 28x28 images,
    # receptive field 5, trees of depth 2
    "conv_b256_c4_28x28_o32_rf5_d2": (256, 4, 32, 6, 1),
    # whole training step of the deep stack through the layer API: (B, features, first layer width, k, O)
    "dwn_stack_b8192_train_step": (8192, 784, 16000, 6, 1),
    # the same model in eval mode (inference): thermometer code and activations as bit-planes, GroupSum as a count
    "dwn_stack_b8192_eval_forward": (8192, 784, 16000, 6, 1),
}


def algorithmic_bytes(B, I, N, k, O):
    """fp32 storage as the configuration states it; addresses recomputed in backward, nothing else
    re-read.  Returns the per-kernel split used for the dominant-kernel roofline and the step total."""
    L = 1 << k
    x, y, tables, mapping = B * I * 4, B * N * O * 4, N * O * L * 4, N * k * 2
    fwd = x + y + tables + mapping
    bwd = y + x + tables + tables + x + mapping  # gy, x again, tables, table grads, gx, map
    per_kernel = {
        "dwn_pack_planes": x,                         # reads every input once
        "dwn_lookup_fwd": y + tables + mapping,       # writes every output once
        "dwn_bwd_transpose_hist": y + tables,         # reads gy once, reads the tables (its launch builds the coefficients)
        "dwn_bwd_gx": x + tables + mapping,           # writes every input gradient once and the table gradients
    }
    return fwd, bwd, per_kernel


def stack_bytes(B, F, nbits, widths, k, train):
    """HBM bytes the chained bit-plane formulation has to move for one batch (a lower bound for THESE kernels, so the
    fraction of the roofline cannot exceed 1): raw features in; every layer's input once written and once read as
    bit-planes (1 bit per value); tables read; logits.  Training adds: the saved address of every (node, row), one
    byte, written forward and read by the histogram and by the gather; the fp32 gradient with respect to every hidden
    activation, written once in tile-major form and read once (the gather that reads it also fills the histogram of the
    layer in front); the gradient of the logits; and nine passes over the tables in all (forward, backward, gradient,
    Adam read p/g/m/v, write p/m/v)."""
    ins = [F * nbits] + widths[:-1]
    tables = sum(widths) * (1 << k) * 4
    planes = sum(ins) * B // 8
    nbytes = B * F * 4 + 2 * planes + tables + B * 10 * 4
    if train:
        nbytes += 3 * B * sum(widths)                   # saved addresses: written, read twice
        nbytes += 2 * 4 * B * sum(widths[:-1])          # hidden-activation gradients: written, read once
        nbytes += 2 * B * 10 * 4 + 8 * tables
    return nbytes


PRERUN_MS = 60.0
PRERUN_MAX_MS = 800.0


def steady_state(step, ms=PRERUN_MS, max_ms=PRERUN_MAX_MS, chunk=8):
    """Brings device and host to their sustained state before anything is timed.  After an idle phase (the setup above
    every timed loop is mostly host work) the first ~60 steps of the headline workload run up to 14 % slower (0.337 ms
    against 0.295 ms per step, settled after about 20 ms), and the first ~200 steps of a freshly built layer object
    through autograd and torch's allocator read 9 % slower than all later ones.  The step is run, untimed, in chunks
    of `chunk` for at least `ms` milliseconds and until the last three chunks agree within 1 % with each other and with
    the fastest chunk so far (at most `max_ms`); the warm-up steps asked for on the command line and the timed steps
    follow without a pause.  Returns the number of steps run."""
    torch.cuda.synchronize()
    t_begin = time.perf_counter()
    times = []
    while True:
        t0 = time.perf_counter()
        for _ in range(chunk):
            step()
        torch.cuda.synchronize()
        now = time.perf_counter()
        times.append(now - t0)
        elapsed = (now - t_begin) * 1e3
        if elapsed >= max_ms:
            break
        if elapsed >= ms and len(times) >= 4:
            last = times[-3:]
            if max(last) <= 1.01 * min(last) and max(last) <= 1.01 * min(times):
                break
    return chunk * len(times)


WINDOWS = 5


def timed_windows(step, steps, windows=WINDOWS):
    """`windows` back-to-back timed regions of exactly `steps` steps, each bracketed by a device synchronisation on both
    sides: milliseconds per step of every window.  The reported figure is the median window; minimum and maximum go
    into the line as well, so that the spread of one run is visible (boxes of the pool differ by several per cent)."""
    out = []
    for _ in range(windows):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        out.append((time.perf_counter() - t0) * 1e3 / steps)
    return out


def window_summary(per_window):
    return {"count": len(per_window), "steps_each": None, "median_ms": float(np.median(per_window)),
            "min_ms": float(min(per_window)), "max_ms": float(max(per_window))}


def time_steps(step, steps, warmup):
    steady_state(step)
    for _ in range(warmup):
        step()
    return float(np.median(timed_windows(step, steps)))


def kernel_times(step, reps):
    from difflut_amd import _native as nat
    nat.profile_enable(True)
    per = {}
    for _ in range(reps):
        step()
        for name, ms in nat.profile_read():
            per.setdefault(name, []).append(ms)
    nat.profile_enable(False)
    return {name: float(np.mean(v)) for name, v in per.items()}


def run_stack(args):
    """Thermometer(4) -> RandomLayer+DWN k=6 with 16000 -> 8000 -> 4000 -> 2000 nodes -> GroupSum(10) ->
    cross-entropy, backward, Adam on the tables: the reference's layer API end to end, one step per batch."""
    from difflut_amd import REGISTRY
    from difflut_amd import _native as nat
    from difflut_amd.nodes.node_config import NodeConfig
    from difflut_amd.utils import GroupSum, cross_entropy

    dev = torch.device("cuda:0")
    B, F, _, k, O = WORKLOADS[args.workload]
    widths = [16000, 8000, 4000, 2000]
    torch.manual_seed(0)
    x = torch.rand(B, F, device=dev)
    labels = torch.randint(0, 10, (B,), device=dev)
    enc = REGISTRY.build_encoder("thermometer", num_bits=4).fit(x)
    layers, width = [], F * 4
    for n in widths:
        layers.append(REGISTRY.get_layer("random")(width, n, REGISTRY.get_node("dwn"),
                                                   NodeConfig(input_dim=k, output_dim=O), seed=42).to(dev))
        width = n * O
    head = GroupSum(k=10, tau=1.0, use_randperm=False)
    params = [p for layer in layers for p in layer.bank_parameters()]
    from difflut_amd.utils import BankAdam
    opt = BankAdam(params, lr=1e-3)  # torch.optim.Adam's arithmetic, one launch of the library for the four table banks
    from difflut_amd.layers import DWNStack
    # same layers; thermometer code and activations as bit-planes, tile-major gradients between layers
    stack = DWNStack(layers, encoder=enc, head=head).train()

    if args.workload.endswith("eval_forward"):
        stack.eval()
        for layer in layers:
            layer.eval()

        def infer():
            with torch.no_grad():
                if args.layer_by_layer:
                    h = enc.encode(x)
                    for layer in layers:
                        h = layer(h)
                    return head(h)
                return stack(x)

        ms = time_steps(infer, args.steps, args.warmup)
        evals = B * sum(widths)
        nbytes = stack_bytes(B, F, 4, widths, k, train=False)
        out = {"metric": "LUT-node evals/sec, inference (thermometer -> 4 DWN k=6 layers -> GroupSum)",
               "value": evals / (ms * 1e-3), "unit": "node-evals/s", "ms_per_step": ms, "dtype": "f32 tables, 1-bit activations",
               "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
               "vs_baseline": None, "data": "synthetic",
               "config": {"workload": args.workload, "batch": B, "features": F, "layers": widths, "k": k,
                          "execution": "layer by layer" if args.layer_by_layer else "chained (DWNStack)"},
               "roofline_step": {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                 "algorithmic_bytes_per_step": nbytes,
                                 "note": "bytes of the bit-plane formulation (features, 1-bit activations written and read, "
                                         "tables, logits); the kernels are bound by L2 gather latency, not by HBM"},
               "kernel_ms": kernel_times(infer, min(args.steps, 5))}
        return out

    def step():
        opt.zero_grad(set_to_none=True)
        if args.layer_by_layer:
            h = enc.encode(x)
            for layer in layers:
                h = layer(h)
            logits = head(h)
        else:
            logits = stack(x)  # the last layer sums per group itself
        loss = cross_entropy(logits, labels)  # one pass for the loss and its gradient (same values as torch's)
        loss.backward()
        opt.step()

    ms = time_steps(step, args.steps, args.warmup)
    evals = B * sum(widths)
    if args.layer_by_layer:
        # fp32 traffic of the layer-by-layer formulation: per layer x and y forward, gy, x and gx backward (no gx for
        # the first layer), plus nine passes over the tables (forward, backward, gradient, Adam)
        ins = [F * 4] + widths[:-1]
        nbytes = sum(4 * B * (2 * i + 2 * n + (i if li else 0)) for li, (i, n) in enumerate(zip(ins, widths)))
        nbytes += 9 * sum(widths) * (1 << k) * 4
    else:
        nbytes = stack_bytes(B, F, 4, widths, k, train=True)
    out = {"metric": "LUT-node evals/sec, training step (thermometer -> 4 DWN k=6 layers -> GroupSum -> CE, Adam)",
           "value": evals / (ms * 1e-3), "unit": "node-evals/s", "ms_per_step": ms, "dtype": "f32",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "data": "synthetic",
           "config": {"workload": args.workload, "batch": B, "features": F, "layers": widths, "k": k, "optimizer": "difflut_amd.utils.BankAdam (Adam, one launch over the table banks)",
                      "execution": "layer by layer" if args.layer_by_layer else "chained (DWNStack)"},
           "roofline_step": {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes_per_step": nbytes},
           "kernel_ms": kernel_times(step, min(args.steps, 5))}
    return out


def run_conv(args):
    """ConvolutionalLayer (DWN nodes, trees of depth 2 over 5x5x4 patches of 28x28 images): forward and backward
    including the input gradient, through the module API."""
    from difflut_amd import REGISTRY
    from difflut_amd.layers import ConvolutionConfig
    from difflut_amd.nodes.node_config import NodeConfig

    dev = torch.device("cuda:0")
    B, C, T, k, O = WORKLOADS[args.workload]
    H = W = 28
    rf, depth = 5, 2
    torch.manual_seed(0)
    cfg = ConvolutionConfig(tree_depth=depth, in_channels=C, out_channels=T, receptive_field=rf, stride=1, padding=0,
                            chunk_size=32, seed=42)
    layer = REGISTRY.get_convolutional_layer("convolutional")(
        convolution_config=cfg, node_type=REGISTRY.get_node("dwn"), node_kwargs=NodeConfig(input_dim=k, output_dim=O),
        layer_type=REGISTRY.get_layer("random"), n_inputs_per_node=k).to(dev).train()
    x = torch.bernoulli(torch.full((B, C, H, W), 0.5, device=dev)).requires_grad_()
    out = H - rf + 1
    gy = torch.randn(B, T, out, out, device=dev)
    banks = layer.bank_parameters()

    def step():
        x.grad = None
        for t in banks:
            t.grad = None
        layer(x).backward(gy)

    ms = time_steps(step, args.steps, args.warmup)
    rows = B * out * out
    nodes = sum(layer.hidden_layers) * T
    out_d = {"metric": "LUT-node evals/sec fwd+bwd (ConvolutionalLayer, DWN k=6 trees of depth 2, 32 channels, 5x5x4 patches)",
             "value": rows * nodes / (ms * 1e-3), "unit": "node-evals/s", "ms_per_step": ms, "dtype": "f32",
             "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
             "vs_baseline": None, "data": "synthetic",
             "config": {"workload": args.workload, "images": B, "in_channels": C, "out_channels": T, "image": [H, W],
                        "receptive_field": rf, "tree_depth": depth, "patch_rows": rows, "nodes": nodes},
             # no roofline fraction: image and output are a few MB, the step is bound by the first level's input
             # gradient (6912 connections onto 100 inputs: lane reads and L2 gathers), see profiles/
             "kernel_ms": kernel_times(step, min(args.steps, 5))}
    return out_d


def run_learnable(args):
    """LearnableLayer (soft connectivity over 3136 inputs -> 8000 DWN nodes with k=6): forward and backward with the
    input, mapping-weight and table gradients, through the module API."""
    from difflut_amd import REGISTRY
    from difflut_amd.nodes.node_config import NodeConfig

    dev = torch.device("cuda:0")
    B, I, N, k, O = WORKLOADS[args.workload]
    torch.manual_seed(0)
    layer = REGISTRY.get_layer("learnable")(I, N, REGISTRY.get_node("dwn"), NodeConfig(input_dim=k, output_dim=O),
                                            tau=1.0, tau_start=1.0, tau_min=1e-4, tau_decay_iters=1000,
                                            use_cuda_soft=False).to(dev).train()
    layer.mapping.precision = args.precision  # 0: fp32 matrix cores, 1: bf16 operands with fp32 accumulation
    with torch.no_grad():
        layer.mapping.W.normal_(0, 0.01)
    x = torch.rand(B, I, device=dev, requires_grad=True)
    gy = torch.randn(B, N * O, device=dev)
    W = layer.mapping.W
    banks = layer.bank_parameters()

    def step():
        x.grad = None
        W.grad = None
        for t in banks:
            t.grad = None
        layer(x).backward(gy)

    ms = time_steps(step, args.steps, args.warmup)
    M = N * k
    flops = 3 * 2 * B * I * M
    peak = 157.3 if args.precision == 0 else 2500.0
    out = {"metric": "LUT-node evals/sec fwd+bwd (LearnableLayer soft connectivity 3136 -> 8000 DWN k=6 nodes, B=512)",
           "value": B * N / (ms * 1e-3), "unit": "node-evals/s", "ms_per_step": ms,
           "dtype": "f32" if args.precision == 0 else "bf16 operands, f32 accumulate (soft connectivity); f32 elsewhere",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "data": "synthetic",
           "config": {"workload": args.workload, "batch": B, "inputs": I, "nodes": N, "k": k, "mapping_rows": M,
                      "precision": args.precision},
           "roofline_step": {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": peak, "unit": "TFLOP/s",
                             "frac": flops / (ms * 1e-3) / 1e12 / peak, "algorithmic_flops_per_step": flops},
           "kernel_ms": kernel_times(step, min(args.steps, 5))}
    return out


def maybe_graph(step, args):
    """With --graph: the step's launches captured once (after warm-up, on a side stream as torch requires) and
    replayed; the library never allocates, synchronises or uses memset nodes, so a step is capturable as it is."""
    if not getattr(args, "graph", False):
        return step
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    return graph.replay


def run_secondary(args):
    """Probabilistic layer (k=4, 1024 x 4096 -> 4096 nodes), DWN-stable and hybrid layers at the headline shape, and
    soft connectivity (512 x 3136 -> 48000 rows), all through the C ABI."""
    from difflut_amd import _native as nat
    from difflut_amd import ops
    from difflut_amd.layers.random_layer import draw_mapping

    lib = nat.lib()
    dev = torch.device("cuda:0")
    B, I, N, k, O = WORKLOADS[args.workload]
    torch.manual_seed(0)
    if args.workload.startswith("prob"):
        dims = (B, I, N, k, O)
        x = torch.sigmoid(torch.randn(B, I, device=dev))
        plan = ops.MappingPlan(draw_mapping(I, N, k, seed=42).to(dev), I)
        raw = torch.rand(N, 1 << k, O, device=dev)
        gy = torch.randn(B, N * O, device=dev)
        y = torch.empty(B, N * O, device=dev); gx = torch.empty(B, I, device=dev); graw = torch.empty_like(raw)
        ws = torch.empty(max(lib.dl_prob_bwd_workspace_bytes(*dims), 256), dtype=torch.uint8, device=dev)
        saved = torch.empty(max(lib.dl_prob_saved_bytes(*dims), 256), dtype=torch.uint8, device=dev)

        def step():
            nat.check(lib.dl_prob_layer_fwd(x.data_ptr(), plan.idx32.data_ptr(), raw.data_ptr(), 1.0, y.data_ptr(),
                                            saved.data_ptr(), saved.numel(), *dims, nat.stream()))
            nat.check(lib.dl_prob_layer_bwd(x.data_ptr(), saved.data_ptr(), plan.idx32.data_ptr(), plan.inv_ptr.data_ptr(),
                                            plan.inv_pos.data_ptr(), raw.data_ptr(), 1.0, gy.data_ptr(), gx.data_ptr(),
                                            graw.data_ptr(), ws.data_ptr(), ws.numel(), *dims, nat.stream()))

        ms = time_steps(maybe_graph(step, args), args.steps, args.warmup)
        nbytes = 5 * B * I * 4 + 3 * N * (1 << k) * O * 4 + 2 * N * k * 2  # x, y, gy, x again, gx; tables r, r, grad
        flops = 320 * B * N
        out = {"metric": "LUT-node evals/sec fwd+bwd (Probabilistic k=4, B=1024, 4096 nodes)", "value": B * N / (ms * 1e-3),
               "unit": "node-evals/s", "ms_per_step": ms, "dtype": "f32",
               "roofline_step": {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                                 "unit": "GB/s", "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                 "algorithmic_bytes_per_step": nbytes},
               "valu": {"achieved_tflops": flops / (ms * 1e-3) / 1e12, "peak_tflops": 157.3}}
    elif args.workload.startswith(("stable", "hybrid")):
        stable = args.workload.startswith("stable")
        dims = (B, I, N, k, O)
        count = N * O * (1 << k)
        x = torch.rand(B, I, device=dev)  # real-valued: the hybrid backward differentiates at x itself
        plan = ops.MappingPlan(draw_mapping(I, N, k, seed=42).to(dev), I)
        raw = torch.randn(N, O, 1 << k, device=dev)
        scale = torch.full((N,), 1.25, device=dev)
        gy = torch.randn(B, N * O, device=dev)
        luts = torch.empty_like(raw); gl = torch.empty_like(raw); graw = torch.empty_like(raw)
        y = torch.empty(B, N * O, device=dev); gx = torch.empty(B, I, device=dev)
        saved = torch.empty(lib.dl_dwn_saved_bytes(*dims), dtype=torch.uint8, device=dev)
        ws = torch.empty(max(lib.dl_dwn_fwd_workspace_bytes(*dims), lib.dl_dwn_bwd_workspace_bytes(*dims),
                             lib.dl_hybrid_bwd_workspace_bytes(*dims)), dtype=torch.uint8, device=dev)

        def step():
            nat.check(lib.dl_table_sigmoid_fwd(raw.data_ptr(), luts.data_ptr(), count, nat.stream()))
            nat.check(lib.dl_dwn_layer_fwd(x.data_ptr(), plan.idx32.data_ptr(), luts.data_ptr(), y.data_ptr(),
                                           saved.data_ptr(), ws.data_ptr(), ws.numel(), *dims, nat.stream()))
            if stable:
                nat.check(lib.dl_dwn_stable_layer_bwd(None, saved.data_ptr(), plan.idx32.data_ptr(), plan.inv_ptr.data_ptr(),
                                                      plan.inv_pos.data_ptr(), luts.data_ptr(), gy.data_ptr(),
                                                      scale.data_ptr(), gx.data_ptr(), gl.data_ptr(), ws.data_ptr(),
                                                      ws.numel(), *dims, nat.stream()))
            else:
                nat.check(lib.dl_hybrid_layer_bwd(x.data_ptr(), plan.idx32.data_ptr(), plan.inv_ptr.data_ptr(),
                                                  plan.inv_pos.data_ptr(), luts.data_ptr(), gy.data_ptr(), gx.data_ptr(),
                                                  gl.data_ptr(), ws.data_ptr(), ws.numel(), *dims, nat.stream()))
            nat.check(lib.dl_table_sigmoid_bwd(gl.data_ptr(), luts.data_ptr(), graw.data_ptr(), count, nat.stream()))

        ms = time_steps(maybe_graph(step, args), args.steps, args.warmup)
        fwd_b, bwd_b, _ = algorithmic_bytes(B, I, N, k, O)  # same tensors cross HBM as for the DWN node
        nbytes = fwd_b + bwd_b
        name = "DWN-stable" if stable else "hybrid"
        out = {"metric": f"LUT-node evals/sec fwd+bwd ({name} k=6, B=4096, 8192 nodes)", "value": B * N / (ms * 1e-3),
               "unit": "node-evals/s", "ms_per_step": ms, "dtype": "f32",
               "roofline_step": {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                                 "unit": "GB/s", "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                 "algorithmic_bytes_per_step": nbytes}}
    else:
        M = N * k
        precision = args.precision
        x = torch.rand(B, I, device=dev)
        W = torch.randn(M, I, device=dev) * 0.01
        gm = torch.randn(B, M, device=dev)
        m = torch.empty(B, M, device=dev); stats = torch.empty(max(lib.dl_soft_map_saved_bytes(B, I, M, precision), 256), dtype=torch.uint8, device=dev)
        gx = torch.empty_like(x); gW = torch.empty_like(W)
        ws = torch.empty(max(lib.dl_soft_map_workspace_bytes(B, I, M, precision), 256), dtype=torch.uint8, device=dev)

        def step():
            nat.check(lib.dl_soft_map_fwd(x.data_ptr(), W.data_ptr(), 1.0, m.data_ptr(), stats.data_ptr(), ws.data_ptr(),
                                          ws.numel(), B, I, M, precision, nat.stream()))
            nat.check(lib.dl_soft_map_bwd(x.data_ptr(), W.data_ptr(), 1.0, m.data_ptr(), stats.data_ptr(), gm.data_ptr(),
                                          gx.data_ptr(), gW.data_ptr(), ws.data_ptr(), ws.numel(), B, I, M, precision,
                                          nat.stream()))

        ms = time_steps(maybe_graph(step, args), args.steps, args.warmup)
        flops = 3 * 2.0 * B * I * M
        peak = 157.3 if precision == 0 else 2500.0
        out = {"metric": "soft-connectivity contraction fwd+bwd (x[512,3136] . softmax(W[48000,3136])^T)",
               "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_step": ms,
               "dtype": "f32" if precision == 0 else "bf16",
               "roofline_step": {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": peak, "unit": "TFLOP/s",
                                 "frac": flops / (ms * 1e-3) / 1e12 / peak, "algorithmic_flops_per_step": flops}}
    out.update({"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
                "vs_baseline": None, "data": "synthetic",
                "config": {"workload": args.workload, "launch": "hip graph replay" if args.graph else "direct"},
                "kernel_ms": kernel_times(step, min(args.steps, 10))})
    return out


def layer_api_step(args, x, gy, idx, luts):
    """forward + backward of the headline layer through RandomLayer / DWNNode modules and autograd."""
    from difflut_amd import REGISTRY
    from difflut_amd.nodes.node_config import NodeConfig
    B, I, N, k, O = WORKLOADS[args.workload]
    layer = REGISTRY.get_layer("random")(I, N, REGISTRY.get_node("dwn"), NodeConfig(input_dim=k, output_dim=O), seed=42,
                                         mapping_indices=idx).to(x.device).train()
    bank = layer.bank_parameters()[0]
    with torch.no_grad():
        bank.copy_(luts)
    xg = x.clone().requires_grad_()

    def step():
        xg.grad = None
        bank.grad = None
        layer(xg).backward(gy)

    ms = time_steps(step, args.steps, args.warmup)
    fwd_b, bwd_b, _ = algorithmic_bytes(B, I, N, k, O)
    gbs = (fwd_b + bwd_b) / (ms * 1e-3) / 1e9
    return {"ms_per_step": ms, "value": B * N / (ms * 1e-3), "unit": "node-evals/s",
            "call": "RandomLayer(...).forward(x).backward(gy), tensors allocated per call by torch's caching allocator",
            "roofline_step": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                              "algorithmic_bytes_per_step": fwd_b + bwd_b}}


def secondary_configs(args):
    """The other benchmark configurations, a few steps each, after the headline's timed region: the probabilistic layer,
    the LearnableLayer with fp32 and with bf16 soft connectivity, and the deep-stack training step.  Each entry carries
    its own metric, time per step and a roofline fraction against the bytes or flops its formulation has to move."""
    import copy
    import gc
    res = {}
    plan = [("prob_k4_b1024_i4096_n4096", {}), ("learnable_layer_b512_i3136_n8000", {"precision": 0}),
            ("learnable_layer_b512_i3136_n8000", {"precision": 1}), ("dwn_stack_b8192_train_step", {})]
    for workload, extra in plan:
        sub = copy.copy(args)
        sub.workload, sub.steps, sub.warmup, sub.graph, sub.layer_by_layer = workload, min(args.steps, 10), 3, False, False
        for key, value in extra.items():
            setattr(sub, key, value)
        gc.collect()
        torch.cuda.empty_cache()
        r = dispatch_other(sub)
        name = workload + ("_bf16" if extra.get("precision") == 1 else "")
        res[name] = {key: r[key] for key in ("metric", "value", "unit", "ms_per_step", "dtype", "roofline_step") if key in r}
    return res


def dispatch_other(args):
    """Every workload but the headline one: its result line as a dict (None for the headline)."""
    if args.workload.startswith("dwn_stack"):
        return run_stack(args)
    if args.workload.startswith("conv"):
        return run_conv(args)
    if args.workload.startswith("learnable"):
        return run_learnable(args)
    if not args.workload.startswith("dwn"):
        return run_secondary(args)
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="dwn_k6_b4096_i16384_n8192", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=4096, help="batch rows of the workload the CPU baseline runs")
    ap.add_argument("--precision", type=int, default=0, help="soft-connectivity workload: 0 fp32, 1 bf16 operands")
    ap.add_argument("--layer-by-layer", action="store_true", help="stack workload: call the layers one by one")
    ap.add_argument("--no-secondary", action="store_true",
                    help="default workload: skip the other benchmark configurations reported under 'secondary'")
    ap.add_argument("--graph", action="store_true",
                    help="C-ABI workloads other than the default: replay the step from a captured HIP graph")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no collective); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    from difflut_amd import _native as nat
    from difflut_amd import ops
    from difflut_amd.layers.random_layer import draw_mapping

    lib = nat.lib()  # raises if the HIP library has not been built
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a ROCm device")
    other = dispatch_other(args)
    if other is not None:
        print(json.dumps(other))
        return
    dev = torch.device("cuda:0")
    B, I, N, k, O = WORKLOADS[args.workload]
    dims = (B, I, N, k, O)
    torch.manual_seed(0)
    x = torch.bernoulli(torch.full((B, I), 0.5, device=dev))
    idx = draw_mapping(I, N, k, seed=42)  # the table RandomLayer(seed=42) registers
    plan = ops.MappingPlan(idx.to(dev), I)
    luts = torch.rand(N, O, 1 << k, device=dev) * 2 - 1
    gy = torch.randn(B, N * O, device=dev)
    alpha, beta = float(np.float32(0.5 * 0.75 ** (k - 1))), float(np.float32(1.0 / 3.0))

    y = torch.empty(B, N * O, device=dev)
    gx = torch.empty(B, I, device=dev)
    gl = torch.empty_like(luts)
    saved = torch.empty(lib.dl_dwn_saved_bytes(*dims), dtype=torch.uint8, device=dev)
    ws_f = torch.empty(lib.dl_dwn_fwd_workspace_bytes(*dims), dtype=torch.uint8, device=dev)
    ws_b = torch.empty(lib.dl_dwn_bwd_workspace_bytes(*dims), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        nat.check(lib.dl_dwn_layer_fwd(x.data_ptr(), plan.idx32.data_ptr(), luts.data_ptr(), y.data_ptr(),
                                       saved.data_ptr(), ws_f.data_ptr(), ws_f.numel(), *dims, stream))
        nat.check(lib.dl_dwn_layer_bwd(None, saved.data_ptr(), plan.idx32.data_ptr(), plan.inv_ptr.data_ptr(),
                                       plan.inv_pos.data_ptr(), luts.data_ptr(), gy.data_ptr(), alpha, beta,
                                       gx.data_ptr(), gl.data_ptr(), ws_b.data_ptr(), ws_b.numel(), *dims, stream))

    prerun_steps = steady_state(step)  # untimed: sustained clocks (see steady_state)
    for _ in range(args.warmup):
        step()
    per_window = timed_windows(step, args.steps)  # WINDOWS regions of exactly --steps steps, each between two syncs
    ms_per_step = float(np.median(per_window))
    evals = B * N

    # per-kernel durations: HIP events recorded by the library around each launch, same stream
    nat.profile_enable(True)
    per = {}
    prof_steps = min(args.steps, 20)
    for _ in range(prof_steps):
        step()
        for name, ms in nat.profile_read():
            per.setdefault(name, []).append(ms)
    nat.profile_enable(False)
    avg = {name: float(np.mean(v)) for name, v in per.items()}
    fwd_b, bwd_b, split = algorithmic_bytes(*dims)
    dominant = max(avg, key=avg.get)
    dom_gbs = split[dominant] / (avg[dominant] * 1e-3) / 1e9
    step_gbs = (fwd_b + bwd_b) / (ms_per_step * 1e-3) / 1e9

    out = {
        "metric": "LUT-node evals/sec fwd+bwd (DWN k=6, B=4096, 8192 nodes); % HBM roofline",
        "value": evals / (ms_per_step * 1e-3),
        "unit": "node-evals/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "timed_windows": dict(window_summary(per_window), steps_each=args.steps,
                              note="ms_per_step is the median window; every window is exactly --steps steps between two "
                                   "device synchronisations"),
        "steady_state_prerun": {"min_ms": PRERUN_MS, "max_ms": PRERUN_MAX_MS, "steps": prerun_steps,
                                "why": "untimed steps before the warm-up, until chunks of 8 steps agree within 1 %: "
                                       "device clocks settle about 20 ms after idle"},
        "config": {"workload": args.workload, "batch": B, "inputs": I, "nodes": N, "k": k, "output_dim": O,
                   "pass": "forward + EFD backward (input and table gradients)", "seed": 0, "mapping_seed": 42},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": dom_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": dom_gbs / HBM_PEAK_GBS, "traffic": measured_traffic(args.workload, dominant),
                     "algorithmic_bytes_per_launch": split[dominant],
                     "avg_launch_ms": avg[dominant]},
        "roofline_step": {"bound": "hbm", "achieved": step_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": step_gbs / HBM_PEAK_GBS, "algorithmic_bytes_per_step": fwd_b + bwd_b},
        "kernel_ms": avg,
    }

    # the same step through the layer API (what a user of the reference calls): RandomLayer.forward allocates its
    # output, saved addresses and workspaces per call and goes through autograd
    y_host = y[:min(B, args.cpu_rows)].cpu().numpy()  # for the check of the CPU baseline's output below
    del y, gx, gl, saved, ws_f, ws_b
    out["layer_api"] = layer_api_step(args, x, gy, idx, luts)
    if not args.no_secondary and args.workload == "dwn_k6_b4096_i16384_n8192":
        out["secondary"] = secondary_configs(args)

    if not args.no_cpu_baseline:
        from oracle import c_oracle
        rows = min(B, args.cpu_rows)
        xs = x[:rows].cpu().numpy()
        ls = luts.cpu().numpy()
        gs = gy[:rows].cpu().numpy().reshape(rows, N, O)
        idn = idx.numpy()
        cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        c_oracle.lib()
        t0 = time.perf_counter()
        yc = c_oracle.dwn_layer_forward(xs, idn, ls)
        c_oracle.dwn_layer_backward(xs, idn, ls, gs, alpha, beta)
        cpu_s = time.perf_counter() - t0
        assert np.array_equal(yc.reshape(rows, -1), y_host)  # the checker, not the measured thing
        out["cpu_baseline"] = {"value": rows * N / cpu_s, "unit": "node-evals/s", "cores": cores, "kind": "port",
                               "sample": f"first {rows} of {B} batch rows, all {N} nodes, forward+backward, "
                                         f"{cpu_s:.2f} s wall"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
