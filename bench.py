#!/usr/bin/env python3
"""Benchmark of the packed on-the-fly quantized-linear hot path on one MI355X.

Workload (the headline configuration): the 48 packed linears of DeiT-Small (12 blocks x qkv 384->1152,
proj 384->384, fc1 384->1536, fc2 1536->384), W4A4, group size 64, fp16 activations in and out,
batch 64 (M = 64*197 = 12608 tokens).  One step = one pass over all 48 layers through
arcq_linear_otf_ws with both scratch workspaces lent; at this batch every DeiT-S (and DeiT-B) layer runs as ONE
launch (otf_rows_kernel / otf_rows_phased_kernel: stage 1 into LDS, the fp16 weights reconstructed cooperatively
into the workspace, fp16 MFMA GEMM + bias), ViT-L's as two (stage 1 into the block layout with the weight
reconstruction carried along, then a weight-stationary GEMM).  Inputs (one synthetic activation tensor per layer
shape, packed weights of 48 distinct random layers) are resident in HBM before the timed region starts.

Prints ONE JSON line.  ``value`` is images/s of that step (packed linears only, on fixed inputs: no attention,
LayerNorm or GELU; ``model_forward`` times the whole skeleton model next to it and ``bs1.chained`` /
``detail.chained`` the linears as a dependency chain).  ``roofline`` is for the dominant kernel of the step --
the one with the largest share of its time; for DeiT-S that is a whole-layer kernel, so its duration includes
stage 1 and the weight reconstruction: algorithmic flops (2*M*N*K) of its launches divided by their time alone,
measured here with HIP events on the launch stream in a graph of only these launches; ``roofline.layer`` is the
whole step against the same peaks; ``roofline.weights_rebuilt_inside_gemm`` the variant that dequantizes inside
the GEMM.  ``other_configs`` times the other BASELINE configurations (DeiT-B W4A4 batch 64, ViT-L W3A3 batch
256) briefly in the same run, each with its own whole-step roofline.  ``cpu_baseline`` times the oracle's
restatement of the reference's fake-quant CPU path (quantize + reconstruct activation and weight, fp32 matmul)
on a bounded sample on this host.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
PROFILE_NAMES = {("deit_small", 4, 64): "deit_small_w4a4_bs64_packed_linears.md",
                 ("deit_base", 4, 64): "deit_base_w4a4_bs64_packed_linears.md",
                 ("vit_large", 3, 256): "vit_large_w3a3_bs256_packed_linears.md"}


def profiled_traffic(model, bits, batch, kernel):
    """HBM bytes per launch of `kernel` (average over the layer shapes it serves) as the committed rocprofv3 summary
    of this workload states it: two --pmc runs (FETCH_SIZE, WRITE_SIZE) scaled by what the same counters read for a
    plain 256 MiB copy.  The summary holds one line `traffic_bytes_per_launch[<kernel>] = <bytes>` per kernel; None
    when there is no summary or no such line."""
    import re
    name = PROFILE_NAMES.get((model, bits, batch))
    if not name:
        return None
    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None
    m = re.search(r"traffic_bytes_per_launch\[" + re.escape(kernel) + r"\]\s*=\s*([0-9.eE+]+)", text)
    return float(m.group(1)) if m else None


def traffic_source(model, bits, batch):
    """Where `roofline.traffic` comes from: the committed profile's file name and the digest of the kernel sources it
    was taken with (the summary records `kernel_sources_sha16 = ...`); `stale` says that the sources have changed
    since, i.e. that the figure describes an older build of the kernel."""
    import re
    name = PROFILE_NAMES.get((model, bits, batch))
    if not name:
        return None
    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None
    m = re.search(r"kernel_sources_sha16\s*=\s*([0-9a-f]+)", text)
    now = kernel_sources_sha16()
    return {"file": "profiles/" + name, "measured_live": False, "kernel_sources_sha16_of_profile": m.group(1) if m else None,
            "kernel_sources_sha16_now": now, "stale": (m.group(1) != now) if m else None}


def kernel_sources_sha16():
    """First 16 hex digits of the SHA-256 over the library's kernel sources (csrc/*.hip, csrc/*.h, in name order)."""
    import glob
    import hashlib
    h = hashlib.sha256()
    for f in sorted(glob.glob(os.path.join(ROOT, "arcq-vit_amd", "csrc", "*.hip")) + glob.glob(os.path.join(ROOT, "arcq-vit_amd", "csrc", "*.h"))):
        h.update(open(f, "rb").read())
    return h.hexdigest()[:16]


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--model", default="deit_small")
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-bs1", action="store_true")
    ap.add_argument("--no-model", action="store_true", help="skip the model_forward block (whole ViT forward)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of the other BASELINE configurations (default run only)")
    ap.add_argument("--fp8", action="store_true",
                    help="also time the same step with FP8 operands (ops.linear_otf_fp8: not the reference's numerics; "
                         "reported in a block of its own, never as `value`)")
    ap.add_argument("--eager", action="store_true",
                    help="launch every kernel from Python instead of replaying one HIP graph per step")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (reference point for rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE)")
    return ap.parse_args()


class Layer:
    """Device buffers of one packed layer plus the raw C-ABI argument lists for a fixed M."""

    def __init__(self, name, k, n, bits, seed, dev):
        import torch
        from arcq_vit_amd import synth
        from arcq_vit_amd.packed_linear import _quantize_weight_reference
        from arcq_vit_amd.pack_py import pack_codes_py
        cb = synth.quantile_codebook(bits)
        thr = synth.midpoint_thresholds(cb)
        w = synth.make_weight(n, k, seed)
        codes, center, scale, code_sum = _quantize_weight_reference(w, thr, cb, 64, 1e-6)
        self.name, self.k, self.n, self.bits = name, k, n, bits
        self.packed = pack_codes_py(codes, bits).to(dev)
        self.cb, self.thr = cb.to(dev), thr.to(dev)
        self.center, self.scale, self.code_sum = center.to(dev), scale.to(dev), code_sum.to(dev)
        self.bias = synth.make_bias(n, seed).to(dev)
        self.w_fp32 = w  # CPU, for the CPU baseline only

    def clone_weights(self):
        """A second copy of the layer's device buffers (distinct addresses), for the cold-cache measurement."""
        import copy
        c = copy.copy(self)
        for name in ("packed", "cb", "thr", "center", "scale", "code_sum", "bias"):
            setattr(c, name, getattr(self, name).clone())
        return c

    # Argument lists of arcq_linear_otf_ws / arcq_linear_fused_ws.  W_WS is one fp16 scratch buffer for the
    # reconstructed weights, shared by all layers (they run back to back on one stream).
    W_WS = None

    def otf_args(self, x, ws, y, stream):
        from arcq_vit_amd._lib import ARCQ_F16
        m = x.shape[0]
        return (x.data_ptr(), ARCQ_F16, self.thr.data_ptr(), self.cb.data_ptr(), self.packed.data_ptr(),
                self.cb.data_ptr(), self.center.data_ptr(), self.scale.data_ptr(), self.code_sum.data_ptr(),
                self.bias.data_ptr(), ws.data_ptr(), Layer.W_WS.data_ptr(), y.data_ptr(), ARCQ_F16, m, self.n, self.k,
                self.bits, 64, stream)

    def gemm_args(self, ws, y, m, stream):
        from arcq_vit_amd._lib import ARCQ_F16
        return (ws.data_ptr(), self.packed.data_ptr(), self.cb.data_ptr(), self.center.data_ptr(),
                self.scale.data_ptr(), self.code_sum.data_ptr(), self.bias.data_ptr(), Layer.W_WS.data_ptr(),
                y.data_ptr(), ARCQ_F16, m, self.n, self.k, self.bits, 64, stream)

    # The two halves of arcq_linear_otf_ws on their own.  Block-layout shapes: arcq_act_quant_blocked_with_weights
    # (stage 1 plus the weight reconstruction carried in the same launch) and arcq_linear_fused_blocked on weights
    # that are ready; other shapes: arcq_act_quant and arcq_linear_fused_ws.  A layer that runs as ONE launch
    # ("rows": otf_rows_kernel / otf_rows_phased_kernel, stage 1 + weight reconstruction + GEMM) has no halves:
    # call_gemm is the whole layer, and call_act runs the stand-alone stage-1 kernel on the layer's input, which the
    # step itself never launches (reported as a reference figure).
    def mode(self, lib, m):
        name = lib.arcq_linear_otf_ws_kernel(m, self.n, self.k, 1)
        return ("rows" if name in (b"otf_rows_kernel", b"otf_rows_phased_kernel") else
                "copy" if name in (b"gemm_slab8_kernel<copy>", b"gemm_pair_kernel") else
                "blocked" if b"slab8" in name else "rowmajor")

    def call_act(self, lib, x, ws, stream):
        from arcq_vit_amd._lib import ARCQ_F16
        mode = self.mode(lib, x.shape[0])
        if mode == "rows":       # no stage-1 launch of its own in the step: the stand-alone kernel, timed for reference
            mode = "blocked"
        if mode == "copy":
            return lib.arcq_act_quant_blocked_with_weights(
                x.data_ptr(), ARCQ_F16, self.thr.data_ptr(), self.cb.data_ptr(), ws.data_ptr(), x.shape[0], self.k,
                self.bits, 1.0e-6, self.packed.data_ptr(), self.cb.data_ptr(), self.center.data_ptr(),
                self.scale.data_ptr(), self.code_sum.data_ptr(), Layer.W_WS.data_ptr(), self.n, stream)
        if mode == "blocked":
            return lib.arcq_act_quant_blocked(x.data_ptr(), ARCQ_F16, self.thr.data_ptr(), self.cb.data_ptr(),
                                              ws.data_ptr(), x.shape[0], self.k, self.bits, 1.0e-6, stream)
        return lib.arcq_act_quant(*self.act_args(x, ws, stream))

    def call_gemm(self, lib, ws, y, m, stream, x=None):
        from arcq_vit_amd._lib import ARCQ_F16
        mode = self.mode(lib, m)
        if mode == "rows":
            return lib.arcq_linear_otf_ws(*self.otf_args(x, ws, y, stream))
        if mode == "rowmajor":
            return lib.arcq_linear_fused_ws(*self.gemm_args(ws, y, m, stream))
        # "copy": W_WS holds some layer's reconstructed weights of at least this size (timing does not depend on which)
        return lib.arcq_linear_fused_blocked(
            ws.data_ptr(), self.packed.data_ptr(), self.cb.data_ptr(), self.center.data_ptr(), self.scale.data_ptr(),
            self.code_sum.data_ptr(), self.bias.data_ptr(), Layer.W_WS.data_ptr() if mode == "copy" else 0,
            1 if mode == "copy" else 0, y.data_ptr(), ARCQ_F16, m, self.n, self.k, self.bits, 64, stream)

    def call_gemm_rebuild_inside(self, lib, ws, y, m, stream, x=None):
        """The fused GEMM with the weights reconstructed inside the kernel (no weight workspace at all); a one-launch
        layer as it is (its weights are rebuilt inside its launch anyway)."""
        from arcq_vit_amd._lib import ARCQ_F16
        if self.mode(lib, m) == "rows":
            return lib.arcq_linear_otf_ws(*self.otf_args(x, ws, y, stream))
        if self.mode(lib, m) == "rowmajor":
            return lib.arcq_linear_fused(ws.data_ptr(), self.packed.data_ptr(), self.cb.data_ptr(), self.center.data_ptr(),
                                         self.scale.data_ptr(), self.code_sum.data_ptr(), self.bias.data_ptr(),
                                         y.data_ptr(), ARCQ_F16, m, self.n, self.k, self.bits, 64, stream)
        return lib.arcq_linear_fused_blocked(
            ws.data_ptr(), self.packed.data_ptr(), self.cb.data_ptr(), self.center.data_ptr(), self.scale.data_ptr(),
            self.code_sum.data_ptr(), self.bias.data_ptr(), 0, 0, y.data_ptr(), ARCQ_F16, m, self.n, self.k, self.bits,
            64, stream)

    def act_args(self, x, ws, stream):
        from arcq_vit_amd._lib import ARCQ_F16
        m = x.shape[0]
        return (x.data_ptr(), ARCQ_F16, self.thr.data_ptr(), self.cb.data_ptr(), 0, 0, 0, 0, 0, ws.data_ptr(),
                ARCQ_F16, m, self.k, self.bits, 64, 1.0e-6, stream)


def build_workload(model, bits, batch, dev):
    import torch
    from arcq_vit_amd import synth
    m = batch * synth.TOKENS
    depth = synth.MODEL_DIMS[model]["depth"]
    layers = []
    for blk in range(depth):
        for i, (name, k, n) in enumerate(synth.block_linear_shapes(model)):
            layers.append(Layer(f"blocks.{blk}.{name}", k, n, bits, synth.SEED + 16 * blk + i, dev))
    inputs = {}
    for i, (name, k, n) in enumerate(synth.block_linear_shapes(model)):
        kind = "gelu" if name == "fc2" else "ln"
        inputs[name] = synth.make_activation(m, k, synth.SEED + 1000 + i, kind).to(torch.float16).to(dev)
    kmax = max(l.k for l in layers)
    nmax = max(l.n for l in layers)
    ws = torch.empty(m * kmax, dtype=torch.float16, device=dev)
    y = torch.empty(m * nmax, dtype=torch.float16, device=dev)
    need = max(l.n * l.k for l in layers)
    if Layer.W_WS is None or Layer.W_WS.numel() < need:
        Layer.W_WS = torch.empty(need, dtype=torch.float16, device=dev)
    return m, layers, inputs, ws, y


def time_loop(fn, steps, warmup):
    """Runs fn() warmup+steps times; returns seconds for exactly `steps`, from HIP events on the
    current stream, bracketed by synchronize on both sides."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3


def run_config(model, bits, batch, steps, warmup, dev, use_graph=False):
    import torch
    from arcq_vit_amd import _lib, synth
    lib = _lib.load()
    m, layers, inputs, ws, y = build_workload(model, bits, batch, dev)
    stream = torch.cuda.current_stream().cuda_stream

    def short(l):
        return l.name.rsplit(".", 1)[-1]

    otf = [l.otf_args(inputs[short(l)], ws, y, stream) for l in layers]

    def step_full():
        for a in otf:
            rc = lib.arcq_linear_otf_ws(*a)
            if rc:
                _lib.check(rc)

    def step_act():
        for l in layers:
            rc = l.call_act(lib, inputs[short(l)], ws, stream)
            if rc:
                _lib.check(rc)

    def step_gemm():
        for l in layers:
            rc = l.call_gemm(lib, ws, y, m, stream, inputs[short(l)])
            if rc:
                _lib.check(rc)

    def step_gemm_inside():
        for l in layers:
            rc = l.call_gemm_rebuild_inside(lib, ws, y, m, stream, inputs[short(l)])
            if rc:
                _lib.check(rc)

    if use_graph:
        # One HIP graph per step (the reference does this for bs <= 1,
        # scripts/benchmark_arcq_on_the_fly.py:223-231).  A launch through ctypes costs ~10 us of host
        # time, more than several of these kernels run, so eager timing would measure Python.
        def capture(kind, subset=None):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                sp = torch.cuda.current_stream().cuda_stream   # the capture stream
                for l in (layers if subset is None else subset):
                    x = inputs[short(l)]
                    if kind == "full":
                        rc = lib.arcq_linear_otf_ws(*l.otf_args(x, ws, y, sp))
                    elif kind == "act":
                        rc = l.call_act(lib, x, ws, sp)
                    elif kind == "inside":
                        rc = l.call_gemm_rebuild_inside(lib, ws, y, m, sp, x)
                    else:
                        rc = l.call_gemm(lib, ws, y, m, sp, x)
                    if rc:
                        _lib.check(rc)
            return g.replay
        step_full()
        torch.cuda.synchronize()
        step_gemm_inside()
        torch.cuda.synchronize()
        step_full, step_act, step_gemm = capture("full"), capture("act"), capture("gemm")
        step_gemm_inside = capture("inside")

    t_full = time_loop(step_full, steps, warmup)
    t_gemm = time_loop(step_gemm, steps, warmup)
    t_act = time_loop(step_act, steps, warmup)
    t_inside = time_loop(step_gemm_inside, steps, warmup)

    # The fused entry point picks one of several kernels per shape; time each kernel's launches on their own so that
    # the roofline figure belongs to one kernel (the one with the largest share of the step).
    per_kernel = {}
    by_kernel = {}
    for l in layers:
        by_kernel.setdefault(lib.arcq_linear_otf_ws_kernel(m, l.n, l.k, 1).decode(), []).append(l)
    for name, sub in by_kernel.items():
        if use_graph:
            fn = capture("gemm", sub)
        else:
            def fn(sub=sub):
                for l in sub:
                    l.call_gemm(lib, ws, y, m, stream, inputs[short(l)])
        t = time_loop(fn, steps, warmup)
        kf = sum(synth.algorithmic_flops(m, l.n, l.k) for l in sub)
        kb = sum(synth.algorithmic_bytes(m, l.n, l.k, bits) for l in sub)
        per_kernel[name] = {"launches_per_step": len(sub), "us_per_launch": t / steps / len(sub) * 1e6,
                            "ms_per_step": t / steps * 1e3, "tflops": kf * steps / t / 1e12,
                            "gbs": kb * steps / t / 1e9, "flops_per_launch": kf / len(sub),
                            "bytes_per_launch": kb / len(sub),
                            "shapes_nk": sorted({(l.n, l.k) for l in sub})}

    act_layers = [l for l in layers if l.mode(lib, m) != "rows"]          # layers with a stage-1 launch of their own
    n_act = len(layers)                                                   # (the stage-1 timing runs it for every layer)
    flops = sum(synth.algorithmic_flops(m, l.n, l.k) for l in layers)
    gemm_bytes = sum(synth.algorithmic_bytes(m, l.n, l.k, bits) for l in layers)
    act_bytes = sum(2 * 2 * m * l.k for l in layers)              # fp16 in, fp16 out
    res = {
        "batch": batch, "M": m, "layers": len(layers),
        "ms_per_step": t_full / steps * 1e3,
        "images_per_s": batch * steps / t_full,
        "gemm_ms_per_step": t_gemm / steps * 1e3,
        "gemm_us_per_launch": t_gemm / steps / len(layers) * 1e6,
        "gemm_tflops": flops * steps / t_gemm / 1e12,
        "gemm_gbs": gemm_bytes * steps / t_gemm / 1e9,
        "gemm_rebuild_inside_us_per_launch": t_inside / steps / len(layers) * 1e6,
        "gemm_rebuild_inside_tflops": flops * steps / t_inside / 1e12,
        "act_ms_per_step": t_act / steps * 1e3,
        "act_us_per_launch": t_act / steps / n_act * 1e6, "act_launches_per_step": len(act_layers),
        "act_gbs": act_bytes * steps / t_act / 1e9,
        "flops_per_step": flops, "gemm_bytes_per_step": gemm_bytes, "gemm_kernels": per_kernel,
        # stage-1 kernel of the first layer's shape (the large-M layers all take the same one)
        "act_kernel": {"copy": "act_quant_blocked2_kernel (block layout, weight reconstruction carried along)",
                       "blocked": "act_quant_blocked2_kernel (block layout)",
                       "rowmajor": "act_quant_g64_kernel / act_quant_small_kernel (row-major)"}[
                           act_layers[0].mode(lib, m) if act_layers else "blocked"],
    }
    return res, layers, inputs


def cold_cache_bs1(model, bits, steps, warmup, dev, footprint_bytes=512 << 20):
    """Batch-1 step with the packed weights coming from HBM: enough distinct copies of the model's weight buffers
    (and inputs) to exceed the 256 MB last-level cache twice are cycled through, one HIP graph per copy, so no
    replay finds its weights cached.  Returns ms/step and the algorithmic bytes/s of the packed linears."""
    import torch
    from arcq_vit_amd import _lib, synth
    lib = _lib.load()
    m, layers, inputs, ws, y = build_workload(model, bits, 1, dev)
    per_copy = sum(t.numel() * t.element_size() for l in layers
                   for t in (l.packed, l.center, l.scale, l.code_sum, l.bias))
    copies = max(2, -(-footprint_bytes // per_copy))
    graphs = []
    for c in range(copies):
        ls = layers if c == 0 else [l.clone_weights() for l in layers]
        xs = {k: v.clone() for k, v in inputs.items()}
        for l in ls:                                   # warm the code path once outside capture
            lib.arcq_linear_otf_ws(*l.otf_args(xs[l.name.rsplit(".", 1)[-1]], ws, y, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            sp = torch.cuda.current_stream().cuda_stream
            for l in ls:
                rc = lib.arcq_linear_otf_ws(*l.otf_args(xs[l.name.rsplit(".", 1)[-1]], ws, y, sp))
                if rc:
                    _lib.check(rc)
        graphs.append((g, ls, xs))
    state = {"i": 0}

    def step():
        graphs[state["i"] % copies][0].replay()
        state["i"] += 1
    t = time_loop(step, max(steps, copies), max(warmup, copies))
    n = max(steps, copies)
    nbytes = sum(synth.algorithmic_bytes(m, l.n, l.k, bits) for l in layers)
    return {"ms_per_step": t / n * 1e3, "images_per_s": n / t, "weight_copies_cycled": copies,
            "bytes_per_copy": per_copy, "algorithmic_gbs": nbytes * n / t / 1e9,
            "hbm_frac": nbytes * n / t / 1e9 / PEAK_HBM_GBS}


def chained_step(model, bits, batch, steps, warmup, dev):
    """The packed linears of the model as a dependency chain: every layer reads what the layer before it wrote (the
    step of `run_config` runs the layers on fixed inputs, so nothing in it waits for a predecessor).  Per block:
    qkv(x) -> q; proj(the first M*dim values of q, standing in for the attention output) -> p; fc1(p) -> h; fc2(h) -> x.
    Two figures under one HIP graph per step: `plain` (arcq_linear_otf_ws per layer) and `fused` (arcq_linear_otf_ex:
    LayerNorm in front of qkv / fc1, GELU behind fc1, the skip connections behind proj / fc2 -- the work that sits
    between the packed linears of a transformer block, inside their launches), and the latter with fc2's stage 1 inside
    fc1's launch as well."""
    import ctypes
    import torch
    from arcq_vit_amd import _lib, synth
    from arcq_vit_amd._lib import ARCQ_F16
    lib = _lib.load()
    m, layers, inputs, ws, _ = build_workload(model, bits, batch, dev)
    dim, hid = synth.MODEL_DIMS[model]["dim"], synth.MODEL_DIMS[model]["mlp"]
    x0 = inputs["qkv"].clone()
    ring = [torch.empty_like(x0) for _ in range(3)]       # the residual stream after attention / after the MLP, rotating
    q = torch.empty(m * 3 * dim, dtype=torch.float16, device=dev)
    h = torch.empty(m * hid, dtype=torch.float16, device=dev)
    ln_w = torch.ones(max(dim, hid), dtype=torch.float32, device=dev)
    ln_b = torch.zeros(max(dim, hid), dtype=torch.float32, device=dev)
    keep = []

    def ex(l, x, y, ln=False, gelu=False, res=None, nxt_layer=None, from_xhat=False):
        a = _lib.LinearExArgs()
        a.struct_size = ctypes.sizeof(_lib.LinearExArgs)
        a.x_dtype = a.y_dtype = ARCQ_F16
        a.bits, a.group_size, a.M, a.N, a.K = l.bits, 64, m, l.n, l.k
        a.x, a.y, a.x_hat_ws, a.w_hat_ws = x.data_ptr(), y.data_ptr(), ws.data_ptr(), Layer.W_WS.data_ptr()
        if ln:
            a.producer, a.ln_weight, a.ln_bias, a.ln_eps = _lib.ARCQ_PRODUCER_LAYERNORM, ln_w.data_ptr(), ln_b.data_ptr(), 1e-6
        if from_xhat:
            a.producer = _lib.ARCQ_PRODUCER_XHAT
        if nxt_layer is not None:
            a.next_a_thresholds, a.next_a_codebook = nxt_layer.thr.data_ptr(), nxt_layer.cb.data_ptr()
        a.activation = _lib.ARCQ_ACT_GELU if gelu else _lib.ARCQ_ACT_NONE
        a.residual = None if res is None else res.data_ptr()
        a.a_thresholds, a.a_codebook, a.packed_w, a.w_codebook = l.thr.data_ptr(), l.cb.data_ptr(), l.packed.data_ptr(), l.cb.data_ptr()
        a.w_center, a.w_scale, a.w_code_sum, a.bias = l.center.data_ptr(), l.scale.data_ptr(), l.code_sum.data_ptr(), l.bias.data_ptr()
        keep.append(a)
        return a

    def run(fused, stream):
        cur, r = x0, 0
        for b in range(len(layers) // 4):
            qkv, proj, fc1, fc2 = layers[4 * b:4 * b + 4]
            mid, nxt = ring[r % 3], ring[(r + 1) % 3]       # cur is x0 or ring[(r + 2) % 3]
            r += 2
            if fused == "xhat":       # fc1's launch ends with fc2's stage 1; fc2 starts from that x_hat
                calls = [ex(qkv, cur, q, ln=True), ex(proj, q, mid, res=cur),
                         ex(fc1, mid, h, ln=True, gelu=True, nxt_layer=fc2), ex(fc2, h, nxt, res=mid, from_xhat=True)]
            elif fused:
                calls = [ex(qkv, cur, q, ln=True), ex(proj, q, mid, res=cur), ex(fc1, mid, h, ln=True, gelu=True),
                         ex(fc2, h, nxt, res=mid)]
            else:
                calls = [ex(qkv, cur, q), ex(proj, q, mid), ex(fc1, mid, h), ex(fc2, h, nxt)]
            for a in calls:
                rc = lib.arcq_linear_otf_ex(ctypes.byref(a), stream)
                if rc:
                    _lib.check(rc)
            cur = nxt

    out = {}
    variants = [("plain", False), ("fused", True), ("fused_mlp_chained_through_x_hat", "xhat")]
    for name, fused in variants:
        run(fused, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            run(fused, torch.cuda.current_stream().cuda_stream)
        t = time_loop(g.replay, steps, warmup)
        out[name + "_ms_per_step"] = t / steps * 1e3
        out[name + "_images_per_s"] = batch * steps / t
        del g
    out["note"] = ("every layer reads its predecessor's output; fused = LayerNorm / GELU / skip connections inside the "
                   "packed layers' launches (arcq_linear_otf_ex)")
    return out


def cpu_baseline(layers, inputs, batch, budget_s=12.0):
    """Oracle restatement of QuantLinearPCARCQ.forward (FQ/quant_backends.py:312-322) on host cores: the four linears
    of ONE block at the benchmark's batch, repeated while the time budget lasts (at least once); images/s = batch /
    (depth * time per block).  Two figures: `value`, faithful to the reference (the weight is quantized and
    reconstructed again on every call), and `value_weights_prebuilt` (the weight fake-quantized once beforehand)."""
    import torch
    import torch.nn.functional as F
    from arcq_vit_amd import synth
    from oracle import arcq_ref
    block = layers[:4]
    depth = len(layers) // 4
    xs = [inputs[l.name.rsplit(".", 1)[-1]].float().cpu() for l in block]
    cb = synth.quantile_codebook(block[0].bits)
    thr = synth.midpoint_thresholds(cb)
    bs = [l.bias.cpu() for l in block]

    def timed(fn, budget):
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            if time.perf_counter() - t0 > budget or reps >= 8:
                break
        return (time.perf_counter() - t0) / reps, reps

    with torch.no_grad():
        arcq_ref.fake_quant_linear(xs[1][:256], block[1].w_fp32, bs[1], thr, cb, thr, cb, 64, 1e-6)  # warm up

        def faithful():
            for l, x, b in zip(block, xs, bs):
                arcq_ref.fake_quant_linear(x, l.w_fp32, b, thr, cb, thr, cb, 64, 1e-6)
        dt, reps = timed(faithful, budget_s)
        wq = [arcq_ref.pcarcq_fake_quant(l.w_fp32, thr, cb, 64, 1e-6) for l in block]

        def prebuilt():
            for w, x, b in zip(wq, xs, bs):
                F.linear(arcq_ref.pcarcq_fake_quant(x, thr, cb, 64, 1e-6), w, b)
        dt2, reps2 = timed(prebuilt, budget_s)
    return {"value": batch / (depth * dt), "unit": "images/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"4 linears of one block at batch {batch} (M={xs[0].shape[0]}), {reps} repetitions (weights "
                      f"re-quantized per call, as the reference does) and {reps2} (weights fake-quantized once), "
                      f"scaled by depth {depth}; torch fp32 on {torch.get_num_threads()} threads "
                      f"(os.cpu_count()={os.cpu_count()})",
            "ms_per_block": dt * 1e3, "value_weights_prebuilt": batch / (depth * dt2),
            "ms_per_block_weights_prebuilt": dt2 * 1e3}


def model_forward(model, bits, batches, steps, warmup, dev):
    """Whole-model forward of the skeleton ViT (fp16 patch embedding, LayerNorm, softmax attention, GELU and head;
    packed on-the-fly block linears with the shared scratch buffers), random-init weights, synthetic normalized
    images: the protocol of scripts/benchmark_arcq_on_the_fly.py:202-243 (HIP graph at batch 1, eager otherwise; both
    figures are given for every batch).  Two models: the block's LayerNorms, GELU and skip connections
    as separate torch kernels (`unfused`, the reference's structure), inside the packed layers' launches
    (`fused_elementwise`), and that with the softmax attention and the fp16 patch embedding on the library's own kernels
    instead of torch's (`fused_elementwise_own_attention_patch_embed`: a block is then five launches, the front end one)."""
    import torch
    from arcq_vit_amd import synth
    from arcq_vit_amd.vit import build_packed_vit
    out = {"model": model, "bits": bits, "trunk": "fp16 (patch embed, LayerNorm, attention, GELU, head)"}
    for name, fuse, own in (("unfused", False, False), ("fused_elementwise", True, False),
                            ("fused_elementwise_own_attention_patch_embed", True, True)):
        vit = build_packed_vit(model, bits, device="cuda", half_chain=True, shared_buffers=True,
                               max_rows=max(batches) * synth.TOKENS, fuse_elementwise=fuse, own_attention=own,
                               own_patch_embed=own)
        out["blocks"] = len(vit.blocks)
        part = {}
        with torch.no_grad():
            for b in batches:
                x = synth.make_images(b, 1).to(dev).half()
                n = max(steps // (4 if b > 1 else 1), 5)
                res = {}
                # eager launches from Python: at batch 1 this measures the host side of the module path (it is slower
                # than the GPU work it issues), which the graph figure below hides
                t = time_loop(lambda: vit(x), n, max(warmup // 2, 2))
                res["eager_images_per_s"] = b * n / t
                res["eager_ms"] = t / n * 1e3
                vit(x)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    vit(x)
                t = time_loop(g.replay, n, max(warmup // 2, 2))
                res["graph_images_per_s"] = b * n / t
                res["graph_ms"] = t / n * 1e3
                part[f"bs{b}"] = res
                del g
        out[name] = part
        del vit
        torch.cuda.empty_cache()
    return out


def fp8_step(layers, inputs, m, steps, warmup):
    """The same step with the operands rounded to FP8 (arcq_linear_otf_fp8: stage 1 -> FP8 in the GEMM's block layout with
    the FP8 weights reconstructed in the same launch, then the library's own FP8 MFMA GEMM with fp32 accumulation):
    ms/step under a HIP graph, how far its outputs are from the fp16 path's, and -- as a timing reference only -- the
    same step with the product on the vendor library's FP8 GEMM (three launches per layer)."""
    import torch
    from arcq_vit_amd import ops
    dev = layers[0].packed.device
    x8 = torch.empty(m * max(ops.fp8_padded_k(l.k) for l in layers), dtype=torch.uint8, device=dev)
    w8 = torch.empty(max(l.n * ops.fp8_padded_k(l.k) for l in layers), dtype=torch.uint8, device=dev)
    mults = [ops.fp8_weight_multiplier(l.cb, l.center, l.scale, l.code_sum) for l in layers]

    def run(l, mult, fn=ops.linear_otf_fp8, xw=x8, ww=w8):
        x = inputs[l.name.rsplit(".", 1)[-1]]
        return fn(x, l.thr, l.cb, l.packed, l.cb, l.center, l.scale, l.code_sum, l.bias, l.bits, w_mult=mult, x8_ws=xw, w8_ws=ww)

    def timed(step):
        step()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            step()
        return time_loop(g.replay, steps, warmup)

    t = timed(lambda: [run(l, mult) for l, mult in zip(layers, mults)])
    x8l, w8l = x8.view(torch.float8_e4m3fn), w8.view(torch.float8_e4m3fn)
    try:
        t_lib = timed(lambda: [run(l, mult, ops.linear_otf_fp8_library_gemm, x8l, w8l) for l, mult in zip(layers, mults)])
    except Exception as e:          # (the library refuses some shapes)
        t_lib = None
    rel = []
    for l, mult in list(zip(layers, mults))[:4]:          # the four layer shapes of the first block
        x = inputs[l.name.rsplit(".", 1)[-1]]
        y16 = ops.linear_otf(x, l.thr, l.cb, l.packed, l.cb, l.center, l.scale, l.code_sum, l.bias, l.bits, 64,
                             out_dtype=torch.float32)
        rel.append(float((run(l, mult).float() - y16).norm() / y16.norm()))
    flops = sum(2.0 * m * l.n * l.k for l in layers)
    tf = flops * steps / t / 1e12
    return {"ms_per_step": t / steps * 1e3, "tflops_whole_step": tf, "frac_of_fp8_mfma_peak": tf / PEAK_FP8_TFLOPS,
            "peak_fp8_tflops": PEAK_FP8_TFLOPS, "launches_per_layer": 2,
            "vendor_library_gemm_ms_per_step": None if t_lib is None else t_lib / steps * 1e3,
            "relative_distance_from_fp16_path": rel,
            "note": "operands rounded to OCP E4M3 (3 mantissa bits): NOT the reference's numerics; stage 3 is this library's "
                    "FP8 MFMA kernel (gemm_fp8_kernel); the vendor-library figure (torch._scaled_mm, three launches per "
                    "layer) is a timing reference only"}


def kernel_note(name):
    if name == "otf_rows_kernel":
        return ("the WHOLE layer in one launch: stage 1 of 64 rows into LDS, the fp16 weights reconstructed cooperatively "
                "into the workspace, fp16 MFMA GEMM + bias; its duration includes stage 1 and the reconstruction")
    if name == "otf_rows_phased_kernel":
        return ("the WHOLE layer in one launch for long rows and few outputs (K = 768 / 1536 with N <= 384, K = 3072 with "
                "N <= 768): the rows are quantized into LDS in slices of 384 or 256 values "
                "while the MFMAs of the previous slice run; weights reconstructed cooperatively into the workspace; "
                "its duration includes stage 1 and the reconstruction")
    if name in ("gemm_slab8_kernel<copy>", "gemm_pair_kernel"):
        return ("fp16 MFMA GEMM + bias on weights that the stage-1 launch of the same layer reconstructed into an "
                "fp16 workspace (copied global -> LDS); its own launch does no dequantization")
    if name == "gemm_slab8_kernel":
        return "packed weights reconstructed into LDS inside the kernel, fp16 MFMA GEMM + bias"
    return "stages 2+3 fused (see arcq_linear_fused_kernel)"


def layer_roofline(res, bits):
    """Algorithmic flops of the step over the time of the whole step (stage 1, weight reconstruction, GEMM, gaps),
    against the MFMA peak and against min(MFMA, HBM), the time either bound alone would allow."""
    t = res["ms_per_step"] * 1e-3
    flops, nbytes = res["flops_per_step"], res["gemm_bytes_per_step"]
    t_mfma, t_hbm = flops / (PEAK_FP16_TFLOPS * 1e12), nbytes / (PEAK_HBM_GBS * 1e9)
    return {"tflops": flops / t / 1e12, "frac_mfma": flops / t / 1e12 / PEAK_FP16_TFLOPS,
            "gbs": nbytes / t / 1e9, "frac_hbm": nbytes / t / 1e9 / PEAK_HBM_GBS,
            "frac_min_mfma_hbm": max(t_mfma, t_hbm) / t, "ms_at_mfma_peak": t_mfma * 1e3, "ms_at_hbm_peak": t_hbm * 1e3}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path issues no collectives); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from arcq_vit_amd import _lib
    _lib.load()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    res, layers, inputs = run_config(args.model, args.bits, args.batch, args.steps, args.warmup, dev,
                                     use_graph=not args.eager)
    dom = max(res["gemm_kernels"], key=lambda k: res["gemm_kernels"][k]["ms_per_step"])
    one = sum(v["launches_per_step"] for k, v in res["gemm_kernels"].items() if k.startswith("otf_rows"))
    launch_note = ("every layer runs as ONE launch (stage 1 inside the GEMM kernel)" if one == res["layers"] else
                   f"{one} of the {res['layers']} layers run as ONE launch (stage 1 inside the GEMM kernel), "
                   f"the others as two (stage 1 + weight reconstruction, then the GEMM)")
    dk = res["gemm_kernels"][dom]
    out = {
        "metric": "DeiT-S W4A4 images/s at bs1/bs64; packed-linear % of MFMA/HBM roofline",
        "value": res["images_per_s"], "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{args.model} {res['layers']} packed linears ({res['layers'] // 4} blocks x qkv/proj/fc1/fc2), W{args.bits}A{args.bits}, "
                               f"g=64, batch {args.batch} (M={res['M']}), fp16 in/out; per layer: stage 1 (activation quantize + reconstruct), the fp16 weights "
                               f"reconstructed from the packed codes, an fp16 MFMA GEMM + bias -- {launch_note}",
                   "model_shapes": args.model, "bits": args.bits, "batch": args.batch, "group_size": 64},
        "roofline": {"bound": "mfma", "kernel": dom, "kernel_does": kernel_note(dom), "achieved": dk["tflops"],
                     "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s", "frac": dk["tflops"] / PEAK_FP16_TFLOPS,
                     "traffic": profiled_traffic(args.model, args.bits, args.batch, dom),
                     "traffic_source": traffic_source(args.model, args.bits, args.batch),
                     "algorithmic_flops_per_launch": dk["flops_per_launch"],
                     "algorithmic_bytes_per_launch": dk["bytes_per_launch"],
                     "avg_launch_us": dk["us_per_launch"], "launches_per_step": dk["launches_per_step"],
                     "hbm_frac_of_same_kernel": dk["gbs"] / PEAK_HBM_GBS,
                     "all_fused_gemm_launches": {"tflops": res["gemm_tflops"], "avg_launch_us": res["gemm_us_per_launch"],
                                                 "frac": res["gemm_tflops"] / PEAK_FP16_TFLOPS},
                     # the same GEMMs with the weights reconstructed inside the kernel (no workspace): the
                     # "dequantization fused into the GEMM" variant, which the step does not run because it is slower
                     "weights_rebuilt_inside_gemm": {"tflops": res["gemm_rebuild_inside_tflops"],
                                                     "avg_launch_us": res["gemm_rebuild_inside_us_per_launch"],
                                                     "frac": res["gemm_rebuild_inside_tflops"] / PEAK_FP16_TFLOPS},
                     # all_fused_gemm_launches counts a one-launch layer whole (stage 1 included)
                     # whole layer = stage 1 (+ weight reconstruction) + GEMM, everything the step runs
                     "layer": layer_roofline(res, args.bits)},
        # the stand-alone stage-1 kernel on every layer's input; the step launches it only for the two-launch layers
        "stage1": {"kernel": res["act_kernel"], "bound": "hbm", "achieved": res["act_gbs"], "peak": PEAK_HBM_GBS,
                   "unit": "GB/s", "frac": res["act_gbs"] / PEAK_HBM_GBS, "avg_launch_us": res["act_us_per_launch"],
                   "launches_in_step": res["act_launches_per_step"], "timed_launches": res["layers"]},
        "detail_bs%d" % args.batch: res,
    }
    if not args.no_bs1:
        r1, _, _ = run_config(args.model, args.bits, 1, max(args.steps, 50), max(args.warmup, 10), dev, use_graph=True)
        out["bs1"] = {"images_per_s": r1["images_per_s"], "ms_per_step": r1["ms_per_step"],
                      "gemm_us_per_launch": r1["gemm_us_per_launch"], "gemm_gbs_warm": r1["gemm_gbs"],
                      "gemm_hbm_frac_warm": r1["gemm_gbs"] / PEAK_HBM_GBS, "act_us_per_launch": r1["act_us_per_launch"],
                      "hip_graph": True}
        out["bs1"]["cold_cache"] = cold_cache_bs1(args.model, args.bits, max(args.steps, 50), max(args.warmup, 10), dev)
        out["bs1"]["chained"] = chained_step(args.model, args.bits, 1, max(args.steps, 50), max(args.warmup, 10), dev)
    if not args.no_other_configs and (args.model, args.bits, args.batch) == ("deit_small", 4, 64):
        # the other BASELINE configurations, a short timed run each (their own whole-step roofline; same kernels as
        # `bench.py --model ... --bits ... --batch ...` times at length)
        out["other_configs"] = {}
        for name, (mo, bi, ba, st) in {"deit_small_w3a3_bs64": ("deit_small", 3, 64, 20), "deit_base_w4a4_bs64": ("deit_base", 4, 64, 10),
                                       "vit_large_w3a3_bs256": ("vit_large", 3, 256, 4)}.items():
            ro, _, _ = run_config(mo, bi, ba, st, 2, dev, use_graph=not args.eager)
            domo = max(ro["gemm_kernels"], key=lambda k: ro["gemm_kernels"][k]["ms_per_step"])
            out["other_configs"][name] = {
                "ms_per_step": ro["ms_per_step"], "images_per_s": ro["images_per_s"], "steps": st, "layers": ro["layers"], "M": ro["M"],
                "dominant_kernel": domo, "dominant_kernel_us_per_launch": ro["gemm_kernels"][domo]["us_per_launch"],
                "dominant_kernel_tflops": ro["gemm_kernels"][domo]["tflops"],
                "dominant_kernel_frac_mfma": ro["gemm_kernels"][domo]["tflops"] / PEAK_FP16_TFLOPS,
                "stage1_us_per_launch": ro["act_us_per_launch"], "stage1_launches_per_step": ro["act_launches_per_step"],
                "layer": layer_roofline(ro, bi)}
            del ro
            torch.cuda.empty_cache()
    if not args.no_model:
        out["model_forward"] = model_forward(args.model, args.bits, sorted({1, args.batch}), args.steps, args.warmup, dev)
    if args.fp8:
        out["fp8_operands"] = fp8_step(layers, inputs, res["M"], args.steps, args.warmup)
    out["launch_mode"] = "eager" if args.eager else "hip_graph_per_step"
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(layers, inputs, args.batch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
