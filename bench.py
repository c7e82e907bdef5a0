#!/usr/bin/env python3
"""Benchmark of the fused-loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload lsr|lmargin|focal|lovasz|taylor|onehot|ohem|dice|layernorm|focal_seg|lsr_c150|lsr_c300|lsr_crop769|lmargin_crop513|taylor_crop769|lsr_vocab|lmargin_vocab|taylor_vocab|lmargin_rows]
                    [--no-cpu-baseline] [--no-others]

A step is one fwd+bwd pass of the loss module over one batch of synthetic input that is
already resident in HBM:  loss = criterion(logits, labels); loss.backward().
The headline workload is LabelSmoothSoftmaxCEV3 on fp32 logits (8, 19, 1024, 1024).
Prints ONE JSON line.  `value` is the bytes the timed module step has to move / time per step
(GB/s): with reduction='mean' the forward writes no per-pixel losses and the backward reads a
scalar upstream gradient, so the step moves less than the autograd-Function contract (unreduced
losses written, per-element upstream gradient read); `function_level` times that contract too
(reduction='none' and a per-element upstream gradient) with its own, larger byte count.
`roofline` prices the dominant kernel (the backward) against the 8 TB/s HBM peak with
HIP events on the launch stream; `cpu_baseline` times the pure-torch restatement of the
reference's CPU path on a bounded sample on the host cores.
Inputs of the configurations that the metric names (LSR, large-margin, focal, Lovasz, and the losses
that share their tensors) come from oracle/synth.py, a counter-based generator in numpy integer
arithmetic: the same bits on every box and under every torch version, so the printed losses can be
compared between runs and with the CPU oracle.
"""
import argparse
import gc
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "pytorch-loss_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, scaled by
# what the same counters read for the plain copy kernel): see profiles/*_hbm_traffic.txt.
# Only valid for the exact workload shape they were taken on; anything else reports null.
MEASURED_TRAFFIC = {
    # profiles/lsr_8x19x1024x1024_hbm_traffic.txt and profiles/all_workloads_hbm_traffic.txt (KiB per dispatch x 1024;
    # for kernels launched with both kinds of upstream gradient, the launches with one value per loss element,
    # which are the ones timed here: the largest FETCH_SIZE of the run)
    ("lsr", (8, 19, 1024, 1024)): {"forward": (688199 + 32768) * 1024, "backward": (720988 + 622621) * 1024},
    ("lmargin", (8, 19, 1024, 1024)): {"forward": (688218 + 32768) * 1024, "backward": (721014 + 622648) * 1024},
    ("taylor", (8, 19, 1024, 1024)): {"forward": (688322 + 32768) * 1024, "backward": (721261 + 622847) * 1024},
    ("focal", (16, 80, 128, 128)): {"forward": (163862 + 81921) * 1024, "backward": (245799 + 81920) * 1024},
    ("dice", (64, 1, 1024, 1024)): {"forward": (524418 + 32) * 1024, "backward": (524377 + 262148) * 1024},
    ("layernorm", (16, 256, 128, 128)): {"forward": (262290 + 262221) * 1024, "backward": (524484 + 262176) * 1024},
    ("lovasz", (4, 19, 512, 1024)): {"forward": 2392181 * 1024, "backward": (327869 + 155670) * 1024},
}

WORKLOADS = {
    # name: (module factory name, logits shape, description)
    "lsr": dict(shape=(8, 19, 1024, 1024), desc="LabelSmoothSoftmaxCEV3 fwd+bwd, fp32 logits (8,19,1024,1024), "
                "int64 labels 5% ignore=255, lb_smooth=0.1, mean"),
    "lmargin": dict(shape=(8, 19, 1024, 1024), desc="LargeMarginSoftmaxV3 fwd+bwd, fp32 logits (8,19,1024,1024), "
                    "int64 labels 5% ignore=255, lam=0.3, mean"),
    "focal": dict(shape=(16, 80, 128, 128), desc="FocalLossV3 fwd+bwd, fp32 logits/labels (16,80,128,128), "
                  "Bernoulli(0.02) labels, alpha=0.25 gamma=2, mean"),
    "lovasz": dict(shape=(4, 19, 512, 1024), desc="LovaszSoftmaxV3 fwd+bwd, fp32 logits (4,19,512,1024), "
                   "Zipf(1.1) int64 labels 5% ignore=255, mean"),
    "taylor": dict(shape=(8, 19, 1024, 1024), desc="TaylorCrossEntropyLossV3 fwd+bwd, fp32 logits (8,19,1024,1024), "
                   "int64 labels 5% ignore=255, n=4, mean"),
    "onehot": dict(shape=(8, 19, 1024, 1024), desc="OnehotEncoder forward, int64 labels (8,1024,1024) 5% ignore=255 -> "
                   "fp32 (8,19,1024,1024), lb_smooth=0.1"),
    "dice": dict(shape=(64, 1, 1024, 1024), desc="SoftDiceLossV3 fwd+bwd, fp32 logits/labels (64,1,1024,1024) as one row, "
                 "Bernoulli(0.3) labels, p=1 smooth=1"),
    "layernorm": dict(shape=(16, 256, 128, 128), desc="LayerNormV3Func fwd+bwd, fp32 (16,256,128,128) normalised over C, "
                      "eps=1e-6, per-element upstream gradient"),
    # the same loss away from the register-resident channel counts: 150 and 300 classes in NCHW (the channels of
    # a pixel shared out over the wavefronts of a block) and vocabulary-sized rows (a block per row)
    "lsr_c150": dict(base="lsr", shape=(8, 150, 512, 512), desc="LabelSmoothSoftmaxCEV3 fwd+bwd, fp32 logits (8,150,512,512), "
                     "int64 labels 5% ignore=255, lb_smooth=0.1, mean"),
    "lsr_c300": dict(base="lsr", shape=(8, 300, 256, 256), desc="LabelSmoothSoftmaxCEV3 fwd+bwd, fp32 logits (8,300,256,256), "
                     "int64 labels 5% ignore=255, lb_smooth=0.1, mean"),
    # the focal loss at the segmentation shape of the other two losses (the shape the >= 70 % target is stated on)
    "focal_seg": dict(base="focal", shape=(8, 19, 1024, 1024), desc="FocalLossV3 fwd+bwd, fp32 logits/labels (8,19,1024,1024), "
                      "Bernoulli(0.02) labels, alpha=0.25 gamma=2, mean"),
    # crops of odd size: every channel plane starts at another offset into a cache line (tiles per image, 4 pixels per lane)
    "lsr_crop769": dict(base="lsr", shape=(16, 19, 769, 769), desc="LabelSmoothSoftmaxCEV3 fwd+bwd, fp32 logits (16,19,769,769), "
                        "int64 labels 5% ignore=255, lb_smooth=0.1, mean"),
    "lmargin_crop513": dict(base="lmargin", shape=(32, 19, 513, 513), desc="LargeMarginSoftmaxV3 fwd+bwd, fp32 logits (32,19,513,513), "
                            "int64 labels 5% ignore=255, lam=0.3, mean"),
    "taylor_crop769": dict(base="taylor", shape=(16, 19, 769, 769), desc="TaylorCrossEntropyLossV3 fwd+bwd, fp32 logits (16,19,769,769), "
                           "int64 labels 5% ignore=255, n=4, mean"),
    "lsr_vocab": dict(base="lsr", shape=(8192, 32000), desc="LabelSmoothSoftmaxCEV3 fwd+bwd, fp32 logits (8192,32000), "
                      "int64 labels 5% ignore=255, lb_smooth=0.1, mean"),
    "lmargin_vocab": dict(base="lmargin", shape=(8192, 32000), desc="LargeMarginSoftmaxV3 fwd+bwd, fp32 logits (8192,32000), "
                          "int64 labels 5% ignore=255, lam=0.3, mean"),
    "taylor_vocab": dict(base="taylor", shape=(8192, 32000), desc="TaylorCrossEntropyLossV3 fwd+bwd, fp32 logits (8192,32000), "
                         "int64 labels 5% ignore=255, n=4, mean"),
    # classifier-sized rows: a wavefront holds a row in its registers
    "lmargin_rows": dict(base="lmargin", shape=(65536, 1000), desc="LargeMarginSoftmaxV3 fwd+bwd, fp32 logits (65536,1000), "
                         "int64 labels 5% ignore=255, lam=0.3, mean"),
    "ohem": dict(shape=(8, 19, 1024, 1024), desc="OhemCELoss fwd+bwd (relabelling and cross entropy in one forward pass), fp32 logits (8,19,1024,1024) "
                 "= 4*N(0,1), int64 labels 5% ignore=255, score_thresh=0.7, n_min=P/16"),
}


def describe(name, dtype):
    return WORKLOADS[name]["desc"].replace("fp32 logits", {"f32": "fp32", "f16": "fp16", "bf16": "bf16"}[dtype] + " logits")


def numel(shape):
    n = 1
    for d in shape:
        n *= d
    return n


ELEM_BYTES = {"f32": 4, "f16": 2, "bf16": 2}
DTYPE_TAG = {"f32": 0, "f16": 1, "bf16": 2}


def algorithmic_bytes(name, shape, dtype="f32"):
    """Bytes a fwd+bwd pass has to move at the autograd-Function level (logits and their gradient
    in `dtype`, int64 labels, fp32 losses / upstream gradient / Jaccard differences):
    forward reads the inputs and writes the unreduced losses, backward reads the inputs and the
    upstream gradient and writes the logits gradient."""
    E = numel(shape)
    P = E // shape[1]
    b = ELEM_BYTES[dtype]
    if name == "ohem":     # forward: logits and labels in, the selection (as new labels) and one loss out; backward: logits, labels, gradient
        return b * E + 8 * P + 8 * P, b * E + 8 * P + b * E
    if name in ("lsr", "lmargin", "taylor"):
        fwd = b * E + 8 * P + 4 * P
        bwd = b * E + 8 * P + 4 * P + b * E
    elif name == "focal":   # the labels are floating point and share the logits' type
        fwd = 2 * b * E + 4 * E
        bwd = 2 * b * E + 4 * E + b * E
    elif name == "layernorm":   # x in, y out; x and the upstream gradient in, the result out
        fwd = 2 * b * E
        bwd = 3 * b * E
    elif name == "dice":    # float labels in the logits' type; one loss and two sums per row
        fwd = 2 * b * E
        bwd = 2 * b * E + b * E
    else:  # lovasz: compulsory I/O only (logits, labels, saved Jaccard differences, gradient)
        fwd = b * E + 8 * P + 4 * E
        bwd = b * E + 4 * E + 8 * P + b * E
    return fwd, bwd


def module_bytes(name, shape, dtype="f32"):
    """Bytes the module-level step has to move (what `value` divides): as algorithmic_bytes(), minus what
    reduction='mean' leaves out: LSR, large-margin and Taylor CE write no per-pixel losses (4P) and read
    one scalar instead of a per-pixel upstream gradient (4P): 3bE + 16P; focal likewise (4E each way): 5bE."""
    fwd, bwd = algorithmic_bytes(name, shape, dtype)
    E = numel(shape)
    P = E // shape[1]
    if name in ("lsr", "lmargin", "taylor"):
        return fwd - 4 * P, bwd - 4 * P
    if name == "focal":
        return fwd - 4 * E, bwd - 4 * E
    return fwd, bwd


# Workloads whose tensors are one of oracle/synth.py's named configurations (seed 15): (configuration, logits factor)
SYNTH_CONFIG = {
    ("lsr", (8, 19, 1024, 1024)): ("cfg2", 1.0), ("lmargin", (8, 19, 1024, 1024)): ("cfg2", 1.0),
    ("taylor", (8, 19, 1024, 1024)): ("cfg2", 1.0), ("ohem", (8, 19, 1024, 1024)): ("cfg2", 2.0),
    ("focal", (16, 80, 128, 128)): ("cfg3", 1.0), ("lovasz", (4, 19, 512, 1024)): ("cfg5", 1.0),
}
_SYNTH_CACHE = {}


def make_inputs(name, shape, device, seed=15, dtype="f32"):
    logits, labels = _make_inputs_f32(name, shape, device, seed)
    if dtype != "f32":
        import torch
        td = {"f16": torch.float16, "bf16": torch.bfloat16}[dtype]
        logits = logits.to(td)
        if name in ("focal", "dice"):
            labels = labels.to(td)
    return logits, labels


def _make_inputs_f32(name, shape, device, seed):
    import torch
    if seed == 15 and (name, tuple(shape)) in SYNTH_CONFIG:
        from oracle import synth     # input generation only; nothing of the oracle runs in a timed region
        cfg, factor = SYNTH_CONFIG[(name, tuple(shape))]
        if cfg not in _SYNTH_CACHE:
            w = synth.workload(cfg)
            _SYNTH_CACHE[cfg] = (torch.from_numpy(w["logits"]), torch.from_numpy(w["labels"]))
        logits, labels = _SYNTH_CACHE[cfg]
        logits = logits.to(device)
        return (logits * factor if factor != 1.0 else logits), labels.to(device)
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    if name == "focal":
        logits = torch.randn(shape, device=device, generator=g) * 1.5 - 2.0
        labels = (torch.rand(shape, device=device, generator=g) < 0.02).float()
        return logits, labels
    if name == "dice":
        logits = torch.randn(shape, device=device, generator=g) * 2.0
        return logits, (torch.rand(shape, device=device, generator=g) < 0.3).float()
    logits = torch.randn(shape, device=device, generator=g) * (4.0 if name == "ohem" else 2.0)
    lshape = shape[:1] + shape[2:]
    if name == "lovasz":
        p = (torch.arange(19, device=device, dtype=torch.float64) + 1.0) ** -1.1
        cdf = torch.cumsum(p / p.sum(), 0)
        u = torch.rand(lshape, device=device, generator=g, dtype=torch.float64)
        labels = torch.searchsorted(cdf, u).clamp_(max=18)
    else:
        labels = torch.randint(0, shape[1], lshape, device=device, generator=g)
    ignore = torch.rand(lshape, device=device, generator=g) < 0.05
    labels[ignore] = 255
    return logits, labels


def make_criterion(name):
    import pytorch_loss as pl
    if name == "lsr":
        return pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="mean", ignore_index=255)
    if name == "lmargin":
        return pl.LargeMarginSoftmaxV3(lam=0.3, reduction="mean", ignore_index=255)
    if name == "focal":
        return pl.FocalLossV3(alpha=0.25, gamma=2, reduction="mean")
    if name == "ohem":
        return pl.OhemCELoss(score_thresh=0.7, n_min=None, ignore_index=255)
    if name == "taylor":
        return pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255, reduction="mean")
    if name == "dice":
        return pl.SoftDiceLossV3(p=1, smooth=1.0)
    return pl.LovaszSoftmaxV3(reduction="mean", ignore_index=255)


def time_steps(crit, logits, labels, steps, warmup):
    import torch
    logits.requires_grad_(True)

    def step():
        logits.grad = None
        loss = crit(logits, labels)
        loss.backward()
        return loss

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, float(loss.item())


def function_level_step(name, logits, labels, steps, warmup, dtype):
    """The autograd-Function contract, timed: unreduced losses out (reduction='none'), a per-element upstream
    gradient in. None for the ops whose module step already is that contract."""
    import torch
    import pytorch_loss as pl
    if name not in ("lsr", "lmargin", "taylor", "focal"):
        return None
    crit = {"lsr": lambda: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="none", ignore_index=255),
            "lmargin": lambda: pl.LargeMarginSoftmaxV3(lam=0.3, reduction="none", ignore_index=255),
            "taylor": lambda: pl.TaylorCrossEntropyLossV3(n=4, ignore_index=255, reduction="none"),
            "focal": lambda: pl.FocalLossV3(alpha=0.25, gamma=2, reduction="none")}[name]()
    logits.requires_grad_(True)
    with torch.no_grad():
        like = crit(logits, labels)
    go = torch.full(like.shape, 1.0 / like.numel(), dtype=like.dtype, device=like.device)
    del like

    def step():
        logits.grad = None
        crit(logits, labels).backward(go)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    nbytes = sum(algorithmic_bytes(name, tuple(logits.shape), dtype))
    gbps = nbytes / (ms * 1e-3) / 1e9
    return {"what": "reduction='none' and a per-element upstream gradient: unreduced losses written, upstream gradient read",
            "ms_per_step": round(ms, 4), "GB/s": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
            "algorithmic_bytes_per_step": nbytes}


def step_distribution(crit, inputs, iters=100):
    """Per-step GPU time (HIP events around each fwd+bwd step): median / p10 / p90 in ms. `inputs` is a
    list of (logits, labels) sets used round-robin: one set = cache-warm, several sets whose total
    size exceeds the 256 MB Infinity Cache = cache-cold."""
    import torch
    for x, _ in inputs:
        x.requires_grad_(True)
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for i in range(iters + 10):
        x, y = inputs[i % len(inputs)]
        x.grad = None
        if i >= 10:
            events[i - 10][0].record()
        crit(x, y).backward()
        if i >= 10:
            events[i - 10][1].record()
    torch.cuda.synchronize()
    ms = sorted(a.elapsed_time(b) for a, b in events)
    return {"median": round(ms[len(ms) // 2], 4), "p10": round(ms[len(ms) // 10], 4),
            "p90": round(ms[(9 * len(ms)) // 10], 4), "iters": iters, "input_sets": len(inputs)}


def graph_step(crit, logits, labels, iters=100):
    """The module step captured once in a HIP graph and replayed: its time on the GPU alone, without the
    host's share (Python, the autograd engine's thread hand-over, launch latency). None if capture fails."""
    import torch
    try:
        logits.requires_grad_(True)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                logits.grad = None
                crit(logits, labels).backward()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        logits.grad = None
        with torch.cuda.graph(graph):
            crit(logits, labels).backward()
        torch.cuda.synchronize()
        ms = time_kernel(graph.replay, iters=iters, warmup=10)
        del graph
        logits.grad = None
        return {"ms": round(ms, 4), "iters": iters,
                "what": "the same fwd+bwd step captured in a HIP graph and replayed (GPU time without the host's share)"}
    except Exception as e:
        return {"error": "%s: %s" % (type(e).__name__, e)}


def time_kernel(launch, iters=30, warmup=5):
    """Average duration (ms) of one launch: HIP events on the stream the kernel runs on."""
    import torch
    for _ in range(warmup):
        launch()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        launch()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def kernel_rooflines(name, logits, labels, dtype="f32"):
    """Per-kernel roofline entries for the forward and backward entry points, called directly
    through the C ABI wrappers with pre-allocated outputs (no allocator, no autograd in the loop)."""
    import torch
    from pytorch_loss import _native
    lib = _native.load()
    shape = tuple(logits.shape)
    fwd_bytes, bwd_bytes = algorithmic_bytes(name, shape, dtype)
    x = logits.detach()
    tag = DTYPE_TAG[dtype]
    n, c = shape[0], shape[1]
    m = numel(shape) // (n * c)
    st = _native._stream
    P = _native._ptr
    out = {}
    if name == "ohem":
        # forward = relabelling + mean cross entropy in one entry point; backward = cross-entropy gradient on the new labels
        kept = torch.empty(labels.numel(), dtype=torch.uint8, device=x.device)
        scratch = torch.empty((2, labels.numel()), dtype=torch.float32, device=x.device)
        loss = torch.empty((), dtype=torch.float32, device=x.device)
        n_valid = torch.empty((), dtype=torch.int64, device=x.device)
        grad = torch.empty_like(x)
        ws_bytes = int(lib.plh_ohem_ce_workspace_bytes(labels.numel()))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
        f = lambda: lib.plh_ohem_ce_forward_kept(P(x), tag, P(labels), P(kept), P(scratch[0]), P(scratch[1]), P(loss),
                                                 P(n_valid), P(ws), ws_bytes, n, c, m, 255, 0.7, labels.numel() // 16, st())
        b = lambda: lib.plh_lsr_backward_kept(P(x), tag, P(labels), P(kept), P(loss), 1.0, P(n_valid), P(grad), n, c, m, 255,
                                              0.0, st())
        # OhemLargeMarginLoss: the same pipeline behind the large-margin forward kernel, and that loss's gradient
        fl = lambda: lib.plh_ohem_lmargin_forward_kept(P(x), tag, P(labels), P(kept), P(scratch[0]), P(scratch[1]),
                                                       P(loss), P(n_valid), P(ws), ws_bytes, n, c, m, 255, 0.3, 0.7,
                                                       labels.numel() // 16, st())
        bl = lambda: lib.plh_lmargin_backward_kept(P(x), tag, P(labels), P(kept), P(loss), 1.0, P(n_valid), P(grad), n, c, m,
                                                   255, 0.3, st())
        assert f() == 0 and b() == 0 and fl() == 0 and bl() == 0
        for key, fn, nbytes in (("forward", f, fwd_bytes), ("backward", b, bwd_bytes),
                                ("large_margin_forward", fl, fwd_bytes), ("large_margin_backward", bl, bwd_bytes)):
            ms = time_kernel(fn)
            gbps = nbytes / (ms * 1e-3) / 1e9
            out[key] = {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None, "ms": round(ms, 4),
                        "algorithmic_bytes": nbytes}
        return out
    if name in ("lsr", "lmargin", "taylor"):
        losses = torch.empty(labels.shape, dtype=torch.float32, device=x.device)
        grad = torch.empty_like(x)
        gout = torch.full(labels.shape, 1.0 / labels.numel(), dtype=torch.float32, device=x.device)
        if name == "taylor":
            f = lambda: lib.plh_taylor_ce_forward(P(x), tag, P(labels), P(losses), None, None, 0, None, 0, n, c, m, 4,
                                                  255, st())
            b = lambda: lib.plh_taylor_ce_backward(P(x), tag, P(labels), P(gout), 1, 1.0, None, P(grad), n, c, m, 4,
                                                   255, st())
        elif name == "lsr":
            f = lambda: lib.plh_lsr_forward(P(x), tag, P(labels), P(losses), n, c, m, 255, 0.1, st())
            b = lambda: lib.plh_lsr_backward(P(x), tag, P(labels), P(gout), 1, P(grad), n, c, m, 255, 0.1, st())
        else:
            f = lambda: lib.plh_lmargin_forward(P(x), tag, P(labels), P(losses), n, c, m, 255, 0.3, st())
            b = lambda: lib.plh_lmargin_backward(P(x), tag, P(labels), P(gout), 1, P(grad), n, c, m, 255, 0.3, st())
    elif name == "focal":
        losses = torch.empty(shape, dtype=torch.float32, device=x.device)
        grad = torch.empty_like(x)
        gout = torch.full(shape, 1.0 / x.numel(), dtype=torch.float32, device=x.device)
        f = lambda: lib.plh_focal_forward(P(x), tag, P(labels), P(losses), x.numel(), 2.0, 0.25, st())
        b = lambda: lib.plh_focal_backward(P(x), tag, P(labels), P(gout), 1, P(grad), x.numel(), 2.0, 0.25, st())
    elif name == "dice":
        losses = torch.empty(1, dtype=torch.float32, device=x.device)
        stats = torch.empty(2, dtype=torch.float32, device=x.device)
        grad = torch.empty_like(x)
        gout = torch.ones(1, dtype=torch.float32, device=x.device)
        ws_bytes = int(lib.plh_soft_dice_workspace_bytes(1, x.numel()))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
        f = lambda: lib.plh_soft_dice_forward(P(x), tag, P(labels), P(losses), P(stats), P(ws), ws_bytes, 1, x.numel(),
                                              1.0, 1.0, st())
        b = lambda: lib.plh_soft_dice_backward(P(gout), P(x), tag, P(labels), P(stats), P(grad), 1, x.numel(), 1.0, st())
    else:
        losses = torch.empty(c, dtype=torch.float32, device=x.device)
        jacc = torch.empty((c, n * m), dtype=torch.float32, device=x.device)
        grad = torch.empty_like(x)
        gout = torch.full((c,), 1.0 / c, dtype=torch.float32, device=x.device)
        ws_bytes = int(lib.plh_lovasz_workspace_bytes(n, c, m))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
        f = lambda: lib.plh_lovasz_forward(P(x), tag, P(labels), P(losses), P(jacc), P(ws), ws_bytes, n, c, m, 255, st())
        b = lambda: lib.plh_lovasz_backward(P(gout), P(x), tag, P(labels), P(jacc), P(grad), n, c, m, 255, st())
    assert f() == 0 and b() == 0
    legs = [("forward", f, fwd_bytes), ("backward", b, bwd_bytes)]
    if name == "taylor":
        # the softmax Function itself (TaylorSoftmaxV3 / LogTaylorSoftmaxV3): x in, y out; grad and x in, grad out
        y_out = torch.empty_like(x)
        eb = x.element_size() * x.numel()
        sf = lambda: lib.plh_taylor_softmax_forward(P(x), tag, P(y_out), n, c, m, 4, 1, st())
        sb = lambda: lib.plh_taylor_softmax_backward(P(y_out), P(x), tag, P(grad), n, c, m, 4, 1, st())
        assert sf() == 0 and sb() == 0
        legs += [("log_softmax_forward", sf, 2 * eb), ("log_softmax_backward", sb, 3 * eb)]
    if name == "lsr" and lib.plh_lsr_saves_lse(tag, n, c, m):
        # channel planes of odd length: the module's own pair of entry points - the reduced forward that keeps every
        # pixel's log-sum-exp and the backward that forms the gradient from it plane by plane (one scalar upstream)
        E, Pn = n * c * m, n * m
        lse = torch.empty(Pn, dtype=torch.float32, device=x.device)
        one_loss = torch.empty((), dtype=torch.float32, device=x.device)
        n_valid = torch.empty((), dtype=torch.int64, device=x.device)
        rws_bytes = int(lib.plh_reduce_workspace_bytes(Pn))
        rws = torch.empty(rws_bytes, dtype=torch.uint8, device=x.device)
        up = torch.ones((), dtype=torch.float32, device=x.device)
        fl = lambda: lib.plh_lsr_forward_reduced_lse(P(x), tag, P(labels), P(lse), P(one_loss), P(n_valid), 1, P(rws), rws_bytes,
                                                     n, c, m, 255, 0.1, st())
        bl = lambda: lib.plh_lsr_backward_scaled_lse(P(x), tag, P(labels), P(lse), None, P(up), 1.0, P(n_valid), P(grad),
                                                     n, c, m, 255, 0.1, st())
        assert fl() == 0 and bl() == 0
        eb = ELEM_BYTES[dtype]
        legs += [("forward_keeping_lse", fl, eb * E + 8 * Pn + 4 * Pn), ("backward_from_lse", bl, 2 * eb * E + 8 * Pn + 4 * Pn)]
    if name == "lmargin" and lib.plh_lmargin_saves_stats(tag, n, c, m):
        # long rows: the module's forward leaves eight floats per row and its backward works from them, elementwise
        E, Pn = n * c * m, n * m
        stats = torch.empty((Pn, 8), dtype=torch.float32, device=x.device)
        one_loss = torch.empty((), dtype=torch.float32, device=x.device)
        n_valid = torch.empty((), dtype=torch.int64, device=x.device)
        rws_bytes = int(lib.plh_reduce_workspace_bytes(Pn))
        rws = torch.empty(rws_bytes, dtype=torch.uint8, device=x.device)
        up = torch.ones((), dtype=torch.float32, device=x.device)
        fs = lambda: lib.plh_lmargin_forward_reduced_stats(P(x), tag, P(labels), P(stats), P(one_loss), P(n_valid), 1, P(rws),
                                                           rws_bytes, n, c, m, 255, 0.3, st())
        bs = lambda: lib.plh_lmargin_backward_scaled_stats(P(x), tag, P(labels), P(stats), None, P(up), 1.0, P(n_valid), P(grad),
                                                           n, c, m, 255, 0.3, st())
        assert fs() == 0 and bs() == 0
        eb = ELEM_BYTES[dtype]
        legs += [("forward_keeping_stats", fs, eb * E + 8 * Pn + 32 * Pn), ("backward_from_stats", bs, 2 * eb * E + 8 * Pn + 32 * Pn)]
    if name == "taylor" and lib.plh_taylor_ce_saves_sums(tag, n, c, m):
        # rows: the module's forward leaves each row's sum of f and its backward works from it, elementwise
        E, Pn = n * c * m, n * m
        sums = torch.empty((Pn,), dtype=torch.float32, device=x.device)
        one_loss = torch.empty((), dtype=torch.float32, device=x.device)
        n_valid = torch.empty((), dtype=torch.int64, device=x.device)
        rws_bytes = int(lib.plh_reduce_workspace_bytes(Pn))
        rws = torch.empty(rws_bytes, dtype=torch.uint8, device=x.device)
        up = torch.ones((), dtype=torch.float32, device=x.device)
        fs = lambda: lib.plh_taylor_ce_forward_reduced_sums(P(x), tag, P(labels), P(sums), P(one_loss), P(n_valid), 1, P(rws),
                                                            rws_bytes, n, c, m, 4, 255, st())
        bs = lambda: lib.plh_taylor_ce_backward_scaled_sums(P(x), tag, P(labels), P(sums), P(up), 1.0, P(n_valid), P(grad),
                                                            n, c, m, 4, 255, st())
        assert fs() == 0 and bs() == 0
        eb = ELEM_BYTES[dtype]
        legs += [("forward_keeping_sums", fs, eb * E + 8 * Pn + 4 * Pn), ("backward_from_sums", bs, 2 * eb * E + 8 * Pn + 4 * Pn)]
    if name == "lovasz":
        # the same forward with its sort passes in the decoupled look-back form (an entry point of its own)
        lb_bytes = int(lib.plh_lovasz_lookback_workspace_bytes(n, c, m))
        lb_ws = torch.empty(lb_bytes, dtype=torch.uint8, device=x.device)
        lf = lambda: lib.plh_lovasz_forward_lookback(P(x), tag, P(labels), P(losses), P(jacc), P(lb_ws), lb_bytes, n, c, m,
                                                     255, st())
        assert lf() == 0
        legs += [("forward_look_back", lf, fwd_bytes)]
    for key, fn, nbytes in legs:
        ms = time_kernel(fn)
        gbps = nbytes / (ms * 1e-3) / 1e9
        traffic = MEASURED_TRAFFIC.get((name, shape), {}).get(key) if dtype == "f32" else None
        out[key] = {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": traffic,
                    "ms": round(ms, 4), "algorithmic_bytes": nbytes}
    return out


def copy_ceiling(device, nbytes=1 << 30):
    import torch
    from pytorch_loss import _native
    src = torch.empty(nbytes // 4, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    ms = time_kernel(lambda: _native.stream_copy(src, dst))
    return round(2 * nbytes / (ms * 1e-3) / 1e9, 1)


def cpu_threads():
    """Host threads of the CPU leg. A one-GPU box hands a job 16 host threads whatever os.cpu_count() shows
    (OMP_NUM_THREADS=16 is exported there), so that is the count used and stated; without the variable, every core
    up to 16."""
    return int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)


def cpu_baseline(name, shape, spot_check=True):
    """Pure-torch restatement of the reference's V2 (V1 for Lovasz) path on the host threads: the whole batch of the
    workload, once warm and twice timed (a step takes 0.02-0.8 s; layer norm and soft dice: one image, scaled)."""
    import torch
    from oracle import synth, torch_ref
    cores = cpu_threads()
    torch.set_num_threads(cores)
    if name == "layernorm":
        g = torch.Generator().manual_seed(15)
        logits = (torch.randn((1, shape[1], shape[2] * shape[3]), generator=g) * 2.0 + 0.5).requires_grad_()
        go = torch.randn(logits.shape, generator=g)
        return _time_cpu(name, shape, cores, lambda: (torch_ref.layer_norm(logits, 1e-6) * go).sum(), logits)
    if name == "dice":
        g = torch.Generator().manual_seed(15)
        logits = (torch.randn((1,) + tuple(shape[1:]), generator=g) * 2.0).requires_grad_()
        labels = (torch.rand(logits.shape, generator=g) < 0.3).float()
        return _time_cpu(name, shape, cores, lambda: torch_ref.soft_dice(logits, labels, 1, 1.0), logits)
    # the whole batch of the workload, the tensors of the GPU legs (oracle/synth.py's named configuration where the
    # workload is one; otherwise make_inputs' distribution from a CPU generator)
    whole = True
    if (name, tuple(shape)) in SYNTH_CONFIG:
        cfg, factor = SYNTH_CONFIG[(name, tuple(shape))]
        if cfg not in _SYNTH_CACHE:
            w = synth.workload(cfg)
            _SYNTH_CACHE[cfg] = (torch.from_numpy(w["logits"]), torch.from_numpy(w["labels"]))
        logits, labels = _SYNTH_CACHE[cfg]
        logits = (logits * factor if factor != 1.0 else logits.detach()).requires_grad_()
    elif name == "focal":
        g = torch.Generator().manual_seed(15)
        logits = (torch.randn(tuple(shape), generator=g) * 1.5 - 2.0).requires_grad_()
        labels = (torch.rand(logits.shape, generator=g) < 0.02).float()
    else:
        raise KeyError("no CPU leg for %s at %s" % (name, (shape,)))
    fn = {"lsr": lambda: torch_ref.lsr(logits, labels, 0.1, "mean", 255),
          "lmargin": lambda: torch_ref.lmargin(logits, labels, 0.3, "mean", 255),
          "focal": lambda: torch_ref.focal(logits, labels, 0.25, 2, "mean"),
          "lovasz": lambda: torch_ref.lovasz(logits, labels, "mean", 255),
          "ohem": lambda: torch_ref.ohem_ce(logits, labels, 0.7, None, 255),
          "taylor": lambda: torch_ref.taylor_ce(logits, labels, 4, "mean", 255)}[name]
    res = _time_cpu(name, shape, cores, fn, logits, whole=whole)
    if not spot_check:
        return res
    # the same input through the HIP module: the two losses are printed side by side
    try:
        with torch.no_grad():
            # Lovasz: the fp32 restatement's own sums over 2 M sorted errors are ~6e-4 off its fp64 evaluation
            # (sequential fp32 accumulation), so the check takes the fp64 one
            want = float((torch_ref.lovasz(logits.detach().double(), labels, "mean", 255) if name == "lovasz" else fn()).item())
        got = float(make_criterion(name)(logits.detach().to("cuda:0"), labels.to("cuda:0")).item())
        res["parity_spot_check"] = {"what": "loss of the CPU leg's input: HIP module on cuda:0 against the CPU restatement",
                                    "hip": got, "cpu": want, "rel_err": abs(got - want) / max(abs(want), 1e-30)}
    except Exception as e:
        res["parity_spot_check"] = {"error": "%s: %s" % (type(e).__name__, e)}
    return res


def _time_cpu(name, shape, cores, fn, logits, whole=False):
    times = []
    for i in range(3 if whole else 4):
        logits.grad = None
        t0 = time.perf_counter()
        fn().backward()
        t1 = time.perf_counter()
        if i:
            times.append((t1 - t0) * 1e3)
    scale = 1 if whole else shape[0]
    ms_full = statistics.median(times) * scale
    fwd, bwd = algorithmic_bytes(name, shape)
    sample = ("the whole batch, fwd+bwd, median of %d" % len(times)) if whole else (
        "1 of %d images of the workload, fwd+bwd, median of %d, time scaled x%d" % (scale, len(times), scale))
    return {"value": round((fwd + bwd) / (ms_full * 1e-3) / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "ms_per_step": round(ms_full, 2), "os_cpu_count": os.cpu_count(),
            "sample": "oracle/torch_ref.py (pure-torch restatement of the reference's V2/V1 CPU path) on " + sample}


def run_onehot(steps, warmup, device):
    """The target encoder is a forward-only write stream: labels (8,1024,1024) -> fp32 (8,19,1024,1024)."""
    import torch
    import pytorch_loss as pl
    from pytorch_loss import _native
    shape = WORKLOADS["onehot"]["shape"]
    _, labels = make_inputs("lsr", shape, device)
    enc = pl.OnehotEncoder(shape[1], lb_smooth=0.1, ignore_idx=255, check=False)
    for _ in range(warmup):
        enc(labels)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = enc(labels)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    nbytes = 4 * numel(shape) + 8 * labels.numel()
    lib = _native.load()
    n, c, m = shape[0], shape[1], labels.numel() // shape[0]
    k_ms = time_kernel(lambda: lib.plh_onehot(_native._ptr(labels), _native._ptr(out), None, n, c, m, 255, 0.1,
                                               _native._stream()))
    gbps = nbytes / (k_ms * 1e-3) / 1e9
    roof = {"encode": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                       "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None, "ms": round(k_ms, 4),
                       "algorithmic_bytes": nbytes}}
    return dict(ms_per_step=ms, gbps=nbytes / (ms * 1e-3) / 1e9, loss=float(out[0, 0, 0, 0].item()), roofline=roof,
                bytes=nbytes, step_ms={"warm": {"median": round(ms, 4), "iters": steps, "input_sets": 1}})


def run_layernorm(steps, warmup, device, dtype):
    """Not a loss: a step is Function forward + backward with a per-element upstream gradient."""
    import torch
    import pytorch_loss as pl
    from pytorch_loss import _native
    shape = WORKLOADS["layernorm"]["shape"]
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    g = torch.Generator(device=device)
    g.manual_seed(15)
    n, c = shape[0], shape[1]
    m = numel(shape) // (n * c)
    x = (torch.randn((n, c, m), device=device, generator=g) * 2.0 + 0.5).to(td).requires_grad_()
    go = torch.randn((n, c, m), device=device, generator=g).to(td)

    def step():
        x.grad = None
        y = pl.LayerNormV3Func.apply(x, 1e-6)
        y.backward(go)
        return y

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        y = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    fwd, bwd = algorithmic_bytes("layernorm", shape, dtype)
    lib = _native.load()
    P, st, tag = _native._ptr, _native._stream, DTYPE_TAG[dtype]
    xd, out = x.detach(), torch.empty_like(x)
    f = lambda: lib.plh_layer_norm_forward(P(xd), tag, P(out), n, c, m, 1e-6, st())
    b = lambda: lib.plh_layer_norm_backward(P(go), P(xd), tag, P(out), n, c, m, 1e-6, st())
    assert f() == 0 and b() == 0
    roof = {}
    for key, fn, nbytes in (("forward", f, fwd), ("backward", b, bwd)):
        k_ms = time_kernel(fn)
        gbps = nbytes / (k_ms * 1e-3) / 1e9
        traffic = MEASURED_TRAFFIC.get(("layernorm", shape), {}).get(key) if dtype == "f32" else None
        roof[key] = {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": traffic, "ms": round(k_ms, 4),
                     "algorithmic_bytes": nbytes}
    return dict(ms_per_step=ms, gbps=(fwd + bwd) / (ms * 1e-3) / 1e9, loss=float(y[0, 0, 0].item()), roofline=roof,
                bytes=fwd + bwd, step_ms={"warm": {"median": round(ms, 4), "iters": steps, "input_sets": 1}})


def run_workload(name, steps, warmup, device, dtype="f32"):
    import torch
    if name == "onehot":
        return run_onehot(max(steps, 20), warmup, device)
    if name == "layernorm":
        return run_layernorm(max(steps, 20), warmup, device, dtype)
    shape = WORKLOADS[name]["shape"]
    name = WORKLOADS[name].get("base", name)       # the op; `shape` is the entry's own
    logits, labels = make_inputs(name, shape, device, dtype=dtype)
    crit = make_criterion(name)
    ms, loss = time_steps(crit, logits, labels, steps, warmup)
    fwd, bwd = module_bytes(name, shape, dtype)
    gbps = (fwd + bwd) / (ms * 1e-3) / 1e9
    func = function_level_step(name, logits, labels, steps, warmup, dtype)
    roof = kernel_rooflines(name, logits, labels, dtype)
    dist = {"warm": step_distribution(crit, [(logits, labels)])}
    set_bytes = ELEM_BYTES[dtype] * numel(shape) * (2 if name in ("focal", "dice") else 1)
    if set_bytes < (256 << 20):
        # working set fits the Infinity Cache: also rotate enough input sets to defeat it
        n_sets = max(4, -(-(768 << 20) // set_bytes))
        sets = [(logits, labels)] + [make_inputs(name, shape, device, seed=100 + i, dtype=dtype) for i in range(n_sets - 1)]
        dist["cold"] = step_distribution(crit, sets)
        del sets
    dist["graph"] = graph_step(crit, logits, labels)
    if ms < 0.15:
        # a step this short can be bound by the autograd engine's hand-over between the calling thread and its
        # worker thread: the same steps with the backward run on the calling thread (a PyTorch switch, not the library's)
        try:
            with torch.autograd.set_multithreading_enabled(False):
                st_ms, _ = time_steps(crit, logits, labels, steps, warmup)
            dist["calling_thread"] = {"ms": round(st_ms, 4), "steps": steps,
                                      "what": "eager steps under torch.autograd.set_multithreading_enabled(False)"}
        except Exception as e:
            dist["calling_thread"] = {"error": "%s: %s" % (type(e).__name__, e)}
    # (beyond 32 channels fb=True runs two passes, except for large margin on (N, C) rows)
    if name == "focal" or (name in ("lsr", "lmargin") and shape[1] <= 32) or (name == "lmargin" and len(shape) == 2):
        # the same module with fb=True (what the reference's repository-root copies of the large-margin and focal
        # modules do: gradient computed in the forward pass and kept; for LSR a keyword the reference does not have):
        # one pass over the inputs per step. Its bytes: LSR and large margin read the logits and write the gradient
        # (2bE) and read the labels twice (the count of valid pixels, then the pass itself: 16P); focal reads logits
        # and labels and writes the gradient (3bE).
        try:
            import pytorch_loss as pl
            fb = {"lsr": lambda: pl.LabelSmoothSoftmaxCEV3(lb_smooth=0.1, reduction="mean", ignore_index=255, fb=True),
                  "lmargin": lambda: pl.LargeMarginSoftmaxV3(lam=0.3, reduction="mean", ignore_index=255, fb=True),
                  "focal": lambda: pl.FocalLossV3(alpha=0.25, gamma=2, reduction="mean", fb=True)}[name]()
            fb_ms, fb_loss = time_steps(fb, logits, labels, steps, warmup)
            eb, E = ELEM_BYTES[dtype], numel(shape)
            fb_bytes = 3 * eb * E if name == "focal" else 2 * eb * E + 16 * (E // shape[1])
            dist["one_pass_fb"] = {"ms": round(fb_ms, 4), "bytes": fb_bytes,
                                   "frac": round(fb_bytes / (fb_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                   "graph_ms": graph_step(fb, logits, labels).get("ms"),
                                   "loss_rel_diff": float("%.2g" % (abs(fb_loss - loss) / max(abs(loss), 1e-30)))}
            del fb
        except Exception as e:
            dist["one_pass_fb"] = {"error": "%s: %s" % (type(e).__name__, e)}
    del crit
    logits.grad = None
    return dict(ms_per_step=ms, gbps=gbps, loss=loss, roofline=roof, bytes=fwd + bwd, step_ms=dist, function_level=func)


TARGETS = ("lsr", "lmargin", "focal", "focal_seg", "lovasz")


def targets_block(headline, main_res, others, headline_cpu, with_cpu):
    """LSR, large margin, focal (at its own shape and at the segmentation shape) and Lovasz in one short object:
    eager module step (ms), the same step replayed from a HIP graph (graph_ms), the bytes the step has to move and the
    fraction of the 8 TB/s peak that makes (frac), forward / backward entry points alone (fwd_ms, bwd_ms), and the CPU
    restatement of the reference's V2 (Lovasz: V1) path on the host threads (cpu: ms per step, GB/s of the
    Function-level bytes, threads, relative difference of its loss from the HIP module's on the same input)."""
    out = {"unit": "ms", "peak_GBps": HBM_PEAK_GBPS}
    for t in TARGETS:
        if t == headline:
            ms, nbytes, step_ms, kern = main_res["ms_per_step"], main_res["bytes"], main_res["step_ms"], main_res["roofline"]
        else:
            o = others.get(t)
            if not o or "error" in o:
                out[t] = {"error": (o or {}).get("error", "not run")}
                continue
            ms, nbytes, step_ms, kern = o["ms_per_step"], o["algorithmic_bytes_per_step"], o["step_ms"], o["kernels"]
        e = {"ms": round(ms, 4), "graph_ms": (step_ms.get("graph") or {}).get("ms"), "bytes": nbytes,
             "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
             "fwd_ms": (kern.get("forward") or {}).get("ms"), "bwd_ms": (kern.get("backward") or {}).get("ms")}
        if "calling_thread" in step_ms:      # short steps: the eager step with the backward on the calling thread
            e["calling_thread_ms"] = step_ms["calling_thread"].get("ms")
        if "one_pass_fb" in step_ms:         # the module with fb=True: eager step, replayed step, fraction of peak on its own bytes
            fb = step_ms["one_pass_fb"]
            e["fb"] = {k: fb.get(k) for k in (("error",) if "error" in fb else ("ms", "graph_ms", "frac"))}
        if with_cpu:
            try:
                c = headline_cpu if (t == headline and headline_cpu and "error" not in headline_cpu) else \
                    cpu_baseline(WORKLOADS[t].get("base", t), WORKLOADS[t]["shape"])
                rel = c.get("parity_spot_check", {}).get("rel_err")
                e["cpu"] = {"ms": c["ms_per_step"], "GB/s": c["value"], "threads": c["cores"],
                            "rel_err": None if rel is None else float("%.2g" % rel)}
            except Exception as ex:
                e["cpu"] = {"error": "%s: %s" % (type(ex).__name__, ex)}
        out[t] = e
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="lsr", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default="f32", choices=sorted(ELEM_BYTES),
                    help="element type of logits and gradients in HBM (the arithmetic is fp32 in every case)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true", help="skip the secondary workloads")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the hot path has no collectives); "
                 "--gpus %d is not supported, run with --gpus 1" % args.gpus)

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    from pytorch_loss import _native
    _native.load()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    # Python's first full garbage collection of a process that has imported torch and numpy takes ~30 ms (measured:
    # once, at about step 100 of a loop of 0.34 ms steps), which is 90 steps' worth inside 50 timed ones. Collect now
    # and move what is alive out of the collector's sight; what the steps allocate is still collected.
    gc.collect()
    gc.freeze()

    name = args.workload
    main_res = run_workload(name, args.steps, args.warmup, device, args.dtype)
    torch.cuda.empty_cache()

    others = {}
    if not args.no_others:
        for other in WORKLOADS:
            if other == name:
                continue
            try:
                r = run_workload(other, max(5, args.steps // 2), max(2, args.warmup // 2), device, args.dtype)
                others[other] = {"workload": describe(other, args.dtype), "ms_per_step": round(r["ms_per_step"], 4),
                                 "step_ms": r["step_ms"], "algorithmic_bytes_per_step": r["bytes"], "loss": r["loss"],
                                 "GB/s": round(r["gbps"], 1), "frac_of_peak": round(r["gbps"] / HBM_PEAK_GBPS, 4),
                                 "function_level": r.get("function_level"),
                                 "kernels": {k: {"ms": v["ms"], "GB/s": v["achieved"], "frac": v["frac"]}
                                             for k, v in r["roofline"].items()}}
            except Exception as e:  # a secondary workload must not take the headline down
                others[other] = {"error": "%s: %s" % (type(e).__name__, e)}
            torch.cuda.empty_cache()

    try:
        ceiling = copy_ceiling(device)
    except Exception as e:
        ceiling = "error: %s" % e

    line = {
        "metric": "fwd+bwd ms/iter + achieved HBM GB/s (% peak), LSR-CE 8x19x1024^2 fp32",
        "value": round(main_res["gbps"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "python_gc": "collected and frozen before the first measurement",
        "ms_per_step": round(main_res["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": describe(name, args.dtype), "storage_dtype": args.dtype,
                   "algorithmic_bytes_per_step": main_res["bytes"],
                   "frac_of_hbm_peak": round(main_res["gbps"] / HBM_PEAK_GBPS, 4), "loss": main_res["loss"]},
        "roofline": dict(main_res["roofline"].get("backward") or list(main_res["roofline"].values())[0],
                         kernel="backward entry point of the workload" if "backward" in main_res["roofline"]
                         else "the workload's single entry point"),
        "roofline_forward": main_res["roofline"].get("forward"),
        "function_level": main_res.get("function_level"),
        "roofline_kernels": {k: {"ms": v["ms"], "GB/s": v["achieved"], "frac": v["frac"]}
                             for k, v in main_res["roofline"].items()},
        "step_ms": main_res["step_ms"],
        "copy_kernel_GBps": ceiling,
        "other_workloads": others,
    }
    if not args.no_cpu_baseline:
        try:
            if "base" in WORKLOADS[name]:
                raise ValueError("the CPU leg is kept for the configurations the reference's metric names")
            line["cpu_baseline"] = cpu_baseline(name, WORKLOADS[name]["shape"])
        except Exception as e:
            line["cpu_baseline"] = {"error": "%s: %s" % (type(e).__name__, e)}
    # Last key of the line, and short: the configurations the metric names, side by side. A record that keeps
    # only the end of a long line still holds all of them.
    line["targets"] = targets_block(name, main_res, others, line.get("cpu_baseline"), not args.no_cpu_baseline)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
