#!/usr/bin/env python3
"""Benchmark of the L_p-distance operator on one MI355X.

A step is one pass of the hot path over one batch of synthetic input at the headline shape
(B = 512, CI = CO = 5120, fully connected):  norm_dist forward + backward (grad_input and grad_weight) at p = 8,
followed by the same at p = infinity.  `value` is the wall time of that step in milliseconds with all inputs
resident in HBM; the per-part times and roofline fractions are in `parts`.

One JSON line is printed.  Besides the contract fields it carries
  roofline      the dominant kernel (fused p = 8 backward): algorithmic flop per launch / its measured duration,
                against the FP32 vector-ALU peak
  cpu_baseline  the same step evaluated by the pure-PyTorch broadcast formulation on the host cores, on a slice
                of the output features, scaled to the full width
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "l_inf-dist-net-v2_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

B, CI, CO = 512, 5120, 5120
PAIRS = B * CI * CO
# algorithmic flop per (b, co, ci) pair
FLOP = {"p8_fwd": 5, "p8_bwd": 9, "inf_fwd": 2}
# SIMD cycles one wave64 needs per pair in the leanest instruction sequence if every vector instruction issued at the
# best rate the part has shown for any stream (2 per 4-cycle issue slot and SIMD, reached only by streams of dependent
# add / mul at exactly 4 or 8 waves per SIMD): add / mul / fma with vector-register operands 2 cycles, everything
# else (min / max / compare / select, a scalar-register operand) 4 but overlapping with a 2-cycle instruction of
# another wave: cycles per pair = max(2 * all instructions, 4 * slow instructions)
#   p8 forward   sub, mul, mul, fma                                    4 fast          ->  8
#   p8 backward  sub, 3 mul, 2 fma fast; mul by the scalar factor slow   6 fast + 1 slow -> 14
#   inf forward  sub fast; half of a three-operand max slow             1 fast + 1/2    ->  3
ISSUE_CYCLES = {"p8_fwd": 8, "p8_bwd": 14, "inf_fwd": 3}
# What the same instruction mixes measure in the issue-rate micro-benchmark, with no memory traffic at all, at the
# occupancy the kernels have (4 waves per SIMD, best number of independent chains), in SIMD cycles per pair at the
# 2.4 GHz datasheet clock (profiles/microbench_valu_issue.txt): the practical floor of a kernel built from that mix.
MICROBENCH_CYCLES = {"p8_fwd": 10.4, "p8_bwd": 18.5, "inf_fwd": 3.9}
PEAK_FP32_TFLOPS = 157.3          # datasheet FP32 vector peak: 256 CU x 128 FMA lanes / clk x 2 flop x 2.4 GHz
SIMD_HZ = 256 * 4 * 2.4e9         # SIMD cycles per second at the datasheet clock
PEAK_HBM_GBS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "pmc_bwd_fused_kernel_p8_b512_5120x5120.txt")


def profiled_traffic_bytes():
    """HBM bytes per launch of the dominant kernel as the tracked rocprofv3 counter summary states them (this run
    does not measure them: counters need the profiler).  The summary holds FETCH_SIZE and WRITE_SIZE per dispatch in
    KiB and the scale factors a plain device copy of known size gave for the same counters; None without the file."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None
    import re
    m = re.search(r"per dispatch[^:]*:\s*FETCH_SIZE\s+([0-9.]+),\s*WRITE_SIZE\s+([0-9.]+)", text)
    f = re.search(r"FETCH_SIZE reads [0-9.]+ for [0-9]+ KiB read: scale factor ([0-9.]+)", text)
    w = re.search(r"WRITE_SIZE reads [0-9.]+: scale factor ([0-9.]+)", text)
    if not (m and f and w):
        return None
    return int((float(m.group(1)) * float(f.group(1)) + float(m.group(2)) * float(w.group(1))) * 1024)


def make_inputs(torch):
    gen = torch.Generator().manual_seed(2021)
    x = torch.randn(B, CI, generator=gen)
    w = torch.randn(CO, CI, generator=gen) / math.sqrt(CI)
    g = torch.randn(B, CO, generator=gen)
    return x, w, g


def cpu_baseline(torch, x, w, g, cols):
    """Pure-PyTorch formulation on the host: forward + autograd backward for p = 8 and p = inf on `cols` output
    features, best of 3 after a warm-up, scaled by CO / cols."""
    from oracle import torch_formulation as TF
    torch.set_num_threads(os.cpu_count() or 1)
    wc, gc = w[:cols].contiguous(), g[:, :cols].contiguous()
    TF.norm_dist_fwd_bwd(x, wc[:64], gc[:, :64], 8.0, chunk=64)  # warm-up: thread pool, allocator
    times = []
    for rep in range(3):
        t0 = time.perf_counter()
        for p in (8.0, float("inf")):
            TF.norm_dist_fwd_bwd(x, wc, gc, p, chunk=64)
        times.append(time.perf_counter() - t0)
    med = min(times)
    return {
        "value": round(med * CO / cols * 1e3, 1),
        "unit": "ms",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "pure-PyTorch broadcast formulation, fwd+bwd at p=8 and p=inf on %d of %d output features "
                  "(%.2f s measured, best of 3), scaled linearly to %d" % (cols, CO, med, CO),
    }


def other_workloads(torch, _C, xd, wd, gd):
    """Wall time per call (ms) of the remaining workloads of the operator, measured after the headline step:
    general p, interval bounds, the 6 x 5120 MLP training step and the 128-channel 3x3 conv layer."""
    import torch.nn.functional as F
    from core.modules import NormDistConv
    from ell_inf_models import MLPModel

    def tm(fn, n=5):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / n
        if ms < 1.5 and n < 20:  # short calls: five repetitions are within reach of one slow launch
            return tm(fn, 20)
        return round(ms, 3)

    res = {}
    dev = xd.device
    out = torch.empty(B, CO, 1, device=dev)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    res["p13.7_forward_b512_5120x5120"] = tm(lambda: _C.norm_dist_forward(xd, wd, out, 1, 13.7))
    o2 = out.clone()
    res["p13.7_backward_b512_5120x5120"] = tm(lambda: _C.norm_dist_backward_input_weight(gd, xd, wd, o2, gx, gw, 1, 13.7))
    for pp in (100.0, 1000.0):  # large exponents of the training schedule: the pair-skipping variants
        res["p%g_forward_b512_5120x5120" % pp] = tm(lambda: _C.norm_dist_forward(xd, wd, out, 1, pp))
        o3 = out.clone()
        res["p%g_backward_b512_5120x5120" % pp] = tm(
            lambda: _C.norm_dist_backward_input_weight(gd, xd, wd, o3, gx, gw, 1, pp))
    # the same exponents on unit-variance weights (the layers' own initialisation): pairs that count no longer line up
    # over the columns, the forward's probe keeps the plain kernel at p = 100
    w1 = wd * float(CI) ** 0.5
    for pp in (100.0, 1000.0):
        res["p%g_forward_unit_weights_b512_5120x5120" % pp] = tm(lambda: _C.norm_dist_forward(xd, w1, out, 1, pp))
        o5 = out.clone()
        res["p%g_backward_unit_weights_b512_5120x5120" % pp] = tm(
            lambda: _C.norm_dist_backward_input_weight(gd, xd, w1, o5, gx, gw, 1, pp))
    # the max-reductions on the same dense data (nothing to skip: behind the hot-tile plan the plain tiled kernel
    # runs), next to the library's own plain path with all data-dependent skipping switched off
    pos1 = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
    xl1, xu1 = xd - 8 / 255, xd + 8 / 255
    yl1, yu1, pu1 = torch.empty_like(out), torch.empty_like(out), torch.empty_like(pos1)
    for tag, skip in (("", -1), ("_skip_off", 0)):
        _C.set_skip_mode(skip, -1)
        try:
            res["pinf_forward_unit_weights%s_b512_5120x5120" % tag] = tm(lambda: _C.inf_dist_forward(xd, w1, out, pos1, 1))
            res["ibp_bounds_forward_unit_weights%s_b512_5120x5120" % tag] = tm(
                lambda: _C.bound_inf_dist_forward(xl1, xu1, w1, yl1, yu1, pos1, pu1, 1))
        finally:
            _C.set_skip_mode(-1, -1)
    del w1, pos1, xl1, xu1, yl1, yu1, pu1
    # small batch (64 rows): bound by streaming w (105 MB) rather than by arithmetic
    xs, gs = xd[:64].contiguous(), gd[:64].contiguous()
    outs = torch.empty(64, CO, 1, device=dev)
    gxs = torch.empty_like(xs)
    res["b64_pinf_forward_nograd_5120x5120"] = tm(lambda: _C.inf_dist_forward_nograd(xs, wd, outs, 1))
    res["b64_p8_forward_5120x5120"] = tm(lambda: _C.norm_dist_forward(xs, wd, outs, 1, 8.0))
    o4 = outs.clone()
    res["b64_p8_backward_5120x5120"] = tm(lambda: _C.norm_dist_backward_input_weight(gs, xs, wd, o4, gxs, gw, 1, 8.0))
    # the same three as streaming rates: algorithmic bytes (x, w read, out written; backward: x, w, out, grad_out read,
    # both gradients written) over the wall time per call, against the 8 TB/s of the HBM
    fwd_bytes = 4 * (64 * CI + CO * CI + 64 * CO)
    bwd_bytes = 4 * (2 * 64 * CI + 2 * CO * CI + 2 * 64 * CO)
    for key, nbytes in (("b64_pinf_forward_nograd_5120x5120", fwd_bytes), ("b64_p8_forward_5120x5120", fwd_bytes),
                        ("b64_p8_backward_5120x5120", bwd_bytes)):
        res[key + "_gbs"] = round(nbytes / res[key] / 1e6, 1)
    xl, xu = xd - 8 / 255, xd + 8 / 255
    yl, yu = torch.empty_like(out), torch.empty_like(out)
    pl = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
    pu = torch.empty_like(pl)
    res["ibp_bounds_forward_nograd_b512_5120x5120"] = tm(lambda: _C.bound_inf_dist_forward_nograd(xl, xu, wd, yl, yu, 1))
    res["ibp_bounds_forward_b512_5120x5120"] = tm(lambda: _C.bound_inf_dist_forward(xl, xu, wd, yl, yu, pl, pu, 1))
    gxu = torch.empty_like(xd)
    res["ibp_bounds_backward_b512_5120x5120"] = tm(
        lambda: _C.bound_inf_dist_backward_input_weight(gd, gd, pl, pu, gx, gxu, gw, 1))
    del out, gx, gw, o2, xl, xu, yl, yu, pl, pu, gxu

    torch.manual_seed(0)
    model = MLPModel(depth=6, width=5120, input_dim=(3, 32, 32), identity_val=10.0).to(dev)
    img = torch.rand(512, 3, 32, 32, device=dev)
    lab = torch.randint(0, 10, (512,), device=dev)

    def set_p(p):
        for m in model.modules():
            if hasattr(m, "p"):
                m.p = p

    from ell_inf_models import hinge
    loss_fn = hinge()
    eps_train = 8 / 255 / 0.2009  # the radius the published CIFAR-10 runs train with, in normalised pixel units

    def train_step():
        # hinge loss on the worst-case margins of the eps-ball (reference: ell_inf_models.py:41-46, main.py:304-310)
        model.zero_grad(set_to_none=True)
        outputs, worst = model(img, targets=lab, eps=eps_train)
        loss_fn(outputs, worst, lab).backward()

    set_p(8.0)
    res["mlp_6x5120_b512_p8_train_step"] = tm(train_step)
    set_p(13.7)  # early in the exponent's ramp: exp2 / log2 kernels, nothing to skip yet
    res["mlp_6x5120_b512_p13.7_train_step"] = tm(train_step)
    set_p(100.0)  # mid-schedule exponent: general-p kernels, pair skipping where the probe allows it
    res["mlp_6x5120_b512_p100_train_step"] = tm(train_step)
    set_p(float("inf"))
    res["mlp_6x5120_b512_pinf_train_step"] = tm(train_step)
    # smaller batches at a large exponent: the step is short, so queueing must not wait for the device
    set_p(100.0)
    img512, lab512 = img, lab
    for bsz in (128, 256):
        img, lab = img512[:bsz].contiguous(), lab512[:bsz].contiguous()
        res["mlp_6x5120_b%d_p100_train_step" % bsz] = tm(train_step)
    img, lab = img512, lab512
    set_p(float("inf"))
    model.eval()

    def certify():
        with torch.no_grad():
            model(img, targets=lab, eps=8 / 255, up=torch.ones_like(img), down=torch.zeros_like(img))

    res["mlp_6x5120_b512_pinf_eval_with_ibp"] = tm(certify)
    # opt-in: the layers keep the pre-pass over their weights between calls (no reference counterpart)
    from core.modules import freeze_weights
    freeze_weights(model)
    res["mlp_6x5120_b512_pinf_eval_with_ibp_frozen_weights"] = tm(certify)
    del model

    conv = NormDistConv(128, 128, 3, padding=1, bias=False, mean_shift=False).to(dev)
    conv.p = float("inf")
    cx = torch.randn(128, 128, 32, 32, device=dev, requires_grad=True)

    def conv_step():
        cx.grad = None
        conv.weight.grad = None
        y = conv(cx)[0]
        y.backward(torch.ones_like(y))

    res["conv3x3_128to128_b128_32x32_pinf_fwd_bwd"] = tm(conv_step)

    def conv_ibp_step():  # the layer with its interval bounds at eps = 8/255, forward and backward of all three outputs
        cx.grad = None
        conv.weight.grad = None
        y, lo, up = conv(cx, cx - 8 / 255, cx + 8 / 255)
        torch.autograd.backward([y, lo, up], [torch.ones_like(y)] * 3)

    res["conv3x3_128to128_b128_32x32_pinf_fwd_bwd_with_ibp"] = tm(conv_ibp_step)
    conv.eval()
    cd = cx.detach()

    def conv_ibp():
        with torch.no_grad():
            conv(cd, cd - 8 / 255, cd + 8 / 255)

    res["conv3x3_128to128_b128_32x32_pinf_eval_with_ibp"] = tm(conv_ibp)
    # the layer's forward alone with arg-max codes (first pass + second pass), and its training step at p = 8
    cw = conv.weight.detach()
    cy = torch.empty(128, 128, 1024, device=dev)
    cpos = torch.empty(128, 128, 1024, device=dev, dtype=torch.int32)
    res["conv3x3_128to128_b128_32x32_pinf_forward_with_codes"] = tm(
        lambda: _C.conv_inf_dist_forward(cd, cw, cy, cpos, 1, 3, 1, 1, 1))
    conv.train()
    conv.p = 8.0
    res["conv3x3_128to128_b128_32x32_p8_fwd_bwd"] = tm(conv_step)
    return res


def run_part(torch, _C, args, xd, wd, gd):
    """One entry point, called --steps times through the binding on pre-allocated outputs (for rocprofv3 runs);
    --batch takes the first rows of the benchmark's batch (64: the small-batch cases)."""
    nb = args.batch
    xd, gd = xd[:nb].contiguous(), gd[:nb].contiguous()
    out = torch.empty(nb, CO, 1, device=xd.device)
    pos = torch.empty(nb, CO, 1, device=xd.device, dtype=torch.int32)
    gx = torch.empty_like(xd)
    gw = torch.empty_like(wd)
    _C.norm_dist_forward(xd, wd, out, 1, 8.0)
    out8 = out.clone()
    _C.norm_dist_forward(xd, wd, out, 1, 13.7)
    out137 = out.clone()
    rmean, bmean, shifted = torch.zeros(CO, device=xd.device), torch.empty(CO, device=xd.device), torch.empty_like(out)
    _C.inf_dist_forward(xd, wd, out, pos, 1)
    calls = {
        "p8_fwd": lambda: _C.norm_dist_forward(xd, wd, out, 1, 8.0),
        "p8_bwd": lambda: _C.norm_dist_backward_input_weight(gd, xd, wd, out8, gx, gw, 1, 8.0),
        "p13.7_fwd": lambda: _C.norm_dist_forward(xd, wd, out, 1, 13.7),
        "p13.7_bwd": lambda: _C.norm_dist_backward_input_weight(gd, xd, wd, out137, gx, gw, 1, 13.7),
        "inf_fwd": lambda: _C.inf_dist_forward(xd, wd, out, pos, 1),
        "inf_fwd_nograd": lambda: _C.inf_dist_forward_nograd(xd, wd, out, 1),
        "inf_bwd": lambda: _C.inf_dist_backward_input_weight(gd, pos, gx, gw, 1),
        # what follows the operator in a layer: batch mean, moving average, subtraction (one launch)
        "mean_shift": lambda: _C.mean_shift_forward(out8, None, None, True, 0.1, rmean, None, None, bmean, shifted, None, None),
    }
    if args.part == "copy":
        # calibration for the FETCH_SIZE / WRITE_SIZE counters: a plain device copy of 256 MiB (read once, written once)
        src = torch.empty(64 * 1024 * 1024, device=xd.device).normal_()
        dst = torch.empty_like(src)
        calls["copy"] = lambda: dst.copy_(src)
    fn = calls[args.part]
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fn()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    print(json.dumps({"part": args.part, "batch": nb, "ms_per_call": round(ms, 4), "steps": args.steps,
                      "warmup": args.warmup}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--cpu-cols", type=int, default=1024, help="output features of the CPU baseline sample (0 = skip)")
    ap.add_argument("--no-other", action="store_true", help="skip the secondary workloads (general p, IBP, MLP, conv)")
    ap.add_argument("--part", default="all",
                    choices=["all", "p8_fwd", "p8_bwd", "p13.7_fwd", "p13.7_bwd", "mean_shift", "inf_fwd", "inf_fwd_nograd", "inf_bwd", "copy", "other"],
                    help="profiling aid: run only one entry point of the step, --steps times, on pre-allocated outputs")
    ap.add_argument("--batch", type=int, default=B, help="with --part: rows of the batch to use (e.g. 64)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus %d is not supported (no collective is built or used)"
                 % args.gpus)

    import torch
    from core import _C
    from core.norm_dist import norm_dist

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    x, w, g = make_inputs(torch)
    xd = x.to(dev).unsqueeze(-1).contiguous().requires_grad_(True)
    wd = w.to(dev).requires_grad_(True)
    gd = g.to(dev).unsqueeze(-1).contiguous()

    if args.part == "other":  # profiling aid: only the secondary workloads
        print(json.dumps({"other_workloads_ms": other_workloads(torch, _C, xd.detach(), wd.detach(), gd)}))
        return
    if args.part != "all":
        run_part(torch, _C, args, xd.detach(), wd.detach(), gd)
        return

    def step():
        for p in (8.0, float("inf")):
            xd.grad = None
            wd.grad = None
            y = norm_dist(xd, wd, p)
            y.backward(gd)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- per-part kernel durations, outside the timed region: HIP events around the dominant kernel of each call,
    # recorded by the library on the stream it launches on
    _C.set_profiling(True)
    reps = max(5, min(args.steps, 50))
    acc = {"p8_fwd": [], "p8_bwd": [], "inf_fwd": [], "inf_bwd": []}
    for _ in range(reps):
        for p, tag in ((8.0, "p8"), (float("inf"), "inf")):
            xd.grad = None
            wd.grad = None
            y = norm_dist(xd, wd, p)
            acc[tag + "_fwd"].append(_C.last_kernel_ms())
            y.backward(gd)
            acc[tag + "_bwd"].append(_C.last_kernel_ms())
    _C.set_profiling(False)
    avg = {k: sum(v) / len(v) for k, v in acc.items()}
    parts = {}
    for k, ms in avg.items():
        srt = sorted(acc[k])
        d = {"kernel_ms": round(ms, 4), "kernel_ms_median": round(srt[len(srt) // 2], 4), "kernel_ms_min": round(srt[0], 4)}
        if k in FLOP:
            d["tflops"] = round(PAIRS * FLOP[k] / ms / 1e9, 2)
            d["frac_fp32_peak"] = round(PAIRS * FLOP[k] / ms / 1e9 / PEAK_FP32_TFLOPS, 4)
            d["frac_issue_model"] = round(PAIRS / 64 * ISSUE_CYCLES[k] / SIMD_HZ * 1e3 / ms, 4)
            d["frac_microbench_floor"] = round(PAIRS / 64 * MICROBENCH_CYCLES[k] / SIMD_HZ * 1e3 / ms, 4)
            if k == "inf_fwd":
                # the p = inf forward looks only at the k-tiles that can hold a maximum (on this data: one or two of
                # 160 per row of x): its rates are algorithmic (all pairs counted over the time of pre-pass + plan
                # + hot-tile kernel), not a measure of instruction issue
                d["note"] = "hot k-tiles only: algorithmic rates"
        else:
            nbytes = 4 * (2 * B * CO + B * CI + CO * CI)  # grad_out + pos read, grad_x + grad_w written
            d["gbs"] = round(nbytes / ms / 1e6, 1)
            d["frac_hbm_peak"] = round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)
        parts[k] = d

    dom = avg["p8_bwd"]
    achieved = PAIRS * FLOP["p8_bwd"] / dom / 1e9
    roofline = {
        "bound": "valu",
        "kernel": "bwd_fused_kernel<7, true, 32, 16> (p = 8 backward, both gradients)",
        "achieved": round(achieved, 2),
        "peak": PEAK_FP32_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_FP32_TFLOPS, 4),
        "issue_model_frac": parts["p8_bwd"]["frac_issue_model"],
        "microbench_floor_frac": parts["p8_bwd"]["frac_microbench_floor"],
        "traffic": profiled_traffic_bytes(),
        "traffic_source": "profiles/pmc_bwd_fused_kernel_p8_b512_5120x5120.txt (rocprofv3 counters of an earlier "
                          "run of the same kernel; not measured by this run)",
    }

    out = {
        "metric": "norm_dist fwd+bwd ms at B512x5120x5120, p=8 and p=inf",
        "value": round(ms_per_step, 3),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "norm_dist forward+backward (grad_input, grad_weight) at p=8 then p=inf; "
                               "x [512,5120] N(0,1), w [5120,5120] N(0,1/5120), grad_out [512,5120] N(0,1), seed 2021",
                   "B": B, "CI": CI, "CO": CO, "groups": 1, "HW": 1},
        "parts": parts,
        "roofline": roofline,
    }
    if not args.no_other:
        out["other_workloads_ms"] = other_workloads(torch, _C, xd.detach(), wd.detach(), gd)
    if args.cpu_cols > 0:
        out["cpu_baseline"] = cpu_baseline(torch, x, w, g, args.cpu_cols)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
