"""Headline benchmark: int8 ResNet-50 forward (8-bit PTQ, batch 128, 224x224) on one MI355X.

One "step" is one forward pass of the whole quantized network over one synthetic batch that is already resident in
HBM.  Prints ONE JSON line with images/s, the roofline of the dominant kernel (the int8-MFMA implicit-GEMM conv,
measured with events on the launch stream) and the CPU baseline (the reference algorithm's restatement timed on the
host cores of the same machine, on a bounded sample).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0      # MI355X dense int8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, GB/s
# HBM bytes one conv_pipe_kernel launch of this workload moves on average, as counted by rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE (KiB per dispatch, scaled by what the same counters read for a 1 GiB copy).  Counters cannot be read
# inside this run: the figure is quoted from the named summary, for the batch size it was taken at, and is not `traffic`.
TRAFFIC_FROM_PROFILE = {"file": "profiles/resnet50_bs128_forward_kernels_and_counters.txt", "kernel": "conv_pipe_kernel", "batch": 128,
                        "bytes_per_launch": 56975238, "launches_per_forward": 29,
                        "note": "FETCH_SIZE + WRITE_SIZE, mean over the conv_pipe_kernel dispatches of 4 forwards, scaled by a 1 GiB copy; "
                                "not measured by this run"}


def cpu_baseline(spec, gpu_logits, images, budget_s=15.0):
    """Times the CPU oracle (port of the reference Frame cells, OpenMP over the host cores) on a bounded sample of
    the same workload and checks the GPU logits of those images against it."""
    import numpy as np
    from oracle import cells
    t0 = time.time()
    out = cells.run_net(spec, images[:1])[spec.output]
    t1 = time.time() - t0
    n = int(max(1, min(images.shape[0] - 1, budget_s / max(t1, 1e-3))))
    t0 = time.time()
    out_n = cells.run_net(spec, images[1:1 + n])[spec.output]
    dt = time.time() - t0
    want = np.concatenate([out, out_n]).astype(np.int64).reshape(1 + n, -1)
    exact = bool(np.array_equal(want, gpu_logits[:1 + n]))
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or len(os.sched_getaffinity(0))
    return {"value": round(n / dt, 4), "unit": "images/s", "cores": cores, "kind": "port",
            "sample": "%d images of the same ResNet-50 forward (batch %d, 224x224), oracle/frame_oracle.c with OpenMP" % (n, n)}, exact


def class_rooflines(net, per_launch_ms, step_ms):
    """Every launch of a forward against the larger of its two bounds (2 * MAC at the int8 matrix peak, algorithmic bytes
    at the HBM peak), summed per class: convolutions / fully-connected cells whose larger bound is the matrix cores,
    those whose larger bound is memory, depthwise convolutions and the other bandwidth cells (pooling, sums, scalings)."""
    classes, floor_ms = {}, 0.0
    for l, t in zip(net.launched, per_launch_ms):
        ops, nbytes = 2.0 * net.layer_macs(l), float(net.layer_bytes(l))
        t_mfma, t_hbm = ops / (PEAK_INT8_TOPS * 1e12) * 1e3, nbytes / (PEAK_HBM_GBS * 1e9) * 1e3
        floor_ms += max(t_mfma, t_hbm)
        if l.type == "conv" and getattr(l, "groups", 1) > 1:
            name = "depthwise_hbm_bound"
        elif l.type in ("conv", "fc") or l.name in net.fused_sums or l.name in net.stem_pools:
            name = "mfma_bound" if t_mfma > t_hbm else "hbm_bound"
        else:
            name = "bandwidth_cells_hbm_bound"
        c = classes.setdefault(name, {"launches": 0, "ms": 0.0, "ops": 0.0, "bytes": 0.0})
        c["launches"] += 1; c["ms"] += t; c["ops"] += ops; c["bytes"] += nbytes
    out = {}
    for name, c in classes.items():
        if name == "mfma_bound":
            ach, peak, unit = c["ops"] / (c["ms"] * 1e-3) / 1e12, PEAK_INT8_TOPS, "TOP/s"
        else:
            ach, peak, unit = c["bytes"] / (c["ms"] * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
        out[name] = {"launches": c["launches"], "ms": round(c["ms"], 4), "achieved": round(ach, 1), "peak": peak, "unit": unit,
                     "frac": round(ach / peak, 4)}
    out["floor_ms"] = round(floor_ms, 4)               # sum over launches of the larger bound
    out["floor_frac"] = round(floor_ms / step_ms, 4)   # of the measured step
    return out


def launch_floor_us(torch, n=64):
    """What one kernel launch costs inside a replayed HIP graph when it depends on the one before it and does next to no
    work: n one-wave kernels, one behind the other, in one graph; median replay time / n."""
    import numpy as np
    t = torch.zeros(64, dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        t.add_(1)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(n):
                t.add_(1)
    torch.cuda.synchronize()
    ms, _, _ = median_step_ms(torch, graph.replay, 20, 3)
    return ms * 1000.0 / n


def median_step_ms(torch, step, steps, warmup, per_call=1):
    """Median and mean, per forward, of `steps` forwards; one call of `step` runs `per_call` of them (a HIP graph that holds
    several forwards), and each call sits between its own pair of events on the launch stream.  `steps` and `warmup` count
    forwards; `steps` must be a multiple of `per_call`."""
    import numpy as np
    assert steps % per_call == 0, (steps, per_call)
    for _ in range((warmup + per_call - 1) // per_call):
        step()
    torch.cuda.synchronize()
    calls = steps // per_call
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(calls + 1)]
    t0 = time.time()
    evs[0].record()
    for k in range(calls):
        step()
        evs[k + 1].record()
    torch.cuda.synchronize()
    wall = (time.time() - t0) * 1000.0 / steps
    per = [evs[k].elapsed_time(evs[k + 1]) / per_call for k in range(calls)]
    return float(np.median(per)), float(np.mean(per)), wall


def other_configs(torch, with_cpu):
    """The other four configurations at their full batch sizes: images/s of HIP graph replays (median of 10 replays),
    the per-class roofline of a forward, and (CPU leg) the GPU result against the CPU oracle: LeNet and the single stage
    convolution in full, with the oracle's own time as their CPU baseline; MobileNet-v1 and ResNet-18 W4A4 on the first
    two images of the batch."""
    import numpy as np
    from n2d2_amd import nets
    from oracle import cells
    out = {}
    rng = np.random.default_rng(77)
    for name, make, batch, full in (("lenet_8bit_bs256", nets.lenet, 256, True), ("resnet18_stage_conv_bs64", nets.single_conv_stage, 64, True),
                                    ("mobilenet_v1_8bit_bs64", nets.mobilenet_v1, 64, False), ("resnet18_w4a4_bs64", nets.resnet18_w4a4, 64, False)):
        spec = make()
        x = rng.integers(0, 256, size=(batch,) + tuple(spec.in_shape))
        net = nets.GpuNet(spec, batch)
        net.set_input(x)
        got = net.forward().to_numpy().astype(np.int64)
        # a graph holds 16 forwards of a network of a few launches, 4 of a larger one: replaying a graph costs about
        # 18 us once, which would otherwise be most of what a one-kernel network is timed at
        per_graph = 16 if len(net.launched) <= 8 else 4
        # (the single stage convolution is an inner layer: its input is another cell's output, already in the form cells
        # exchange, not a graph edge)
        at_edge = name != "resnet18_stage_conv_bs64"
        replay = net.capture(per_graph, with_input_conversion=at_edge)
        ms, mean_ms, _ = median_step_ms(torch, replay, 10 * per_graph, per_graph, per_graph)
        fwd_ms = ms
        if at_edge:     # the forward alone, as earlier bench lines timed these configurations
            replay_fwd = net.capture(per_graph)
            fwd_ms, _, _ = median_step_ms(torch, replay_fwd, 10 * per_graph, per_graph, per_graph)
            del replay_fwd
        runs = [net.forward_timed() for _ in range(5)]
        per_launch = [float(np.median([r[k][1] for r in runs])) for k in range(len(net.launched))]
        entry = {"batch": batch, "value": round(batch / (ms * 1e-3), 1), "unit": "images/s", "ms_per_step": round(ms, 4),
                 "step_is": "graph-edge conversion of the resident byte planes + forward" if at_edge else "forward (input resident as cells exchange it)",
                 "forward_without_edge_conversion_ms": round(fwd_ms, 4), "images_per_s_forward_only": round(batch / (fwd_ms * 1e-3), 1),
                 "launches": len(net.launched) + (1 if at_edge else 0), "forwards_per_graph": per_graph, "gmac_per_image": round(spec.macs_per_image() / 1e9, 4),
                 "roofline_by_class": class_rooflines(net, per_launch, ms)}
        if with_cpu:
            n = batch if full else 2
            t0 = time.time()
            want = cells.run_net(spec, x[:n])[spec.output].astype(np.int64)
            dt = time.time() - t0
            entry["bit_exact_vs_cpu"] = bool(np.array_equal(got[:n].reshape(n, -1), want.reshape(n, -1)))
            entry["cpu_baseline"] = {"value": round(n / dt, 3), "unit": "images/s", "kind": "port",
                                     "cores": int(os.environ.get("OMP_NUM_THREADS", 0)) or len(os.sched_getaffinity(0)),
                                     "sample": ("the whole batch" if full else "the first %d images of the batch" % n)}
        out[name] = entry
        del net, replay
    return out


PEAK_FP32_TFLOPS = 157.3


def qat_conv_step(torch, steps=10):
    """The float side of the path, reported beside the headline: one quantization-aware training iteration of a
    ResNet-18 stage convolution (64 -> 64 channels, 3x3, 56x56, batch 64) through the C ABI: SAT weight quantization,
    convolution, SAT activation quantization (range 15), then their backward passes, backward-filter, backward-data and
    the SGD update.  Timed with events on the stream the kernels are launched on; flops are those of the three
    convolution passes."""
    import ctypes as C
    from n2d2_amd import capi, runtime
    lib, sp, chk = capi.lib, runtime.stream_ptr, capi.check
    B, Cn, H, O, k = 64, 64, 56, 64, 3
    d = capi.ConvDesc(Cn, O, k, k, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0)
    gen = torch.Generator(device="cuda").manual_seed(5)
    f32 = dict(dtype=torch.float32, device="cuda")
    x = torch.rand(B, Cn, H, H, generator=gen, **f32) * 6
    w = torch.randn(O, Cn, k, k, generator=gen, **f32) * 0.05
    wq, dwq, dw = torch.empty_like(w), torch.empty_like(w), torch.empty_like(w)
    y = torch.empty(B, O, H, H, **f32)
    fp, dy, dx = torch.empty_like(y), torch.randn(B, O, H, H, generator=gen, **f32), torch.empty_like(x)
    stats, alpha, dalpha = torch.zeros(2, **f32), torch.full((1,), 6.0, **f32), torch.zeros(1, **f32)
    n, nw = y.numel(), w.numel()
    wsq = torch.empty(int(lib.n2d2hip_quantizer_workspace_bytes(max(n, nw))), dtype=torch.uint8, device="cuda")
    need = int(lib.n2d2hip_conv2d_f32_workspace_bytes(C.byref(d), B, H, H))
    wsf = torch.empty(max(need, 4), dtype=torch.uint8, device="cuda")
    g = torch.empty_like(y)

    def step():
        s = sp()
        chk(lib.n2d2hip_sat_weight_forward(w.data_ptr(), wq.data_ptr(), nw, 15.0, capi.SAT_DEFAULT, 0, 1, stats.data_ptr(), wsq.data_ptr(), wsq.numel(), s))
        chk(lib.n2d2hip_conv2d_f32_forward(C.byref(d), B, H, H, x.data_ptr(), wq.data_ptr(), None, 0.0, y.data_ptr(), wsf.data_ptr(), need, s))
        chk(lib.n2d2hip_sat_act_forward(y.data_ptr(), fp.data_ptr(), n, 15.0, alpha.data_ptr(), s))
        chk(lib.n2d2hip_sat_act_backward(dy.data_ptr(), fp.data_ptr(), g.data_ptr(), n, 15.0, alpha.data_ptr(), 0.0, dalpha.data_ptr(),
                                         wsq.data_ptr(), wsq.numel(), s))
        chk(lib.n2d2hip_conv2d_f32_backward_filter(C.byref(d), B, H, H, x.data_ptr(), g.data_ptr(), 0.0, dwq.data_ptr(), wsf.data_ptr(), need, s))
        chk(lib.n2d2hip_conv2d_f32_backward_data(C.byref(d), B, H, H, wq.data_ptr(), g.data_ptr(), 0.0, dx.data_ptr(), wsf.data_ptr(), need, s))
        chk(lib.n2d2hip_sat_weight_backward(dwq.data_ptr(), w.data_ptr(), dw.data_ptr(), nw, 15.0, capi.SAT_DEFAULT, 0, stats.data_ptr(), s))
        chk(lib.n2d2hip_sgd_update_f32(w.data_ptr(), dw.data_ptr(), nw, 0.01 / B, 0.0, 0.0, None, 0, 0.0, 0.0, s))
        chk(lib.n2d2hip_sgd_update_f32(alpha.data_ptr(), dalpha.data_ptr(), 1, 0.01 / B, 0.0, 0.0, None, 0, 0.0, 0.0, s))
    for _ in range(2):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    flops = 3 * 2.0 * B * O * H * H * Cn * k * k
    ach = flops / (ms * 1e-3) / 1e12
    return {"workload": "SAT QAT iteration of one 64->64 3x3 convolution on 56x56, batch 64, float32", "ms_per_iteration": round(ms, 4),
            "bound": "mfma", "achieved": round(ach, 2), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / PEAK_FP32_TFLOPS, 4),
            "finite": bool(torch.isfinite(w).all().item() and torch.isfinite(alpha).all().item())}


def qat_batchnorm_step(torch, steps=10):
    """BatchNorm of the same learning graph (64 channels on 56x56, batch 64, float32): learning forward (batch statistics,
    running statistics, normalisation) and backward (parameter and input gradients) through the C ABI, timed with events
    on the stream the kernels are launched on; bytes are the algorithmic ones, 16 and 20 per value."""
    from n2d2_amd import capi, runtime
    lib, sp, chk = capi.lib, runtime.stream_ptr, capi.check
    B, Cn, H = 64, 64, 56
    n = B * Cn * H * H
    gen = torch.Generator(device="cuda").manual_seed(6)
    f32 = dict(dtype=torch.float32, device="cuda")
    x, dy = torch.randn(n, generator=gen, **f32), torch.randn(n, generator=gen, **f32)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    vec = lambda v: torch.full((Cn,), v, **f32)
    scale, bias, mean, var, smean, svar, dscale, dbias, dsm, dsv = (vec(1.0), vec(0.0), vec(0.0), vec(1.0), vec(0.0), vec(1.0), vec(0.0), vec(0.0),
                                                                    vec(0.0), vec(0.0))
    nws = int(lib.n2d2hip_batchnorm_f32_workspace_bytes(B, Cn, H, H))
    ws = torch.empty(nws, dtype=torch.uint8, device="cuda")

    def fwd():
        chk(lib.n2d2hip_batchnorm_f32_forward(B, Cn, H, H, x.data_ptr(), scale.data_ptr(), bias.data_ptr(), mean.data_ptr(), var.data_ptr(),
                                              smean.data_ptr(), svar.data_ptr(), 1e-5, 0.1, 0, y.data_ptr(), ws.data_ptr(), nws, sp()))

    def bwd():
        chk(lib.n2d2hip_batchnorm_f32_backward(B, Cn, H, H, x.data_ptr(), scale.data_ptr(), smean.data_ptr(), svar.data_ptr(), 1e-5, dy.data_ptr(),
                                               0.0, dscale.data_ptr(), 0.0, dbias.data_ptr(), dsm.data_ptr(), dsv.data_ptr(), dx.data_ptr(),
                                               ws.data_ptr(), nws, sp()))

    def timed(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps
    tf, tb = timed(fwd), timed(bwd)
    gf, gb = 16.0 * n / (tf * 1e-3) / 1e9, 20.0 * n / (tb * 1e-3) / 1e9
    return {"workload": "BatchNorm learning pass, 64 channels on 56x56, batch 64, float32", "bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "forward": {"us": round(tf * 1e3, 1), "achieved": round(gf, 1), "frac": round(gf / PEAK_HBM_GBS, 4)},
            "backward": {"us": round(tb * 1e3, 1), "achieved": round(gb, 1), "frac": round(gb / PEAK_HBM_GBS, 4)},
            "finite": bool(torch.isfinite(y).all().item() and torch.isfinite(dx).all().item())}


def kernel_phases(torch, config, batch):
    """Where the time of a launch goes inside the kernel, per instantiation, from the probes of a library built with
    `python -m n2d2_amd.build --probe` (run with N2D2HIP_LIB=n2d2_amd/lib/libn2d2hip_probe.so): every work-group of the
    convolution kernels records its shader clock at its first instruction, at its first operand load, when its first ring
    stage has landed, and at its end, the clocks its epilogues took, and the constant 100 MHz counter at both ends
    (include/n2d2hip_probe.h).  One forward is probed after three warm ones; prints a text table."""
    import ctypes as C
    import numpy as np
    from n2d2_amd import capi, nets
    if not hasattr(capi.lib, "n2d2hip_probe_begin"):
        print("bench.py --kernel-phases needs the probe build: python -m n2d2_amd.build --probe, then "
              "N2D2HIP_LIB=n2d2_amd/lib/libn2d2hip_probe.so python bench.py --kernel-phases", file=sys.stderr)
        sys.exit(5)
    capi.lib.n2d2hip_probe_begin.argtypes = [C.c_void_p, C.c_size_t]
    capi.lib.n2d2hip_probe_end.argtypes = [C.c_void_p]
    make, default_batch = CONFIGS[config]
    spec = getattr(nets, make)()
    B = batch or default_batch
    net = nets.GpuNet(spec, B)
    net.set_input(np.random.default_rng(2025).integers(0, 256, size=(B,) + tuple(spec.in_shape)))
    for _ in range(3):
        net.forward()
    torch.cuda.synchronize()
    REC = 16
    buf = torch.zeros(REC * 65536, dtype=torch.int64, device="cuda")
    capi.check(capi.lib.n2d2hip_probe_begin(buf.data_ptr(), buf.numel() * 8))
    launches = []
    for k, ((l, cell, fn), (ins, out)) in enumerate(zip(net.steps, net._io)):
        with capi.launch_log() as log:
            fn(cell, ins, out)
        launches += [(l.name,) + e for e in log.entries]
    torch.cuda.synchronize()
    capi.check(capi.lib.n2d2hip_probe_end(None))
    rec = buf.cpu().numpy().reshape(-1, REC).astype(np.float64)
    rows = {}
    for lname, kname, grid, block, slot in launches:
        if slot < 0:
            continue
        r = rec[slot:slot + grid]
        r = r[(r[:, 5] != 0) & (r[:, 7] > 0)]     # work-groups that had work
        if len(r) == 0:
            continue
        w0, w1 = r[:, 5], r[:, 6]
        span_us = (w1.max() - w0.min()) / 100.0
        mhz = ((r[:, 3] - r[:, 0]).sum() / ((w1 - w0).sum() / 100.0))        # shader clocks per microsecond
        has12 = r[:, 2].max() > 0
        d = {"launches": 1, "blocks": len(r), "span_us": span_us,
             "start_spread_us": (w0.max() - w0.min()) / 100.0,
             "to_first_load_us": float(np.mean(r[:, 1] - r[:, 0]) / mhz) if has12 else float("nan"),
             "to_first_mfma_us": float(np.mean(r[:, 2] - r[:, 0]) / mhz) if has12 else float("nan"),
             "block_life_us": float(np.mean(w1 - w0) / 100.0),
             "epilogue_us": float(np.mean(r[:, 4]) / mhz),
             "per_unit_us": float(np.mean((r[:, 3] - (r[:, 2] if has12 else r[:, 0])) / np.maximum(r[:, 7], 1)) / mhz),
             "units": float(np.mean(r[:, 7])),
             "end_spread_us": (w1.max() - w1.min()) / 100.0,
             "idle_frac": 1.0 - float((w1 - w0).sum() / 100.0) / (span_us * len(r)),
             "mhz": mhz}
        if r[:, 8:14].max() > 0:          # kernels that time their phases: mean microseconds per unit of work
            d["phases_us"] = [float(np.mean(r[:, 8 + k] / np.maximum(r[:, 7], 1)) / mhz) for k in range(6)]
        a = rows.setdefault(kname, [])
        a.append(d)
    keys = ["blocks", "span_us", "start_spread_us", "to_first_load_us", "to_first_mfma_us", "block_life_us", "units", "per_unit_us",
            "epilogue_us", "end_spread_us", "idle_frac", "mhz"]
    print("%s, batch %d: in-kernel phases per instantiation (mean over its launches of one forward; times in us)" % (config, B))
    print("span = first work-group's start to last work-group's end; start_spread = last start - first start; to_first_load /"
          " to_first_mfma = from a work-group's first instruction (mean over work-groups); block_life = a work-group's start to"
          " its end; units = ring steps (tiles for the bottleneck kernel) per work-group; per_unit = (end - first mfma) / units;"
          " epilogue = clocks in epilogues per work-group; end_spread = last end - first end; idle_frac = 1 - sum of work-group"
          " lives / (span x work-groups); mhz = shader clocks per microsecond inside the kernel")
    print("%-64s %3s " % ("kernel", "n") + " ".join("%12s" % k[:12] for k in keys))
    for kname, lst in sorted(rows.items(), key=lambda kv: -sum(d["span_us"] for d in kv[1])):
        def col(k):
            vals = [d[k] for d in lst if d[k] == d[k]]      # (a kernel without that mark leaves a NaN)
            return "%12.2f" % float(np.mean(vals)) if vals else "%12s" % "-"
        print("%-64s %3d " % (kname[:64], len(lst)) + " ".join(col(k) for k in keys))
    for kname, lst in rows.items():
        if "phases_us" in lst[0]:
            print("%s: microseconds per unit of work in its phases 0..5 (see the kernel's source): %s" % (
                kname, " ".join("%.3f" % float(np.mean([d["phases_us"][k] for d in lst])) for k in range(6))))
    total = sum(d["span_us"] for lst in rows.values() for d in lst)
    print("sum of spans of the probed launches: %.1f us (%d launches of %d in the forward)" % (total, sum(len(v) for v in rows.values()), len(launches)))


# name -> (constructor in n2d2_amd.nets, benchmark batch)
CONFIGS = {"resnet50": ("resnet50", 128), "lenet": ("lenet", 256), "resnet18_stage_conv": ("single_conv_stage", 64),
           "mobilenet_v1": ("mobilenet_v1", 64), "resnet18_w4a4": ("resnet18_w4a4", 64)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--forwards-per-graph", type=int, default=4,
                    help="forwards recorded into the HIP graph that is replayed (lowered to a divisor of --steps); a replay "
                         "costs about 18 us once, whatever it holds")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=0, help="images per step (default: the configuration's own, 128 for the headline)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="only the headline workload")
    ap.add_argument("--no-graph", action="store_true", help="time cell-by-cell launches instead of a HIP graph replay")
    ap.add_argument("--forward-only", action="store_true",
                    help="profiling runs: time the forward of --config and stop (no per-kernel replays, no side figures)")
    ap.add_argument("--config", default="resnet50", choices=sorted(CONFIGS),
                    help="with --forward-only: which configuration's forward to run (at its benchmark batch unless --batch is given)")
    ap.add_argument("--kernel-phases", action="store_true",
                    help="probe build only (python -m n2d2_amd.build --probe; N2D2HIP_LIB=n2d2_amd/lib/libn2d2hip_probe.so): "
                         "print where the time goes inside the convolution kernels of --config, per instantiation, and stop")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run one 1 GiB device-to-device copy first (known traffic, to scale FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards by batch: one process "
              "per GPU on its slice of the images, no exchange step)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from n2d2_amd import nets

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    if args.copy_calibration:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.kernel_phases:
        kernel_phases(torch, args.config, args.batch)
        return
    import math
    per_graph = math.gcd(max(args.forwards_per_graph, 1), args.steps)
    if args.forward_only:
        make, batch = CONFIGS[args.config]
        spec = getattr(nets, make)()
        B = args.batch or batch
        net = nets.GpuNet(spec, B)
        net.set_input(np.random.default_rng(2025).integers(0, 256, size=(B,) + tuple(spec.in_shape)))
        def eager():
            net.convert_input()
            return net.forward()
        step = eager if args.no_graph else net.capture(per_graph, with_input_conversion=True)
        ms, mean_ms, wall_ms = median_step_ms(torch, step, args.steps, args.warmup, 1 if args.no_graph else per_graph)
        print(json.dumps({"forward_only": args.config, "batch": B, "value": round(B / (ms * 1e-3), 1), "unit": "images/s",
                          "ms_per_step": round(ms, 4), "launches_per_step": len(net.launched) + 1, "step_is": "graph-edge conversion + forward",
                          "launch": "eager" if args.no_graph else "hipGraph replay, %d forwards per graph" % per_graph,
                          "steps": args.steps, "warmup": args.warmup}))
        return
    spec = nets.resnet50()
    B = args.batch or 128
    net = nets.GpuNet(spec, B)
    rng = np.random.default_rng(2025)
    images = rng.integers(0, 256, size=(B, 3, 224, 224))
    net.set_input(images)
    torch.cuda.synchronize()

    def timed(step, per_call=1):
        return median_step_ms(torch, step, args.steps, args.warmup, per_call)

    # one step = the graph-edge conversion of the uint8 NCHW batch (resident in HBM) into the first cell's layout, then one
    # forward of the whole network; launched cell by cell ("eager") and from a HIP graph that holds `per_graph` steps one
    # behind the other (each replay is timed and divided by that number)
    def eager_step():
        net.convert_input()
        return net.forward()
    eager_ms, eager_mean_ms, eager_wall_ms = timed(eager_step)
    eager_logits = net.tensors[spec.output].to_numpy().reshape(B, -1)
    if args.no_graph:
        ms, mean_ms, wall_ms, launch = eager_ms, eager_mean_ms, eager_wall_ms, "eager"
    else:
        replay = net.capture(per_graph, with_input_conversion=True)
        ms, mean_ms, wall_ms = timed(replay, per_graph)
        launch = "hipGraph replay, %d forwards per graph" % per_graph
    # the conversion alone, and the forward without it (what earlier bench lines called a step)
    edge_ms, _, _ = timed(net.convert_input)
    if args.no_graph:
        forward_ms = timed(net.forward)[0]
    else:
        forward_ms = timed(net.capture(per_graph), per_graph)[0]
    logits = net.tensors[spec.output].to_numpy().reshape(B, -1)
    if not np.array_equal(logits, eager_logits):
        print("bench.py: graph replay and eager launches disagree", file=sys.stderr)
        sys.exit(4)
    # the engine clock the chip holds under matrix-core load, right behind the timed steps: the published 5.0 POP/s assume
    # 2.4 GHz (256 CUs x 8192 int8 operations per clock)
    import ctypes as C
    from n2d2_amd import capi, runtime
    mhz = C.c_double(0.0)
    capi.check(capi.lib.n2d2hip_measure_clock(200.0, C.byref(mhz), runtime.stream_ptr()))
    clock = {"engine_clock_mhz_under_mfma_load": round(mhz.value, 1),
             "int8_peak_at_that_clock_tops": round(256 * 8192 * mhz.value * 1e6 / 1e12, 1)}

    # Which kernel runs a launch of the forward: asked of the library (its launch log names what every cell launched), so
    # the labels below cannot drift from what ran.
    launched_kernels = net.kernel_names()

    def kernel_of(k):
        # the last kernel a cell launches does its arithmetic (a cell with several inputs gathers them first)
        name = launched_kernels[k][-1].split("<")[0]
        return name if name.startswith("conv_") or name.startswith("bottleneck") else "bandwidth"
    kernels = [kernel_of(k) for k in range(len(net.launched))]

    # Dominant kernel: conv_pipe_kernel.  Its launches are replayed alone, back to back, between two events on the launch
    # stream: elapsed / launches is the average launch duration (inter-launch gaps included).
    def replay_alone(idx):
        for _ in range(3):
            net.forward_subset(idx)
        torch.cuda.synchronize()
        p0, p1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        p0.record()
        for _ in range(args.steps):
            net.forward_subset(idx)
        p1.record()
        torch.cuda.synchronize()
        return p0.elapsed_time(p1) / args.steps
    pipe = [k for k, name in enumerate(kernels) if name == "conv_pipe_kernel"]
    conv_ms = replay_alone(pipe)
    conv_ops = 2.0 * sum(net.layer_macs(net.launched[k]) for k in pipe)
    achieved = conv_ops / (conv_ms * 1e-3) / 1e12
    profile_applies = B == TRAFFIC_FROM_PROFILE["batch"] and len(pipe) == TRAFFIC_FROM_PROFILE["launches_per_forward"]
    # Which roof bounds these launches: the larger of (their operations at the matrix cores' peak) and (their algorithmic
    # bytes at the memory's peak).  With the 3x3 layers on the patch kernel and the first block on the bottleneck kernel,
    # what is left on conv_pipe_kernel is mostly 1x1 layers: memory is the larger bound.  The other view is kept beside it.
    pipe_bytes = float(sum(net.layer_bytes(net.launched[k]) for k in pipe))
    achieved_gbs = pipe_bytes / (conv_ms * 1e-3) / 1e9
    hbm_bound = pipe_bytes / (PEAK_HBM_GBS * 1e9) >= conv_ops / (PEAK_INT8_TOPS * 1e12)
    mfma_view = {"achieved": round(achieved, 2), "peak": PEAK_INT8_TOPS, "unit": "TOP/s", "frac": round(achieved / PEAK_INT8_TOPS, 4)}
    hbm_view = {"achieved": round(achieved_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(achieved_gbs / PEAK_HBM_GBS, 4)}
    roofline = {"bound": "hbm" if hbm_bound else "mfma",
                "kernel": "conv_pipe_kernel (%d launches of one forward: conv/fc cells with a multiple of 64 input "
                "channels, residual sums folded in; not the cells of the launches that take a whole block or its 3x3 convolution, expansion "
                "and sum: conv_chain_kernel and bottleneck_kernel under roofline_kernels)" % len(pipe),
                "bound_is": "the larger of ops / int8 peak and algorithmic bytes / HBM peak over these launches",
                "floor_us_per_launch": {"mfma": round(conv_ops / (PEAK_INT8_TOPS * 1e12) * 1e6 / len(pipe), 2),
                                        "hbm": round(pipe_bytes / (PEAK_HBM_GBS * 1e9) * 1e6 / len(pipe), 2)},
                **(hbm_view if hbm_bound else mfma_view),
                "mfma_view": mfma_view, "hbm_view": hbm_view,
                # HBM bytes per launch cannot be counted from inside this process: the figure is the one the committed profile
                # holds, given only while this run launches what that profile covered (same batch, same number of launches)
                "traffic": TRAFFIC_FROM_PROFILE["bytes_per_launch"] if profile_applies else None,
                "traffic_from_profile": TRAFFIC_FROM_PROFILE if profile_applies else None,
                "algorithmic_bytes_per_launch": round(sum(net.layer_bytes(net.launched[k]) for k in pipe) / len(pipe)),
                "launches_per_step": len(pipe), "avg_launch_us": round(conv_ms * 1000.0 / len(pipe), 2),
                "ops_per_launch": conv_ops / len(pipe), "frac_of_peak_at_measured_clock": round(achieved / clock["int8_peak_at_that_clock_tops"], 4)}
    # the other convolution kernels of the forward, each replayed alone the same way
    roofline_kernels = {}
    for name in ("conv_chain_kernel", "conv_patch3x3_kernel", "bottleneck_kernel", "conv_s2d_kernel", "conv_stem_kernel"):
        idx = [k for k, kn in enumerate(kernels) if kn == name]
        if not idx:
            continue
        t = replay_alone(idx)
        ops = 2.0 * sum(net.layer_macs(net.launched[k]) for k in idx)
        nbytes = float(sum(net.layer_bytes(net.launched[k]) for k in idx))
        roofline_kernels[name] = {"launches": len(idx), "avg_launch_us": round(t * 1000.0 / len(idx), 2),
                                  "tops": round(ops / (t * 1e-3) / 1e12, 1), "frac_of_int8_peak": round(ops / (t * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4),
                                  "gbs": round(nbytes / (t * 1e-3) / 1e9, 1), "frac_of_hbm_peak": round(nbytes / (t * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
    all_bytes = sum(net.layer_bytes(l) for l in net.launched)
    hbm = all_bytes / (ms * 1e-3) / 1e9
    roofline_hbm = {"bound": "hbm", "kernel": "whole forward (%d launches)" % len(net.launched), "achieved": round(hbm, 1),
                    "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(hbm / PEAK_HBM_GBS, 4), "bytes_per_step": all_bytes}

    # Per-class view: every launch timed with its own pair of events (median of 7 forwards), put against the larger of
    # its two bounds.  The per-launch events add about 10 % to the sum, so the class times are an upper estimate of their
    # share of `ms_per_step`.
    runs = [net.forward_timed() for _ in range(7)]
    per_launch = [float(np.median([r[k][1] for r in runs])) for k in range(len(net.launched))]
    by_class = class_rooflines(net, per_launch, ms)
    # the same north_star figure over the convolution / fully-connected launches' own time (each between its own pair of
    # events, which adds about 10 % to their sum): what the kernels reach while they run, launch gaps left out
    conv_idx = [k for k, l in enumerate(net.launched) if net.layer_macs(l) > 0]
    conv_own_ms = sum(per_launch[k] for k in conv_idx)
    conv_frac_own_time = 2.0 * sum(net.layer_macs(net.launched[k]) for k in conv_idx) / (conv_own_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS
    # the same floor with what the launches themselves cost (measured on this GPU, in this run) added to it
    floor_us = launch_floor_us(torch)
    by_class["launch_floor_us"] = round(floor_us, 2)
    by_class["floor_with_launches_ms"] = round(by_class["floor_ms"] + len(net.launched) * floor_us * 1e-3, 4)
    by_class["floor_with_launches_frac"] = round(by_class["floor_with_launches_ms"] / ms, 4)

    # Two batches in flight: a second, independent forward of the same network on another batch of the same size runs on
    # its own stream, so each stream's launch gaps and tails are filled by the other's kernels.  Reported next to `value`
    # (which stays one batch at a time); both forwards are checked against their one-at-a-time results.
    overlapped = None
    if not args.no_graph:
        net2 = nets.GpuNet(spec, B)
        images2 = rng.integers(0, 256, size=(B, 3, 224, 224))
        net2.set_input(images2)
        want2 = net2.forward().to_numpy().reshape(B, -1)
        torch.cuda.synchronize()
        s1, s2, cap = torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.stream(cap):
            with torch.cuda.graph(graph2, stream=cap):
                fork = torch.cuda.Event()
                fork.record(cap)
                joins = []
                for n, st in ((net, s1), (net2, s2)):
                    st.wait_event(fork)
                    with torch.cuda.stream(st):
                        for _ in range(per_graph):
                            n.forward()
                        j = torch.cuda.Event()
                        j.record(st)
                        joins.append(j)
                for j in joins:
                    cap.wait_event(j)
        torch.cuda.synchronize()
        ms2, _, _ = timed(graph2.replay, per_graph)
        ok2 = (np.array_equal(net.tensors[spec.output].to_numpy().reshape(B, -1), eager_logits)
               and np.array_equal(net2.tensors[spec.output].to_numpy().reshape(B, -1), want2))
        if not ok2:
            print("bench.py: overlapped forwards disagree with the one-at-a-time results", file=sys.stderr)
            sys.exit(4)
        overlapped = {"batches_in_flight": 2, "value": round(2 * B / (ms2 * 1e-3), 1), "unit": "images/s",
                      "ms_per_pair_of_steps": round(ms2, 4), "bit_exact_vs_sequential": True}
        del net2, graph2

    result = {
        "metric": "int8 ResNet-50 images/sec @bs128 on 1 MI355X", "value": round(B / (ms * 1e-3), 1), "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "ms_per_step_is": "median over the graph replays of replay time / forwards per graph",
        "mean_ms_per_step": round(mean_ms, 4), "wall_ms_per_step": round(wall_ms, 4),
        "step_is": "graph-edge conversion of the resident uint8 NCHW batch + forward of the 84 cells",
        "edge_conversion_us": round(edge_ms * 1000.0, 2), "forward_without_edge_conversion_ms": round(forward_ms, 4),
        "launch": launch, "launches_per_step": len(net.launched) + 1, "eager_ms_per_step": round(eager_ms, 4),
        # north_star's figure: the operations of every convolution / fully-connected launch of a forward over the whole
        # measured step (pooling and the edge conversion included in the time), against the int8 matrix peak
        "conv_layers_frac_of_int8_peak": round(2.0 * spec.macs_per_image() * B / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4),
        "conv_layers_frac_of_int8_peak_over_their_own_launch_time": round(conv_frac_own_time, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "resnet50_int8_ptq_forward_224", "global_batch": B, "input": "uint8 %dx3x224x224" % B,
                   "layers": len(spec.layers), "gmac_per_image": round(spec.macs_per_image() / 1e9, 3)},
        "roofline": roofline, "roofline_kernels": roofline_kernels, "roofline_hbm": roofline_hbm, "roofline_by_class": by_class,
        "clock": clock,
    }
    if overlapped is not None:
        result["two_batches_in_flight"] = overlapped
    try:
        result["qat_conv_iteration"] = qat_conv_step(torch)
    except Exception as e:       # the side figure must not take the headline down with it
        result["qat_conv_iteration"] = {"error": "%s: %s" % (type(e).__name__, e)}
    try:
        result["qat_batchnorm"] = qat_batchnorm_step(torch)
    except Exception as e:
        result["qat_batchnorm"] = {"error": "%s: %s" % (type(e).__name__, e)}
    if not args.no_cpu_baseline:
        base, exact = cpu_baseline(spec, logits, images)
        result["cpu_baseline"] = base
        result["bit_exact_vs_cpu"] = exact
    if not args.no_other_configs:
        try:
            result["other_configs"] = other_configs(torch, not args.no_cpu_baseline)
        except Exception as e:
            result["other_configs"] = {"error": "%s: %s" % (type(e).__name__, e)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
