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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run one 1 GiB device-to-device copy first (known traffic, to scale FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards by batch, "
              "see DESIGN.md)" % args.gpus, file=sys.stderr)
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
    spec = nets.resnet50()
    B = args.batch
    net = nets.GpuNet(spec, B)
    rng = np.random.default_rng(2025)
    images = rng.integers(0, 256, size=(B, 3, 224, 224))
    net.set_input(images)
    torch.cuda.synchronize()

    for _ in range(args.warmup):
        net.forward()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.time()
    e0.record()
    for _ in range(args.steps):
        net.forward()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.time() - t0) * 1000.0 / args.steps
    ms = e0.elapsed_time(e1) / args.steps
    logits = net.tensors[spec.output].to_numpy().reshape(B, -1)

    # per-kernel timing: the same steps again with events around every launch
    per = {}
    for _ in range(args.steps):
        for l, t in net.forward_timed():
            per[l.name] = per.get(l.name, 0.0) + t / args.steps
    convs = [l for l in spec.layers if (l.type == "conv" and l.groups == 1) or l.type == "fc"]
    conv_ms = sum(per[l.name] for l in convs)
    conv_ops = 2.0 * sum(net.layer_macs(l) for l in convs)
    all_ms = sum(per.values())
    all_bytes = sum(net.layer_bytes(l) for l in net.launched)
    achieved = conv_ops / (conv_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": "conv_igemm_kernel (all %d conv/fc launches of one forward)" % len(convs),
                "achieved": round(achieved, 2), "peak": PEAK_INT8_TOPS, "unit": "TOP/s", "frac": round(achieved / PEAK_INT8_TOPS, 4),
                "traffic": None, "launches_per_step": len(convs), "avg_launch_us": round(conv_ms * 1000.0 / len(convs), 2),
                "ops_per_step": conv_ops}
    hbm = all_bytes / (all_ms * 1e-3) / 1e9
    roofline_hbm = {"bound": "hbm", "kernel": "whole forward (%d launches)" % len(net.launched), "achieved": round(hbm, 1),
                    "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(hbm / PEAK_HBM_GBS, 4), "bytes_per_step": all_bytes,
                    "sum_kernel_ms": round(all_ms, 4)}

    result = {
        "metric": "int8 ResNet-50 images/sec @bs128 on 1 MI355X", "value": round(B / (ms * 1e-3), 1), "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "resnet50_int8_ptq_forward_224", "global_batch": B, "input": "uint8 %dx3x224x224" % B,
                   "layers": len(spec.layers), "gmac_per_image": round(spec.macs_per_image() / 1e9, 3)},
        "roofline": roofline, "roofline_hbm": roofline_hbm,
    }
    if not args.no_cpu_baseline:
        base, exact = cpu_baseline(spec, logits, images)
        result["cpu_baseline"] = base
        result["bit_exact_vs_cpu"] = exact
    print(json.dumps(result))


if __name__ == "__main__":
    main()
