#!/usr/bin/env python3
"""Benchmark of the BNN inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--net imagenet_resnet] [--batch 256]
                    [--variant auto|popc|mfma_i8|mfma_f4] [--no-cpu] [--layers]

A step is one forward pass of the whole network (every layer, one launch each, one stream) over
one batch of seeded synthetic input that is already resident in HBM; weight packing and host
copies are outside the timed region (the reference times only its network kernel,
imagenet_resnet.cu:358-363).  Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PAPER_IMAGES_PER_S = 5600.0  # README.md:16 of the reference (ResNet-18, ImageNet, Turing)

# Rooflines.  VALU: 256 CU x 64 lane-ops/clk x 2.4 GHz = 39.3 T lane-op/s; one v_xor_b32 +
# one v_bcnt_u32_b32 (2 lane-ops) do 32 multiply-accumulates = 64 binary ops.
PEAKS = {
    "popc": ("valu", 256 * 64 * 2.4e9 / 2 * 64 / 1e12),  # 1258.3 T binary op/s
    "mfma_i8": ("mfma", 5000.0),                          # published dense int8, TOP/s
    "mfma_f4": ("mfma", 10100.0),                         # published dense fp4, TFLOP/s
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--net", default="imagenet_resnet", choices=["imagenet_resnet", "cifar10_vgg", "mnist_mlp"])
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--variant", default="auto")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-batch", type=int, default=None)
    ap.add_argument("--layers", action="store_true", help="also print a per-layer table to stderr")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build drives one GPU (one process, one device); --gpus %d is not supported. "
                 "The path shards by batch with replicated weights and no exchange inside the forward."
                 % args.gpus)

    import numpy as np
    import tcbnn_amd
    from tcbnn_amd import _lib, nets
    from tcbnn_amd.device import Event, Stream

    if _lib.device_count() < 1:
        sys.exit("bench.py: no HIP device visible")
    _lib.set_device(0)
    if args.variant != "auto":
        _lib.check(_lib.lib.tcbnn_set_default_variant(_lib.VARIANTS[args.variant]))
    variant = {v: k for k, v in _lib.VARIANTS.items()}[_lib.lib.tcbnn_get_default_variant()]

    default_batch = {"imagenet_resnet": 256, "cifar10_vgg": 256, "mnist_mlp": 8192}[args.net]
    batch = args.batch or default_batch
    spec = nets.SPECS[args.net](batch=batch)
    weights = tcbnn_amd.synthetic_weights(spec, seed=0)
    x = tcbnn_amd.synthetic_input(spec, seed=0)
    net = tcbnn_amd.Network(spec, weights, x)
    stream = Stream()
    bops, flops = nets.binary_ops(spec)

    # ------------------------------------------------------------------ timed region
    for _ in range(args.warmup):
        net.forward(stream)
    stream.synchronize()
    _lib.device_synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.forward(stream)
    stream.synchronize()
    _lib.device_synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    images_per_s = batch * args.steps / wall

    # ------------------------------------------------------------------ per-launch timing (HIP events
    # on the launch stream), outside the timed region
    per_layer = {L["name"]: [] for L in spec}
    evs = [Event() for _ in range(len(spec) + 1)]
    for _ in range(max(3, min(args.steps, 10))):
        evs[0].record(stream)
        for i, layer in enumerate(net.order):
            layer.forward(stream)
            evs[i + 1].record(stream)
        stream.synchronize()
        for i, L in enumerate(spec):
            per_layer[L["name"]].append(evs[i].elapsed_ms(evs[i + 1]))
    layer_ms = {k: float(np.median(v)) for k, v in per_layer.items()}

    # group launches by device kernel, as a profiler does
    groups = {}
    for L, layer in zip(spec, net.order):
        if L["kind"] in ("conv", "fc"):
            name = layer.kernel_name()
            ops = nets.binary_ops([L])[0]
            g = groups.setdefault(name, dict(ops=0.0, ms=0.0, launches=0))
            g["ops"] += ops
            g["ms"] += layer_ms[L["name"]]
            g["launches"] += 1
    dom_name, dom = max(groups.items(), key=lambda kv: kv[1]["ms"])
    bound, peak = PEAKS[variant]
    achieved = dom["ops"] / (dom["ms"] * 1e-3) / 1e12
    roofline = {
        "bound": bound, "achieved": round(achieved, 2), "peak": round(peak, 1), "unit": "TOP/s",
        "frac": round(achieved / peak, 4), "traffic": None, "kernel": dom_name,
        "launches_per_step": dom["launches"], "avg_launch_ms": round(dom["ms"] / dom["launches"], 4),
        "algorithmic_ops_per_launch": dom["ops"] / dom["launches"],
        "bit_layers_tops": round(sum(g["ops"] for g in groups.values()) /
                                 (sum(g["ms"] for g in groups.values()) * 1e-3) / 1e12, 2),
    }

    if args.layers:
        sys.stderr.write("%-8s %-34s %10s %10s\n" % ("layer", "kernel", "ms", "TOP/s"))
        for L, layer in zip(spec, net.order):
            ops = nets.binary_ops([L])[0]
            kn = layer.kernel_name() if hasattr(layer, "kernel_name") else L["kind"]
            ms = layer_ms[L["name"]]
            sys.stderr.write("%-8s %-34s %10.4f %10.1f\n" % (L["name"], kn, ms, ops / (ms * 1e-3) / 1e12))
        sys.stderr.write("sum of layers: %.4f ms; step: %.4f ms\n" % (sum(layer_ms.values()), ms_per_step))

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    cpu = None
    if not args.no_cpu:
        from oracle import nets as orc_nets, orc
        cb = args.cpu_batch or {"imagenet_resnet": 16, "cifar10_vgg": 64, "mnist_mlp": 8192}[args.net]
        cb = min(cb, batch)
        cspec = nets.SPECS[args.net](batch=cb)
        xs = x[:cb]
        orc_nets.run(cspec, weights, xs)  # warm-up (page-in, thread pool)
        t0 = time.perf_counter()
        reps = 0
        while True:
            cpu_out = orc_nets.run(cspec, weights, xs)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 10:
                break
        cpu_s = (time.perf_counter() - t0) / reps
        # the GPU result of the same images must agree with what the CPU leg just computed
        got = net.logits()[:cb]
        np.testing.assert_allclose(got, cpu_out[spec[-1]["name"]]["out"], rtol=1e-5, atol=0)
        cpu = {"value": round(cb / cpu_s, 2), "unit": "images/s", "cores": orc.num_threads(), "kind": "port",
               "sample": "%s forward, batch %d, mean of %d reps after 1 warm-up, OpenMP XOR/popcount "
                         "(64-bit words), same seeds" % (args.net, cb, reps),
               "binary_tops": round(nets.binary_ops(cspec)[0] / cpu_s / 1e12, 4)}

    out = {
        "metric": "images/sec ResNet-18 BNN 224x224 batch 256 on 1 MI355X" if args.net == "imagenet_resnet"
        else "images/sec %s batch %d on 1 MI355X" % (args.net, batch),
        "value": round(images_per_s, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": round(images_per_s / PAPER_IMAGES_PER_S, 2) if args.net == "imagenet_resnet" and batch == 256
        else None,
        "dtype": "u32 xor+popcount -> int32" if variant == "popc" else
        ("int8 mfma -> int32" if variant == "mfma_i8" else "fp4 mfma -> fp32 (exact integers)"),
        "data": "synthetic",
        "config": {"workload": "%s, reference topology (%s), batch %d, seeded synthetic weights and input"
                               % (args.net, {"imagenet_resnet": "imagenet_resnet.cu:223-325",
                                             "cifar10_vgg": "cifar10_vgg.cu:162-199",
                                             "mnist_mlp": "mnist_mlp.cu:111-124"}[args.net], batch),
                   "variant": variant, "layers": len(spec)},
        "binary_tops": round(bops * args.steps / wall / 1e12, 2),
        "binary_ops_per_step": bops, "fp32_first_layer_flops_per_step": flops,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    net.release()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
