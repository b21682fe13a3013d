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

# Published MI355X peaks.  The XOR+popcount engine runs on the VALU, for which there is no
# published figure: 256 CU x 64 lane-ops/clk x 2.4 GHz = 39.3 T lane-op/s, and one v_xor_b32 +
# one v_bcnt_u32_b32 (2 lane-ops) do 32 multiply-accumulates = 64 binary ops.
HBM_PEAK_GBS = 8000.0
COMPUTE_PEAKS_TOPS = {
    "popc": ("valu", 256 * 64 * 2.4e9 / 2 * 64 / 1e12),  # 1258.3 T binary op/s
    "mfma_i8": ("mfma", 5000.0),                          # dense int8
    "mfma_f4": ("mfma", 10100.0),                         # dense fp4
}

# HBM bytes per launch (roofline.traffic) are not measured in this process: hardware counters need a profiler run
# of their own.  They are read from a data file under profiles/ that records the rocprofv3 commands, the commit
# and a digest of the kernel sources it was measured on.  When the kernel sources have changed since (or the file
# is missing, or names no figure for a kernel), traffic is null and traffic_stale says why.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_resnet18_b256_fp4.json")


def kernel_source_digest():
    """sha256 over the device sources and headers the library is built from (names and contents, sorted)."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "tcbnn_amd", "csrc")
    for name in sorted(os.listdir(src)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(src, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def load_measured_traffic():
    """(bytes per launch by kernel name, stale flag, note)."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return {}, True, "no traffic file"
    if rec.get("kernel_source_sha256") != kernel_source_digest():
        return {}, True, "kernel sources changed since the counters were read (commit %s)" % rec.get("git_commit")
    return rec.get("bytes_per_launch", {}), False, "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at commit %s" % rec.get("git_commit")


MEASURED_TRAFFIC_BYTES, TRAFFIC_STALE, TRAFFIC_NOTE = {}, True, "not loaded"


def layer_work(L, spec=(), res_bytes=None, pooled=()):
    """Algorithmic work of one layer launch: binary ops (2 per +-1 multiply-accumulate, border taps
    included), fp32 adds of the first layer, and the HBM bytes the launch has to move once
    (inputs + outputs + weights, packed activations at 1 bit per value, residuals at the width
    they are stored in: res_bytes[layer name] = 1.5, 2 or 4 bytes per value of that layer's saved
    residual, 4 = the reference's int32 when not given; `pooled` = names of the layers whose saved residual
    is stored as its maximum over 2x2 windows of pixels, a quarter of the tensor, because only pooling
    consumers read it)."""
    res_bytes = res_bytes or {}
    from tcbnn_amd import nets
    bops, flops = nets.binary_ops([L])
    B = L["batch"]
    if L["kind"] == "in":
        byts = B * L["features"] * 4 + B * L["features"] / 8
    elif L["kind"] == "pool":  # bits in + out, residual in + out
        oh = (L["h"] + 2 * L["pad"] - L["window"]) // L["stride"] + 1
        rb = res_bytes.get(L.get("res_src"), 4) if L.get("res_src") else 0
        byts = B * L["channels"] * (L["h"] * L["w"] + oh * oh) * (1 / 8 + rb)
    elif L["kind"] == "avgfc":
        byts = B * L["h"] * L["w"] * L["channels"] * res_bytes.get(L.get("res_src"), 4) + \
            L["channels"] * L["out"] * 4 + B * L["out"] * 4
    elif L["kind"] in ("fc", "out"):
        byts = B * L["inp"] / 8 + L["inp"] * L["out"] / 8 + (B * L["out"] * 4 if L["kind"] == "out" else B * L["out"] / 8)
    else:
        oh = -(-L["h"] // L["stride"]); ow = -(-L["w"] // L["stride"])
        poh, pow_ = -(-oh // L["pool"]), -(-ow // L["pool"])
        out_bits = B * poh * pow_ * L["cout"] / 8
        if L["kind"] == "inconv":
            byts = B * 3 * L["h"] * L["w"] * 4 + out_bits + L["r"] * L["s"] * 3 * L["cout"] * 4
            if L["save_residual"]:
                byts += B * oh * ow * L["cout"] * res_bytes.get(L["name"], 4)
        else:
            byts = B * L["h"] * L["w"] * L["cin"] / 8 + out_bits + L["r"] * L["s"] * L["cin"] * L["cout"] / 8
            if L["save_residual"]:
                byts += B * oh * ow * L["cout"] * res_bytes.get(L["name"], 4) / (4 if L["name"] in pooled else 1)
            if L["inject_residual"]:
                # channels actually injected: those the source layer saved, capped by residual_channels
                src_ch = [S.get("cout", S.get("channels")) for S in spec if S["name"] == L.get("res_src")]
                ch = min([L["residual_channels"], L["cout"]] + src_ch)
                src_pixels = 4 if L["residual_pool"] and L.get("res_src") not in pooled else 1
                byts += B * oh * ow * src_pixels * ch * res_bytes.get(L.get("res_src"), 4)
    return dict(bops=bops, flops=flops, bytes=float(byts))


def roofline_of(name, g, variant):
    """Roofline record of one kernel (all its launches in a step): the binding roof is HBM when the
    kernel's arithmetic intensity is below the ridge of the compute peak, else the compute peak."""
    bound_c, peak_c = COMPUTE_PEAKS_TOPS[variant]
    secs = g["ms"] * 1e-3
    tops = g["bops"] / secs / 1e12
    gbs = g["bytes"] / secs / 1e9
    ridge = peak_c * 1e12 / (HBM_PEAK_GBS * 1e9)  # binary ops per byte
    intensity = g["bops"] / g["bytes"] if g["bytes"] else float("inf")
    hbm_bound = g["bops"] == 0 or intensity < ridge
    rec = {
        "bound": "hbm" if hbm_bound else bound_c,
        "achieved": round(gbs if hbm_bound else tops, 2),
        "peak": HBM_PEAK_GBS if hbm_bound else round(peak_c, 1),
        "unit": "GB/s" if hbm_bound else ("TFLOP/s" if variant == "mfma_f4" else "TOP/s"),
        "frac": round((gbs / HBM_PEAK_GBS) if hbm_bound else (tops / peak_c), 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get(name),
        "traffic_stale": TRAFFIC_STALE or name not in MEASURED_TRAFFIC_BYTES, "traffic_source": TRAFFIC_NOTE,
        "kernel": name, "launches_per_step": g["launches"],
        "avg_launch_ms": round(g["ms"] / g["launches"], 4),
        "algorithmic_bytes_per_launch": round(g["bytes"] / g["launches"]),
        "algorithmic_ops_per_launch": round(g["bops"] / g["launches"]),
        "ops_per_byte": round(intensity, 1) if g["bytes"] else None,
        "binary_tops": round(tops, 2), "hbm_gbs": round(gbs, 1),
    }
    if g.get("flops"):
        # The fp32 first layer is far from the HBM roof because its additions bind it: one dependent fp32 add per
        # (tap, output channel, pixel, image) is the least the reference's summation order allows (its 2 flops per
        # input value and tap are 6 per such add).  Peak: the published 157.3 TFLOP/s counts packed FMAs; plain adds
        # issue at a quarter of that (64 lanes per CU and clock).
        adds = g["flops"] / 6.0
        rec["valu_fp32"] = {"adds_per_launch": round(adds / g["launches"]), "achieved": round(adds / secs / 1e12, 2),
                            "peak": round(157.3 / 4, 1), "unit": "Tadd/s", "frac": round(adds / secs / 1e12 / (157.3 / 4), 4)}
        # `bound` stays the roof the kernel's algorithmic bytes and operations put it under; what the hardware
        # counters show it waiting for is the issue rate of its dependent fp32 additions
        rec["binding"] = "valu (dependent fp32 adds in the reference's summation order); see valu_fp32"
    return rec


def sweep(args, np, _lib):
    """Stand-alone kernels of the reference's benchmarks: BMMAS_new (tensorcore_kernel.cu:336-356) as
    tcbnn_bmm, BTC_Conv2d_balance (bmma_kernel.cu:101-165) as tcbnn_bconv; operands resident, packed
    once outside the timed launches; int32 outputs.  Binary operations: 2 per +-1 multiply-accumulate,
    border taps included; bytes: packed operands + int32 output, each moved once."""
    import ctypes as C
    from tcbnn_amd.device import DeviceBuffer, Event, Stream
    lib = _lib.lib
    stream = Stream()
    rng = np.random.default_rng(0)
    reps = max(args.steps, 10)

    def timed(launch):
        for _ in range(args.warmup):
            launch()
        stream.synchronize()
        ts = []
        e0, e1 = Event(), Event()
        for _ in range(3):  # `reps` back-to-back launches between two events (includes the gap between two launches)
            e0.record(stream)
            for _r in range(reps):
                launch()
            e1.record(stream)
            stream.synchronize()
            ts.append(e0.elapsed_ms(e1) / reps)
        return float(np.median(ts))

    rows = []
    for name, v in (("popc", _lib.VARIANTS["popc"]), ("mfma_i8", _lib.VARIANTS["mfma_i8"]), ("mfma_f4", _lib.VARIANTS["mfma_f4"])):
        for m, n, k in ((1024, 1024, 1024), (8192, 1024, 1024), (8192, 8192, 8192)):
            a = DeviceBuffer.from_numpy(rng.integers(0, 2 ** 32, size=(k // 32, m), dtype=np.uint64).astype(np.uint32))
            b = DeviceBuffer.from_numpy(rng.integers(0, 2 ** 32, size=(n, k // 32), dtype=np.uint64).astype(np.uint32))
            c = DeviceBuffer(4 * m * n)
            ms = timed(lambda: _lib.check(lib.tcbnn_bmm(a.ptr, b.ptr, c.ptr, m, n, k, v, stream.handle)))
            ops, byts = 2.0 * m * n * k, (m + n) * k / 8 + 4.0 * m * n
            rows.append(dict(case="bmm %dx%dx%d" % (m, n, k), engine=name, ms=round(ms, 4),
                             binary_tops=round(ops / ms / 1e9, 1), hbm_gbs=round(byts / ms / 1e6, 1)))
            for buf in (a, b, c):
                buf.free()
        for h, ch in ((32, 128), (16, 256), (8, 512), (56, 64), (28, 128), (14, 256), (7, 512)):
            B = 256
            inp = DeviceBuffer.from_numpy(rng.integers(0, 2 ** 32, size=h * h * (ch // 32) * B, dtype=np.uint64).astype(np.uint32))
            f = DeviceBuffer.from_numpy((rng.integers(0, 2, size=(3, 3, ch, ch)) * 2 - 1).astype(np.float32))
            filt = DeviceBuffer(4 * lib.tcbnn_conv_filter_words(3, 3, ch, ch))
            _lib.check(lib.tcbnn_pack_conv_filter(f.ptr, filt.ptr, 3, 3, ch, ch, stream.handle))
            out = DeviceBuffer(4 * B * h * h * ch)
            ms = timed(lambda: _lib.check(lib.tcbnn_bconv(inp.ptr, filt.ptr, out.ptr, B, h, h, ch, ch, 3, 3, 1, 1, 1, 1,
                                                          h, h, v, stream.handle)))
            ops = 2.0 * B * h * h * ch * ch * 9
            byts = B * h * h * ch / 8 + 9 * ch * ch / 8 + 4.0 * B * h * h * ch
            rows.append(dict(case="bconv 3x3 %dx%d C=%d b256" % (h, h, ch), engine=name, ms=round(ms, 4),
                             binary_tops=round(ops / ms / 1e9, 1), hbm_gbs=round(byts / ms / 1e6, 1)))
            for buf in (inp, f, filt, out):
                buf.free()
    sys.stderr.write("%-28s %-8s %9s %12s %9s\n" % ("case", "engine", "ms", "binary TOP/s", "GB/s"))
    for r in rows:
        sys.stderr.write("%-28s %-8s %9.4f %12.1f %9.1f\n" % (r["case"], r["engine"], r["ms"], r["binary_tops"], r["hbm_gbs"]))
    print(json.dumps({"metric": "binary TOP/s of the stand-alone bit-GEMM / 3x3 bit-convolution kernels (int32 outputs)",
                      "unit": "TOP/s", "n_gpus": 1, "data": "synthetic", "rows": rows}))
    return 0


def cpu_model():
    """Model name of the host processor (first entry of /proc/cpuinfo), for the CPU baseline record."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--net", default="imagenet_resnet", choices=["imagenet_resnet", "cifar10_vgg", "mnist_mlp", "alexnet", "cifar10_resnet", "imagenet_vgg",
                                                                 "imagenet_resnet_textbook"])
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--variant", default="auto")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-batch", type=int, default=None)
    ap.add_argument("--layers", action="store_true", help="also print a per-layer table to stderr")
    ap.add_argument("--graph", action="store_true",
                    help="time the steps as replays of one captured HIP graph instead of eager launches")
    ap.add_argument("--preheat-ms", type=float, default=100.0,
                    help="untimed forward passes for this long before the --warmup steps: a freshly started process "
                         "finds the GPU in a low clock state, and the step time keeps falling for the first 30-40 "
                         "passes (about 20 ms); 0 = none")
    ap.add_argument("--in-flight", type=int, default=2,
                    help="after the timed steps, also time the same number of steps with this many independent "
                         "batches in flight (one network copy and one stream each); reported as a separate "
                         "object, never as `value`; 1 = skip")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of a network: the stand-alone bit-GEMM and 3x3 bit-convolution shapes "
                         "(int32 outputs), every engine; one JSON line with a row per case")
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

    if args.sweep:
        return sweep(args, np, _lib)

    default_batch = {"mnist_mlp": 8192}.get(args.net, 256)
    batch = args.batch or default_batch
    spec = nets.SPECS[args.net](batch=batch)
    weights = tcbnn_amd.synthetic_weights(spec, seed=0)
    x = tcbnn_amd.synthetic_input(spec, seed=0)
    net = tcbnn_amd.Network(spec, weights, x)
    stream = Stream()
    bops, flops = nets.binary_ops(spec)

    # ------------------------------------------------------------------ timed region
    # Untimed: bring the GPU to its steady clock state first (measured on this device, fresh process, batch 256: the
    # first pass after start-up takes 0.546 ms, the 40th and every later one 0.473 ms), then the W warm-up steps.
    # The same K steps are first timed exactly as launched (W warm-up steps, nothing else before them) and reported
    # as `as_launched`, so that both figures are on the line.
    as_launched = None
    if args.preheat_ms > 0 and not args.graph:
        for _ in range(args.warmup):
            net.forward(stream)
        stream.synchronize()
        _lib.device_synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            net.forward(stream)
        stream.synchronize()
        _lib.device_synchronize()
        wall0 = time.perf_counter() - t0
        as_launched = {"value": round(batch * args.steps / wall0, 1), "unit": "images/s",
                       "ms_per_step": round(wall0 / args.steps * 1e3, 4),
                       "what": "the same K steps after the W warm-up steps only, in a process that has just started "
                               "(GPU clocks still rising)"}
    preheat_steps = 0
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < args.preheat_ms:
        for _ in range(8):
            net.forward(stream)
        stream.synchronize()
        preheat_steps += 8
    for _ in range(args.warmup):
        net.forward(stream)
    stream.synchronize()
    _lib.device_synchronize()
    step = lambda: net.forward(stream)
    if args.graph:  # the forward allocates nothing and uses no memset: it can be captured whole
        from tcbnn_amd.device import Graph
        graph = Graph(stream, net.forward)
        step = graph.launch
        step()
        stream.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    stream.synchronize()
    _lib.device_synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    images_per_s = batch * args.steps / wall

    # ------------------------------------------------------------------ several batches in flight (a serving
    # pipeline: batch n + 1 starts while batch n is still in its later layers, so the ragged end of one launch and
    # the gap before the next are filled with the other batch's workgroups).  Same K steps = K forward passes of one
    # batch each, dealt round-robin to N network copies (own activations, residuals and input; same weights) on N
    # streams of the same priority.  Latency of one batch grows; reported beside `value`, never as `value`.
    in_flight = None
    if args.in_flight > 1 and not args.graph:
        others = [tcbnn_amd.Network(spec, weights, tcbnn_amd.synthetic_input(spec, seed=i + 1))
                  for i in range(args.in_flight - 1)]
        copies = [net] + others
        streams = [stream] + [Stream() for _ in others]
        for k in range(max(args.warmup, args.in_flight)):
            copies[k % len(copies)].forward(streams[k % len(copies)])
        _lib.device_synchronize()
        steps_n = max(args.steps, 100)  # (filling and draining the pipeline is one batch latency: keep it small)
        t0 = time.perf_counter()
        for k in range(steps_n):
            copies[k % len(copies)].forward(streams[k % len(copies)])
        for st in streams:
            st.synchronize()
        _lib.device_synchronize()
        wall_n = time.perf_counter() - t0
        in_flight = {"batches_in_flight": args.in_flight, "steps": steps_n,
                     "value": round(batch * steps_n / wall_n, 1), "unit": "images/s",
                     "ms_per_step": round(wall_n / steps_n * 1e3, 4),
                     "note": "K forward passes of one batch each, round-robin over %d network copies on %d streams; "
                             "throughput of a pipeline, not the latency of a batch" % (len(copies), len(streams))}
        for o in others:
            o.release()

    # ------------------------------------------------------------------ per-launch timing (HIP events
    # on the launch stream), outside the timed region.  A layer's duration = R back-to-back launches of it between
    # two events, divided by R: it includes the gap between two launches of a stream, as the layer's share of a step
    # does, but not the two event records, which cost about 5 us per launch when every launch of a pass is bracketed
    # (the sum of such per-layer figures was 0.09 ms above the step they were taken from).  Layers are idempotent:
    # every output word is rewritten by each launch.  One pass over the layers first, so that each layer finds its
    # inputs as the forward leaves them.
    R = 10
    per_layer = {L["name"]: [] for L in spec}
    e0, e1 = Event(), Event()
    net.forward(stream)
    for _ in range(3):
        for L, layer in zip(spec, net.order):
            e0.record(stream)
            for _r in range(R):
                layer.forward(stream)
            e1.record(stream)
            stream.synchronize()
            per_layer[L["name"]].append(e0.elapsed_ms(e1) / R)
    layer_ms = {k: float(np.median(v)) for k, v in per_layer.items()}

    # ------------------------------------------------------------------ packed first-layer input (a request,
    # never the default): the upload also makes a zero-padded, batch-innermost copy of the input on the device and
    # the first layer reads that with a kernel that needs no staging.  The same K steps on a second network built
    # that way, what the extra pass of the upload costs, and the rate with that pass charged to every step, are
    # reported beside `value`; `value` itself is the default path, which reads the uploaded array as it is.
    packed_input = None
    if spec[0]["kind"] == "inconv" and spec[0]["pool"] == 1 and not args.graph:
        pnet = tcbnn_amd.Network(spec, weights, x, input_layout=_lib.INCONV_INPUT_PACKED)
        first = pnet.order[0]
        t0 = time.perf_counter()  # (building the network left the GPU idle: settle the clocks again, as for `value`)
        while (time.perf_counter() - t0) * 1e3 < args.preheat_ms:
            for _ in range(8):
                pnet.forward(stream)
            stream.synchronize()
        for _ in range(max(args.warmup, 3)):
            pnet.forward(stream)
        stream.synchronize()
        _lib.device_synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            pnet.forward(stream)
        stream.synchronize()
        _lib.device_synchronize()
        wall_p = time.perf_counter() - t0
        pack = lambda: _lib.check(_lib.lib.tcbnn_inconv_pack_input(
            first.input_gpu.ptr, first.input_packed_gpu.ptr, first.batch, first.input_height, first.input_width,
            first.filter_height, first.filter_width, first.stride_height, first.stride_width, int(first.padding),
            stream.handle))
        ts, fs = [], []
        for _ in range(3):
            for fn, acc in ((pack, ts), (lambda: first.forward(stream), fs)):
                e0.record(stream)
                for _r in range(R):
                    fn()
                e1.record(stream)
                stream.synchronize()
                acc.append(e0.elapsed_ms(e1) / R)
        pack_ms, first_ms = float(np.median(ts)), float(np.median(fs))
        packed_input = {"first_layer_input": "float [Hp][Wp][batch][3], zero-padded; made from the uploaded "
                                             "[batch][3][H][W] array by inconv_pack_input_kernel at set_input",
                        "kernel": first.kernel_name(), "first_layer_ms": round(first_ms, 4),
                        "value": round(batch * args.steps / wall_p, 1), "unit": "images/s",
                        "ms_per_step": round(wall_p / args.steps * 1e3, 4),
                        "pack_ms": round(pack_ms, 4),
                        "pack_gbs": round((first.input_size() * 4 + first.input_packed_gpu.nbytes) / pack_ms / 1e6, 1),
                        "value_with_pack_in_every_step": round(batch / (wall_p / args.steps * 1e3 + pack_ms) * 1e3, 1)}
        pnet.release()

    # width each saved residual is stored in (16 bits where its bound proves that exact)
    width = {_lib.RES_I32: 4, _lib.RES_I16: 2, _lib.RES_I12: 1.5}
    res_bytes = {L["name"]: width[net.layers[L["name"]].output_residual_gpu.format]
                 for L in spec if L.get("save_residual") or (L["kind"] == "pool" and L.get("res_src"))}
    # saved residuals stored as their 2x2 maximum (every reader pools): what the buffers hold after the forward
    pooled = {name for name in res_bytes if net.layers[name].output_residual_gpu.pooled}
    # group launches by device kernel, as a profiler does
    groups = {}
    for L, layer in zip(spec, net.order):
        name = layer.kernel_name() if hasattr(layer, "kernel_name") else \
            {"in": "in128_kernel"}[L["kind"]]
        w = layer_work(L, spec, res_bytes, pooled)
        g = groups.setdefault(name, dict(bops=0.0, flops=0.0, bytes=0.0, ms=0.0, launches=0))
        g["bops"] += w["bops"]
        g["flops"] += w["flops"]
        g["bytes"] += w["bytes"]
        g["ms"] += layer_ms[L["name"]]
        g["launches"] += 1
    by_time = sorted(groups.items(), key=lambda kv: -kv[1]["ms"])
    global MEASURED_TRAFFIC_BYTES, TRAFFIC_STALE, TRAFFIC_NOTE
    if args.net == "imagenet_resnet" and batch == 256 and variant == "mfma_f4":  # the workload the file covers
        MEASURED_TRAFFIC_BYTES, TRAFFIC_STALE, TRAFFIC_NOTE = load_measured_traffic()
    else:
        MEASURED_TRAFFIC_BYTES, TRAFFIC_STALE, TRAFFIC_NOTE = {}, True, "no counter run covers this workload"
    roofline = roofline_of(by_time[0][0], by_time[0][1], variant)
    roofline_all = [roofline_of(n, g, variant) for n, g in by_time]
    bit = [g for n, g in groups.items() if g["bops"] > 0]
    bit_ops, bit_ms = sum(g["bops"] for g in bit), sum(g["ms"] for g in bit)
    bit_layers_tops = round(bit_ops / (bit_ms * 1e-3) / 1e12, 2)
    # every bit-matmul / bit-convolution launch of the step together against the engine's compute peak
    peak_name, peak_tops = COMPUTE_PEAKS_TOPS[variant]
    roofline_bit_layers = {
        "bound": peak_name, "achieved": bit_layers_tops, "peak": round(peak_tops, 1),
        "unit": "TFLOP/s" if variant == "mfma_f4" else "TOP/s", "frac": round(bit_layers_tops / peak_tops, 4),
        "binary_ops_per_step": bit_ops, "ms_per_step": round(bit_ms, 4), "launches_per_step": sum(g["launches"] for g in bit),
        "hbm_gbs": round(sum(g["bytes"] for g in bit) / (bit_ms * 1e-3) / 1e9, 1),
        "what": "all bit layers of the step (binary ops: 2 per +-1 multiply-accumulate, border taps included) over the "
                "sum of their launch durations (10 launches back to back between two events, the gap between launches "
                "included)"}

    # ------------------------------------------------------------------ shader clock while the step runs: the
    # published peaks are quoted at the nominal clock; one wavefront on a second stream counts shader cycles against
    # the device's constant-rate wall clock while forward passes run (outside the timed region)
    shader_clock = None
    try:
        from tcbnn_amd.device import DeviceBuffer
        counts = DeviceBuffer(16)
        side = Stream()
        khz = C.c_int(0)
        for _ in range(20):
            net.forward(stream)
        probe_us = int(max(2.0, min(50.0, 10 * ms_per_step)) * 1000)
        _lib.check(_lib.lib.tcbnn_shader_clock_probe(counts.ptr, probe_us, C.byref(khz), side.handle))
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e6 < probe_us * 1.5:
            for _ in range(4):
                net.forward(stream)
            stream.synchronize()
        side.synchronize()
        cyc, ticks = (int(v) for v in counts.to_numpy(np.uint64, (2,)))
        shader_clock = {"mhz": round(cyc / ticks * khz.value / 1000.0, 1), "nominal_mhz": 2400,
                        "what": "shader cycles counted by one wavefront over %d us of the device's %d kHz wall clock "
                                "while forward passes of this network run; the peaks above are quoted at the nominal "
                                "clock" % (probe_us, khz.value)}
        counts.free()
    except Exception as e:  # (a measurement aid: the line is valid without it)
        shader_clock = {"mhz": None, "error": str(e)}

    if args.layers:
        sys.stderr.write("%-8s %-34s %10s %10s %9s\n" % ("layer", "kernel", "ms", "TOP/s", "GB/s"))
        for L, layer in zip(spec, net.order):
            ops = nets.binary_ops([L])[0]
            kn = layer.kernel_name() if hasattr(layer, "kernel_name") else L["kind"]
            byts = layer_work(L, spec, res_bytes, pooled)["bytes"]
            ms = layer_ms[L["name"]]
            sys.stderr.write("%-8s %-34s %10.4f %10.1f %9.0f\n" % (L["name"], kn, ms, ops / (ms * 1e-3) / 1e12,
                                                                   byts / (ms * 1e-3) / 1e9))
        sys.stderr.write("sum of layers: %.4f ms; step: %.4f ms\n" % (sum(layer_ms.values()), ms_per_step))

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    cpu = None
    if not args.no_cpu:
        from oracle import nets as orc_nets, orc
        cb = args.cpu_batch or {"imagenet_resnet": 64, "cifar10_vgg": 64, "mnist_mlp": 8192, "alexnet": 32,
                                   "cifar10_resnet": 16, "imagenet_vgg": 8, "imagenet_resnet_textbook": 16}[args.net]
        cb = min(cb, batch)
        cspec = nets.SPECS[args.net](batch=cb)
        xs = x[:cb]
        orc_nets.run(cspec, weights, xs)  # warm-up (page-in, thread pool)
        t0 = time.perf_counter()
        reps = 0
        while True:
            cpu_out = orc_nets.run(cspec, weights, xs)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 1000:  # about 10 s of CPU work
                break
        cpu_s = (time.perf_counter() - t0) / reps
        # the GPU result of the same images must agree with what the CPU leg just computed
        got = net.logits()[:cb]
        np.testing.assert_allclose(got, cpu_out[spec[-1]["name"]]["out"], rtol=1e-5, atol=0)
        cpu = {"value": round(cb / cpu_s, 2), "unit": "images/s", "cores": orc.num_threads(), "kind": "port",
               "sample": "%s forward, batch %d, mean of %d reps (%.1f s) after 1 warm-up, OpenMP XOR/popcount "
                         "(64-bit words), same seeds" % (args.net, cb, reps, cpu_s * reps),
               "binary_tops": round(nets.binary_ops(cspec)[0] / cpu_s / 1e12, 4), "cpu_model": cpu_model()}

    out = {
        "metric": "images/sec ResNet-18 BNN 224x224 batch 256 on 1 MI355X" if args.net == "imagenet_resnet"
        else "images/sec %s batch %d on 1 MI355X" % (args.net, batch),
        "value": round(images_per_s, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "preheat": {"ms": args.preheat_ms, "steps": preheat_steps,
                                           "what": "untimed forward passes before the warm-up steps, until the GPU's "
                                                   "clocks have settled"},
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": round(images_per_s / PAPER_IMAGES_PER_S, 2) if args.net == "imagenet_resnet" and batch == 256
        else None,
        "dtype": "u32 xor+popcount -> int32" if variant == "popc" else
        ("int8 mfma -> int32" if variant == "mfma_i8" else "fp4 mfma -> fp32 (exact integers)"),
        "data": "synthetic",
        "config": {"workload": "%s, reference topology (%s), batch %d, seeded synthetic weights and input"
                               % (args.net, {"imagenet_resnet": "imagenet_resnet.cu:223-325",
                                             "cifar10_vgg": "cifar10_vgg.cu:162-199",
                                             "mnist_mlp": "mnist_mlp.cu:111-124",
                                             "alexnet": "alexnet.cu:143-177",
                                             "cifar10_resnet": "cifar10_resnet.cu:189-259",
                                             "imagenet_vgg": "imagenet_vgg.cu:217-286",
                                             "imagenet_resnet_textbook": "no reference driver"}[args.net], batch),
                   "variant": variant, "layers": len(spec), "launch": "hip graph replay" if args.graph else "eager",
                   "residual_storage": ("the narrowest width the bound of |residual| proves exact: 12 bits for %d, "
                                        "16 bits for %d, int32 for %d of %d tensors"
                                        % (sum(1 for v in res_bytes.values() if v == 1.5),
                                           sum(1 for v in res_bytes.values() if v == 2),
                                           sum(1 for v in res_bytes.values() if v == 4), len(res_bytes)))
                   + ("; %d of them stored as their maximum over 2x2 windows of pixels (every reader takes that "
                      "maximum, kernel.cuh:775-782)" % len(pooled) if pooled else "")
                   if res_bytes else "none"},
        "binary_tops": round(bops * args.steps / wall / 1e12, 2),
        "binary_ops_per_step": bops, "fp32_first_layer_flops_per_step": flops,
        "roofline": roofline,
        "cpu_baseline": cpu,
        "as_launched": as_launched,
        "packed_input": packed_input,
        "batches_in_flight": in_flight,
        "bit_layers_binary_tops": bit_layers_tops,
        "roofline_bit_layers": roofline_bit_layers,
        "shader_clock": shader_clock,
        "roofline_all_kernels": roofline_all,
    }
    net.release()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
