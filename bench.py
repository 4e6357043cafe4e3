#!/usr/bin/env python3
"""Benchmark of the GPU layer stack on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload stylenet|resnet50|resnet50ref|stylenet3x3ref|stylenet9x9ref|conv1|mobilenet|stylenet9x9|copy|bw-<layer>]

A step is one forward pass of the named network over one synthetic input frame that is already
resident in HBM (uploaded before the timed region); weights are synthetic (random init).  Prints ONE
JSON line on stdout; progress goes to stderr.  The default workload is BASELINE.json configs[1], the
Johnson style-transfer net at 512x624 in fp32 storage; ResNet-50 imgs/s is measured in the same run and
reported under "also".
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

import fyusenet_amd as fa  # noqa: E402
from fyusenet_amd import networks  # noqa: E402

PEAK_MFMA_F16_TFLOPS = 2500.0   # MI355X dense fp16/bf16 matrix peak
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E
# (layer type, kernel, cin, cout, h, w) -> measured HBM bytes per launch (fetch + write), fp32 storage
MEASURED_TRAFFIC = {(6, 3, 128, 128, 156, 128): 27.13e6 + 10.22e6}  # launches with the fused residual read


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_net(workload):
    if workload == "stylenet":
        return networks.StyleNet(fa.STORAGE_F32, 512, 624, 3), "stylenet 512x624 ms/frame", "ms/frame", "fp32 storage, fp16x2-split MFMA, fp32 accumulate"
    if workload == "stylenet9x9":
        return networks.StyleNet(fa.STORAGE_F16, 1524, 1856, 9), "stylenet9x9 1524x1856 ms/frame", "ms/frame", "fp16 storage, fp16 MFMA, fp32 accumulate"
    if workload == "resnet50":
        return networks.ResNet50(fa.STORAGE_F32), "ResNet-50 224x224 imgs/s", "imgs/s", "fp32 storage"
    if workload == "resnet50ref":   # the reference's own sample graph (explicit batch-norm layers), .dat-compatible
        from fyusenet_amd import samples
        return samples.ResNet50Sample(fa.STORAGE_F32), "ResNet-50 (reference sample graph) 224x224 imgs/s", "imgs/s", "fp32 storage"
    if workload in ("stylenet3x3ref", "stylenet9x9ref"):   # the reference's own sample graphs (shallow, fractional-step convolutions)
        from fyusenet_amd import samples
        k = 3 if workload == "stylenet3x3ref" else 9
        return samples.StyleNetSample(k, 512, 624, fa.STORAGE_F32), "stylenet%dx%d (reference sample graph) 512x624 ms/frame" % (k, k), "ms/frame", "fp32 storage"
    if workload == "mobilenet":
        return networks.MobileNetV2(fa.STORAGE_F16), "MobileNetV2 224x224 imgs/s", "imgs/s", "fp16 storage"
    if workload == "conv1":
        return networks.SingleConvNet(fa.STORAGE_F32), "conv3x3 64->64 256x256 us/layer", "us", "fp32 storage"
    if workload == "resconv":  # the style net's dominant layer on its own (for counter runs)
        return networks.SingleConvNet(fa.STORAGE_F32, channels=128, width=128, height=156), "conv3x3 128->128 128x156 us/layer", "us", "fp32 storage"
    if workload == "copy":
        return CopyNet(fa.STORAGE_F32), "copy 64x1024x1024 fp32 GB/s", "GB/s", "fp32"
    if workload.startswith("bw-"):   # one bandwidth-bound layer at a size far beyond the caches
        kind = workload[3:]
        if kind not in BandwidthNet.KINDS:
            raise SystemExit("unknown workload %s (bw-%s)" % (workload, "|bw-".join(BandwidthNet.KINDS)))
        return BandwidthNet(kind), "%s 128x1024x1024 fp16 GB/s" % kind, "GB/s", "fp16 storage"
    raise SystemExit("unknown workload %s" % workload)


class BandwidthNet(fa.NeuralNetwork):
    """One layer of a bandwidth-bound class on a 128 x 1024 x 1024 fp16 tensor (268 MB), inputs fed from the host."""
    KINDS = ("dwconv", "maxpool", "avgpool", "batchnorm", "add", "concat", "scale", "sigmoid")
    C, S = 128, 1024
    output_layer = 1

    def __init__(self, kind):
        super().__init__(fa.STORAGE_F16)
        self.kind = kind
        self.input_key = (1, 0)

    def buildLayers(self, f):
        C, S, k = self.C, self.S, self.kind
        if k == "dwconv":
            b = fa.ConvLayerBuilder(3, k).type(fa.LayerType.CONVOLUTION2D).shape(C, S, S, C).groupSize(C).inputPadding(1).prefixAct(fa.ActType.RELU)
        elif k in ("maxpool", "avgpool"):
            op = fa.PoolLayerBuilder.POOL_MAX if k == "maxpool" else fa.PoolLayerBuilder.POOL_AVG
            b = fa.PoolLayerBuilder(op, k).shape(C, S, S, C).poolSize(2).downsample(2)
        elif k == "batchnorm":
            b = fa.GPULayerBuilder(k).type(fa.LayerType.BATCHNORM).shape(C, S, S, C).prefixAct(fa.ActType.RELU)
        elif k == "add":
            b = fa.GPULayerBuilder(k).type(fa.LayerType.ADD).shape(C, S, S, C)
        elif k == "concat":
            b = fa.ConcatLayerBuilder(k).input(C // 2, 0).input(C // 2, 0)
            b.size(S, S)
            b.outputChannels_ = C
        elif k == "scale":
            b = fa.ScaleLayerBuilder(k).shape(C, S // 2, S // 2, C).scale(2.0)
        else:
            b = fa.GPULayerBuilder(k).type(fa.LayerType.SIGMOID).shape(C, S, S, C)
        if k != "add":
            b.deep()
        b.number(1).push(f)

    def connectLayers(self, layers, bm):
        pass

    def initializeWeights(self, layers):
        C = self.C
        if self.kind == "dwconv":
            layers[1].loadWeightsAndBiases(np.concatenate([np.zeros(C, np.float32), np.full(9 * C, 1.0 / 9.0, np.float32)]), 0)
        elif self.kind == "batchnorm":
            layers[1].loadScaleAndBias(np.concatenate([np.full(C, 0.5, np.float32), np.zeros(C, np.float32)]), 0)

    def ports(self):
        C, S = self.C, self.S
        if self.kind == "add":
            return [(C, S, S)] * 2
        if self.kind == "concat":
            return [(C // 2, S, S)] * 2
        if self.kind == "scale":
            return [(C, S // 2, S // 2)]
        return [(C, S, S)]

    def makeInput(self):
        return np.ones(self.ports()[0], np.float32)

    def setInput(self, x):
        for port, shape in enumerate(self.ports()):
            self.layers[1].setInput(x if port == 0 else np.ones(shape, np.float32), port)

    def algorithmic_bytes(self):
        """Bytes one launch has to move: every input element once, every output element once (fp16)."""
        n_in = sum(c * h * w for c, h, w in self.ports())
        oc, oh, ow = self.layers[1].outputShape()[:3]
        return 2 * (n_in + oc * oh * ow)


class CopyNet(fa.NeuralNetwork):
    """A concat layer with a single input: a plain copy kernel of known size (268 MB read, 268 MB written),
    used to scale the FETCH_SIZE / WRITE_SIZE counters of rocprofv3."""
    C, S = 64, 1024
    output_layer = 1
    input_key = (1, 0)

    def buildLayers(self, f):
        b = fa.ConcatLayerBuilder("copy").number(1).deep().input(self.C, 0)
        b.size(self.S, self.S)
        b.outputChannels_ = self.C
        b.push(f)

    def connectLayers(self, layers, bm):
        pass

    def makeInput(self):
        return np.ones((self.C, self.S, self.S), np.float32)

    def setInput(self, x):
        self.layers[1].setInput(x, 0)


def conv_work(b):
    """Algorithmic FLOPs and bytes of one convolution-type layer: flops = 2*Hout*Wout*Cout*Cin*K^2
    (transposed: input pixels); bytes = s*(in + out [+ residual]) + s*(weights + 2*Cout), halo and
    channel padding excluded."""
    k = getattr(b, "kernel_", 1)
    t = int(b.type_)
    cin, cout, h, w = b.inputChannels_, b.outputChannels_, b.height_, b.width_
    if t == int(fa.LayerType.TRANSCONVOLUTION2D):
        ho, wo = 2 * h + k - 2 - b.transconvCrop_, 2 * w + k - 2 - b.transconvCrop_
        flops = 2.0 * h * w * cout * cin * k * k
    else:
        ho, wo = h // b.downsample_[1], w // b.downsample_[0]
        flops = 2.0 * ho * wo * cout * cin * k * k
    return flops, (cin * h * w, cout * ho * wo, cout * cin * k * k + 2 * cout)


def timed_forwards(net, steps, warmup, graph=True):
    net.useGraph(graph)
    for _ in range(warmup):
        net.forward()
    net.finish()
    t0 = time.perf_counter()
    for _ in range(steps):
        net.forward()
    net.finish()
    return (time.perf_counter() - t0) * 1e3 / steps


def dominant_conv_roofline(net, storage_bytes):
    """Times every layer's kernel(s) alone with HIP events on the network's stream and returns the
    roofline record of the layer class that takes the most time (identical-shape layers pooled)."""
    groups = {}
    for lyr in net.layers:
        t = int(lyr.builder.type_)
        if t in (int(fa.LayerType.UPLOAD), int(fa.LayerType.DOWNLOAD)):
            continue
        iters = 20
        lyr.timeKernel(3)
        ms = lyr.timeKernel(iters)            # launches back to back in one hipGraph (dispatch gaps included)
        b = lyr.builder
        key = (t, getattr(b, "kernel_", 0), b.inputChannels_, b.outputChannels_, b.height_, b.width_, tuple(b.downsample_),
               bool(int(b.getFlags()) & 1))
        g = groups.setdefault(key, {"ms": 0.0, "n": 0, "layer": lyr})
        g["ms"] += ms
        g["n"] += 1
    key, g = max(groups.items(), key=lambda kv: kv[1]["ms"])
    lyr, b = g["layer"], g["layer"].builder
    avg_ms = g["ms"] / g["n"]
    rec = {"kernel": lyr.kernelInfo(), "layer": lyr.name, "launches_per_step": g["n"], "avg_launch_us": avg_ms * 1e3}
    if int(b.type_) in (int(fa.LayerType.CONVOLUTION2D), int(fa.LayerType.TRANSCONVOLUTION2D)) and getattr(b, "groupSize_", 1) == 1:
        flops, (ein, eout, ew) = conv_work(b)
        res = eout if int(b.getFlags()) & 1 else 0
        nbytes = storage_bytes * (ein + eout + res + ew)
        # fp32 storage: every algorithmic FLOP is issued as three fp16 MFMA FLOPs (hi*hi, lo*hi, hi*lo),
        # which decides the bound; `achieved` stays the ALGORITHMIC rate against the fp16 matrix peak
        passes = 3 if storage_bytes == 4 else 1
        t_mfma = passes * flops / (PEAK_MFMA_F16_TFLOPS * 1e12)
        t_hbm = nbytes / (PEAK_HBM_GBS * 1e9)
        if t_mfma >= t_hbm:
            ach = flops / (avg_ms * 1e-3) / 1e12
            rec.update({"bound": "mfma", "achieved": ach, "peak": PEAK_MFMA_F16_TFLOPS, "unit": "TFLOP/s", "frac": ach / PEAK_MFMA_F16_TFLOPS,
                        "mfma_passes": passes, "mfma_issue_frac": passes * ach / PEAK_MFMA_F16_TFLOPS})
        else:
            ach = nbytes / (avg_ms * 1e-3) / 1e9
            rec.update({"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS})
        rec["algorithmic_flops_per_launch"] = flops
        rec["algorithmic_bytes_per_launch"] = nbytes
    # HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled by the copy-kernel factors
    # (profiles/conv_mfma_stylenet_512x624_fp32.md); only known for the profiled workload's dominant kernel
    rec["traffic"] = MEASURED_TRAFFIC.get((key[0], key[1], key[2], key[3], key[4], key[5]))
    per_layer = sorted(((v["ms"], v["n"], v["layer"].name) for v in groups.values()), reverse=True)
    return rec, per_layer


def host_io_rates(net, x, frames):
    """Frame rate with the frame handed over and returned in host memory (PCIe in both directions inside the timed
    region): the synchronous call sequence, then the frame pipeline at depth 2 and 3.  Reported beside `value`,
    never as `value`."""
    in_layer, in_port = net.input_key
    net.useGraph(False)
    rec = {}
    for _ in range(3):
        net.setInput(x); net.forward(); net.finish(); y = net.getOutput(net.output_layer)
    t0 = time.perf_counter()
    for _ in range(frames):
        net.setInput(x); net.forward(); net.finish(); net.getOutput(net.output_layer)
    rec["ms_per_frame_synchronous"] = (time.perf_counter() - t0) * 1e3 / frames
    for depth in (2, 3):
        outs = [np.empty_like(y) for _ in range(depth + 1)]
        net.asyncBegin(in_layer, net.output_layer, depth=depth, inPort=in_port)
        for i in range(depth + 2):
            t = net.asyncSubmit(x, outs[i % len(outs)])
        net.asyncWait(t)
        t0 = time.perf_counter()
        for i in range(frames):
            t = net.asyncSubmit(x, outs[i % len(outs)])
        net.asyncWait(t)
        rec["ms_per_frame_pipeline_depth%d" % depth] = (time.perf_counter() - t0) * 1e3 / frames
        net.asyncEnd()
        assert np.array_equal(outs[(frames - 1) % len(outs)], y)
    rec["bytes_in"], rec["bytes_out"] = int(x.nbytes), int(y.nbytes)
    return rec


def frame_pool_rate(workload, x, y_shape, frames, instances=4, graph=True):
    """Frames per second through a pool of `instances` networks of this workload, each with its own streams and frame
    pipeline; frames come from host memory and results return there (PCIe inside the timed region).  Reported beside
    `value`, never as `value`."""
    pool = fa.FramePool(lambda: make_net(workload)[0], instances=instances, depth=2, graph=graph)
    outs = [np.empty(y_shape, np.float32) for _ in range(3 * instances)]
    for i in range(2 * instances):
        t = pool.submit(x, outs[i % len(outs)])
    pool.wait(t)
    t0 = time.perf_counter()
    for i in range(frames):
        t = pool.submit(x, outs[i % len(outs)])
    pool.wait(t)
    dt = time.perf_counter() - t0
    pool.close()
    return {"instances": instances, "launch": "hipGraph replay" if graph else "eager launches", "frames_per_s": frames / dt,
            "ms_per_frame": dt * 1e3 / frames}


def frame_pool_rate_in_child(workload, frames, instances=4, graph=True):
    """frame_pool_rate in a process of its own (started as a child, never exec'ed into): the side measurement gets a
    fresh HIP runtime with the hardware queues to itself, and a failure in it cannot take the main record with it."""
    import subprocess
    cmd = [sys.executable, os.path.abspath(__file__), "--frame-pool-only", "--workload", workload, "--steps", str(frames),
           "--instances", str(instances)] + ([] if graph else ["--pool-eager"])
    try:
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
        if r.returncode != 0:
            return {"error": "child exited with %d: %s" % (r.returncode, r.stderr.strip()[-300:])}
        return json.loads(r.stdout.strip().splitlines()[-1])
    except Exception as e:   # noqa: BLE001 -- a side measurement must not fail the benchmark
        return {"error": repr(e)}


def cpu_baseline(net, x, total_flops):
    """Times the CPU oracle (plain C restatement of the reference's unit-test convolution, OpenMP over
    output channels) on the dominant convolution of the workload at full size and scales by the
    network's algorithmic FLOPs."""
    from oracle import oracle as O
    threads = min(os.cpu_count() or 1, 16)
    O.set_threads(threads)
    conv_layers = [l for l in net.layers if int(l.builder.type_) == int(fa.LayerType.CONVOLUTION2D) and getattr(l.builder, "groupSize_", 1) == 1]
    lyr = max(conv_layers, key=lambda l: conv_work(l.builder)[0])
    b = lyr.builder
    flops, _ = conv_work(b)
    from fyusenet_amd import prng
    xin = prng.uniform(77, (b.inputChannels_, b.height_, b.width_), -1, 1)
    ins = [xin]
    if int(b.getFlags()) & 1:
        ins.append(prng.uniform(78, (b.outputChannels_, b.height_ // b.downsample_[1], b.width_ // b.downsample_[0]), -1, 1))
    t0 = time.perf_counter()
    O.run_layer(b, lyr.weights, ins)
    dt = time.perf_counter() - t0
    return dt, flops, threads, lyr.name


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="stylenet")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-also", action="store_true")
    ap.add_argument("--no-pool", action="store_true", help="skip the side measurement of several instances side by side")
    ap.add_argument("--frame-pool-only", action="store_true", help="(internal) print the frame pool's record for --workload; --steps = frames")
    ap.add_argument("--instances", type=int, default=4)
    ap.add_argument("--pool-eager", action="store_true", help="(internal) the pool's instances launch eagerly instead of replaying graphs")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this engine is single-GPU (batch 1 inference); run with --gpus 1")

    if args.frame_pool_only:
        probe = make_net(args.workload)[0]
        probe.setup()
        x = probe.makeInput()
        probe.setInput(x)
        probe.forward()
        probe.finish()
        y_shape = probe.getOutput(probe.output_layer).shape
        probe.cleanup()
        print(json.dumps(frame_pool_rate(args.workload, x, y_shape, args.steps, args.instances, not args.pool_eager)), flush=True)
        return

    log(fa.capi.device_info(0))
    net, metric, unit, dtype = make_net(args.workload)
    net.setup()
    x = net.makeInput()
    net.setInput(x)
    # both launch modes of the engine are timed over exactly K steps; the faster one is reported as `value`
    ms_graph = timed_forwards(net, args.steps, args.warmup, graph=True)
    ms_eager = timed_forwards(net, args.steps, args.warmup, graph=False)
    log("%s: %.4f ms/step (hipGraph), %.4f ms/step (eager launches)" % (args.workload, ms_graph, ms_eager))
    ms = min(ms_graph, ms_eager)
    launch = "hipGraph replay" if ms_graph <= ms_eager else "eager launches on one stream"
    net.useGraph(False)
    storage_bytes = 4 if net.storage == fa.STORAGE_F32 else 2
    roof, per_layer = dominant_conv_roofline(net, storage_bytes)
    for t, n, name in per_layer[:8]:
        log("   %-12s x%-2d %.1f us total" % (name, n, t * 1e3))
    total_flops = sum(conv_work(l.builder)[0] for l in net.layers if int(l.builder.type_) in (6, 8) and getattr(l.builder, "groupSize_", 1) == 1)

    if unit == "ms/frame":
        value, hib = ms, False
    elif unit == "us":
        value, hib = ms * 1e3, False
    elif unit == "GB/s":
        nbytes = net.algorithmic_bytes() if isinstance(net, BandwidthNet) else 2 * 4 * CopyNet.C * CopyNet.S * CopyNet.S
        value, hib = nbytes / (ms * 1e-3) / 1e9, True
    else:
        value, hib = 1e3 / ms, True

    out = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": ms, "higher_is_better": hib, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
           "config": {"workload": args.workload, "input": list(x.shape), "batch": 1, "launch": launch,
                      "algorithmic_gflop_per_step": total_flops / 1e9},
           "ms_per_step_graph": ms_graph, "ms_per_step_eager": ms_eager, "roofline": roof}
    if isinstance(net, BandwidthNet):   # a single bandwidth-bound kernel: the roofline record is the step itself
        nbytes = net.algorithmic_bytes()
        ach = nbytes / (roof["avg_launch_us"] * 1e-6) / 1e9
        roof.update({"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
                     "algorithmic_bytes_per_launch": nbytes})

    if hasattr(net, "input_key") and args.workload != "copy" and not isinstance(net, BandwidthNet):
        out["host_io"] = host_io_rates(net, x, max(args.steps, 50))
        log("host I/O inclusive: %s" % out["host_io"])

    if not args.no_cpu_baseline and total_flops > 0:
        dt, flops, threads, lname = cpu_baseline(net, x, total_flops)
        cpu_ms = dt * 1e3 * total_flops / flops
        if unit == "ms/frame":
            cv = cpu_ms
        elif unit == "us":
            cv = cpu_ms * 1e3
        else:
            cv = 1e3 / cpu_ms
        out["cpu_baseline"] = {"value": cv, "unit": unit, "cores": threads, "kind": "port",
                               "sample": "layer %s at full size (%.2f GFLOP, %.2f s on %d threads), scaled by the step's %.1f GFLOP"
                                         % (lname, flops / 1e9, dt, threads, total_flops / 1e9)}
    net.cleanup()
    if hasattr(net, "input_key") and unit == "imgs/s":
        # several instances side by side: batch-1 networks of small layers are latency-bound.  (The style nets' launches
        # fill most of the chip: 2 to 4 instances of them run at the single frame pipeline's rate, 0.43-0.50 ms/frame.)
        if not args.no_pool:
            out["frame_pool"] = frame_pool_rate_in_child(args.workload, max(8 * args.steps, 400))
            log("frame pool: %s" % out["frame_pool"])

    if not args.no_also and args.workload == "stylenet":
        also = {}
        for wl in ("resnet50", "resnet50ref", "stylenet3x3ref", "stylenet9x9ref"):
            n2, m2, u2, d2 = make_net(wl)
            n2.setup()
            n2.setInput(n2.makeInput())
            ms2g = timed_forwards(n2, max(args.steps, 100), args.warmup, graph=True)
            ms2e = timed_forwards(n2, max(args.steps, 100), args.warmup, graph=False)
            ms2 = min(ms2g, ms2e)
            also[m2] = {"value": 1e3 / ms2 if u2 == "imgs/s" else ms2, "unit": u2, "ms_per_step": ms2, "ms_per_step_graph": ms2g, "ms_per_step_eager": ms2e, "dtype": d2}
            log("%s: %.4f ms/step (hipGraph) %.4f (eager)" % (wl, ms2g, ms2e))
            n2.cleanup()
            if wl == "resnet50" and not args.no_pool:
                also[m2]["frame_pool"] = frame_pool_rate_in_child(wl, 800)
        out["also"] = also
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
