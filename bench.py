#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: DCGAN-64 generator forward, fp32, batch 256.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

A step is one forward pass of the generator over one batch of synthetic latents that are already resident in HBM
(the fused C-ABI path: Linear, 4 x (BatchNorm + ReLU, transposed conv 4x4 s2 p1), tanh).  Order of the run: the CPU
baseline (before anything touches the GPU), W warm-up + K timed steps from a cold start (reported), a sustained
stretch of load (reported; the clocks settle; at most 300 steps under a counter run of rocprofv3), then the W warm-up +
K timed steps that `value` comes from, the same steps with the latents uploaded from the host, the K steps with
per-kernel events, and the other configurations (c1, c2, c4, c5, gan: `secondary`, --no-secondary skips them).
Prints ONE JSON line:
value = images/s of the whole step; conv_gflops / conv_frac_of_fp32_mfma_peak = algorithmic FLOPs (2*MAC, non-zero
taps only) of the four transposed convolutions over the time of their kernels; roofline = the dominant kernel
(the matrix-core implicit GEMM of the three large transposed convolutions) measured with HIP events on the
library's stream inside the timed region; cpu_baseline = the reference's CPU path (oracle/_ref when built, else
the C restatement) timed on this host on a bounded sample of the same workload.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "cuda-cnn-gan-vae_amd"))

FP32_MFMA_PEAK_TFLOPS = 157.3
BATCH = 256


def hip_events():
    """hipEvent helpers on the library's stream (torch.cuda.Event would watch torch's own stream)."""
    hip = ctypes.CDLL("libamdhip64.so")
    def create():
        e = ctypes.c_void_p()
        assert hip.hipEventCreate(ctypes.byref(e)) == 0
        return e
    def record(e, stream):
        assert hip.hipEventRecord(e, ctypes.c_void_p(stream)) == 0
    def elapsed_ms(a, b):
        assert hip.hipEventSynchronize(b) == 0
        ms = ctypes.c_float()
        assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value
    return create, record, elapsed_ms


def measured_traffic():
    """HBM-side bytes per launch of the dominant kernel, as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each
    scaled by what the same counter reads for a plain copy of known size); the summary of those runs is kept under
    profiles/ and carries the figure on a line of its own.  None when the summary is missing."""
    path = os.path.join(ROOT, "profiles", "dcgan64_b256_forward_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return int(line.split(":")[1])
    except OSError:
        pass
    return None


def cpu_baseline(sample_batch):
    """The CPU path on this host, single thread (the reference has no active OpenMP), on `sample_batch` images."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle_api                       # the checker's library, timed here as the reported baseline only
    import layer_sequences as seq
    import generator as G
    kind = "reference" if oracle_api.available("ref") else "port"
    cpu = oracle_api.Oracle("ref" if kind == "reference" else "oracle")
    params, z = G.make_parameters(), G.make_latent(sample_batch)
    t0 = time.perf_counter()
    seq.dcgan_generator_forward(cpu, params, z)
    dt = time.perf_counter() - t0
    return {"value": sample_batch / dt, "unit": "images/s", "cores": 1, "kind": kind,
            "sample": "one generator forward at batch %d (%.1f s), scaled linearly; host has %d cores" % (sample_batch, dt, os.cpu_count() or 0)}


def memory_bound_ops(args):
    """Secondary workload: the HBM-bound tensor operations on the largest activation of the measured configuration,
    [256,64,32,32] fp32 (67 MB), each timed on its own with HIP events; achieved = algorithmic bytes / time against the
    8 TB/s HBM peak.  One JSON line."""
    import numpy as np
    import mi355tensor as mt
    from mi355tensor import CTensor, CTensorApplyFunc as F, CTensorMath as M, Fused
    mt.init(0)
    W = args.ops_batch   # 256: the activation of the measured configuration (67 MB, within the 256 MB Infinity Cache)
    shape, s1 = (W, 64, 32, 32), (1, 64, 32, 32)
    n = W * 64 * 32 * 32
    rng = np.random.default_rng(0)
    a, b, out = (CTensor.from_numpy(rng.standard_normal(shape).astype(np.float32)) for _ in range(3))
    g, be, m1, v1 = (CTensor.from_numpy(np.abs(rng.standard_normal(s1)).astype(np.float32) + 0.5) for _ in range(4))
    xhat, sums, bias = CTensor(*shape), CTensor(W, 64, 1, 1), CTensor.from_numpy(np.ones((1, 64, 1, 1), np.float32))
    half, pos, up = CTensor(W, 64, 16, 16), CTensor(W, 64, 16, 16, pos=True), CTensor(W, 64, 64, 64)
    big = CTensor(W, 64, 64, 64)
    mom, vel = CTensor.from_numpy(np.zeros(shape, np.float32)), CTensor.from_numpy(np.zeros(shape, np.float32))
    B = 4.0 * n
    ops = [  # name, callable, algorithmic bytes
        ("Fill", lambda: M.Fill(out, 1.0), B),
        ("Set (copy)", lambda: M.Set(out, a, 1.0, 0.0), 2 * B),
        ("Add", lambda: M.Add(out, a, b, 1.0, 1.0), 3 * B),
        ("Add, broadcast right operand [1,Z,Y,X]", lambda: M.Add(out, a, g, 1.0, 1.0), 2 * B),
        ("TensorItemProduction", lambda: M.TensorItemProduction(out, a, b), 3 * B),
        ("Pow2", lambda: M.Pow2(out, a, 1.0), 2 * B),
        ("ApplyReLU", lambda: F.ApplyReLU(out, a), 2 * B),
        ("ApplyTangence", lambda: F.ApplyTangence(out, a), 2 * B),
        ("ApplyDifferentialLeakyReLU", lambda: F.ApplyDifferentialLeakyReLU(out, a), 2 * B),
        ("AddBias", lambda: M.AddBias(out, bias), 2 * B),
        ("AddSumW (sum over the batch)", lambda: M.AddSumW(m1, m1, a, 1.0, 1.0 / W), B),
        ("SummXY", lambda: M.SummXY(sums, a), B),
        ("batch norm forward, training mode, fused + ReLU", lambda: Fused.BatchNormForwardTrain(out, a, g, be, func="relu"), 2 * B),
        ("batch norm forward, training mode, keeping xhat", lambda: Fused.BatchNormForwardTrain(out, a, g, be, xhat, v1), 3 * B),
        ("batch norm forward, inference mode, fused + ReLU", lambda: Fused.BatchNormForwardInfer(out, a, g, be, m1, v1, func="relu"), 2 * B),
        ("batch norm backward, fused", lambda: Fused.BatchNormBackward(out, m1, v1, a, g, b, be), 3 * B),
        ("MaxPooling 2x2 (+ positions)", lambda: M.MaxPooling(half, pos, a, 2, 2), B + 3 * B / 4),
        ("MaxPoolingBackward 2x2", lambda: M.MaxPoolingBackward(out, pos, half, 2, 2), B + 3 * B / 4),
        ("UpSampling x2", lambda: M.UpSampling(up, a, 2, 2), B + 4 * B),
        ("DownSampling x2", lambda: M.DownSampling(a, big, 2, 2), 4 * B + B),
        ("Adam", lambda: M.Adam(out, a, mom, vel, W, 2e-4, 0.5, 0.999, 1e-8, 1.0), 7 * B),
    ]
    stream = mt.get_stream()
    create, record, elapsed_ms = hip_events()
    results = {}
    for name, fn, nbytes in ops:
        for _ in range(args.warmup):
            fn()
        e0, e1 = create(), create()
        record(e0, stream)
        for _ in range(args.steps):
            fn()
        record(e1, stream)
        us = elapsed_ms(e0, e1) / args.steps * 1e3
        results[name] = {"us": us, "GB/s": nbytes / us / 1e3, "frac_of_hbm_peak": nbytes / us / 1e3 / 8000.0, "algorithmic_MB": nbytes / 1e6}
    rates = [r["GB/s"] for r in results.values()]
    print(json.dumps({
        "metric": "GB/s of the HBM-bound tensor operations on a [%d,64,32,32] fp32 activation (secondary workload)" % W,
        "value": float(np.median(rates)), "unit": "GB/s (median over the operations)", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sum(r["us"] for r in results.values()) / 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "config": {"workload": "every HBM-bound operation of the tensor-op layer, one launch each per step"},
        "roofline": {"bound": "hbm", "peak": 8000.0, "unit": "GB/s", "achieved": float(np.median(rates)), "frac": float(np.median(rates)) / 8000.0},
        "operations": results}))


def discriminator_step(args):
    """Secondary workload (configs[4]): forward, backward and Adam update of the DCGAN-64 discriminator at batch 128
    through the fused entry points.  Same two timed regions as the main workload; returns the JSON object."""
    import mi355tensor as mt
    import discriminator as D
    batch = 128
    net = D.Discriminator(batch)
    net.set_batch(*D.make_batch(batch))
    stream = mt.get_stream()
    create, record, elapsed_ms = hip_events()
    for _ in range(args.warmup):
        net.step(fused=True)
    mt.synchronize()
    # The calls issued one by one come first: once a recorded graph writes the weights, the library no longer trusts the
    # re-ordered copies it keeps of them (a replay changes the weights without a call that it sees) and re-orders them on
    # every use, which a training loop that records nothing -- the reference's own -- never pays.
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.step(fused=True)
    mt.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3
    mt.profile_enable(True)
    for _ in range(args.steps):
        net.step(fused=True)
    prof = mt.profile_report()
    mt.profile_enable(False)
    # the step is recorded once as a HIP graph and replayed; Adam's iteration count is an argument of the recorded
    # kernels, so the replays repeat one iteration (same work, same arithmetic)
    graph = mt.Graph(lambda: net.step(fused=True))
    for _ in range(3):
        graph.launch()
    mt.synchronize()
    e0, e1 = create(), create()
    t0 = time.perf_counter()
    record(e0, stream)
    for _ in range(args.steps):
        graph.launch()
    record(e1, stream)
    mt.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = elapsed_ms(e0, e1)
    graph_ms_per_step = max(gpu_ms, wall_ms) / args.steps
    ms_per_step = min(graph_ms_per_step, eager_ms / args.steps)   # whichever way of issuing the same step is faster
    conv = {k: v for k, v in prof.items() if k.startswith(("mt_forward_convolution", "mt_backward_convolution", "mt_convolution_backward_weights_sum"))}
    conv_ms = sum(v[1] for v in conv.values()) / args.steps
    flop = 3.0 * sum(D.conv_flops(batch))   # forward, input gradient, weight gradient
    return ({
        "metric": "images/sec, DCGAN-64 discriminator training step fp32 b=128 (secondary workload)",
        "value": batch / (ms_per_step * 1e-3), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[4]: DCGAN-64 discriminator, batch 128: conv 4x4 s2 p1 3->64->128->256->512 with BN + leaky ReLU, "
                               "Linear 8192->1, sigmoid; forward, backward (input, weight, bias, BN gradients), Adam", "global_batch": batch,
                   "path": "fused C-ABI entry points, " + ("step replayed as a HIP graph" if graph_ms_per_step <= eager_ms / args.steps
                                                           else "calls issued one by one from Python")},
        "ms_per_step_graph_replay": graph_ms_per_step,
        "gpu_ms_per_step_events": gpu_ms / args.steps, "host_ms_per_step_wall": wall_ms / args.steps,
        "ms_per_step_eager_from_python": eager_ms / args.steps,
        "kernel_ms_per_step_sum": sum(v[1] for v in prof.values()) / args.steps,
        "conv_gflops": flop / (conv_ms * 1e-3) / 1e9, "conv_ms_per_step": conv_ms,
        "conv_frac_of_fp32_mfma_peak": flop / (conv_ms * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS,
        "gflop_per_step": {"conv": flop / 1e9},
        "tflops_over_the_step": flop / (ms_per_step * 1e-3) / 1e12,
        "frac_of_fp32_mfma_peak_over_the_step": flop / (ms_per_step * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS,
        "kernels_ms_per_step": {k: v[1] / args.steps for k, v in sorted(prof.items(), key=lambda kv: -kv[1][1])}})


def secondary_forward(args):
    """Secondary workloads configs[0], configs[1], configs[3]: one forward pass per step, timed twice -- recorded once as a
    HIP graph and replayed, and issued call by call from Python -- the faster of the two is the step; then the steps with
    per-kernel events.  Returns the JSON object."""
    import numpy as np
    import mi355tensor as mt
    from mi355tensor import CTensor, CTensorConv, Fused
    mt.init(0)
    rng = np.random.default_rng({"c1": 1, "c2": 2, "c4": 4, "gan": 6}[args.workload])
    if args.workload == "c1":
        batch, name = 16, "configs[0]: one convolution layer, batch 16: 3x64x64 -> 32 filters 5x5 stride 1 padding 2, leaky ReLU"
        image = CTensor.from_numpy(rng.uniform(-1, 1, (16, 3, 64, 64)).astype(np.float32))
        kernel = CTensor.from_numpy((rng.standard_normal((1, 1, 32, 75)) * np.sqrt(2.0 / 75)).astype(np.float32))
        bias, out = CTensor.from_numpy(np.zeros((1, 32, 1, 1), np.float32)), CTensor(16, 32, 64, 64)
        flop = {"conv": 2.0 * 16 * 32 * 64 * 64 * 75}
        step = lambda: CTensorConv.ForwardConvolution(out, image, kernel, 5, 5, 3, 32, bias, 1, 1, 2, 2, func="leaky_relu")
    elif args.workload == "c2":
        batch, name = 256, "configs[1]: Linear 4096 -> 3072, ReLU, Linear 3072 -> 768, batch 256"
        x = CTensor.from_numpy(rng.standard_normal((256, 1, 4096, 1)).astype(np.float32))
        w1 = CTensor.from_numpy(rng.uniform(-1, 1, (1, 1, 3072, 4096)).astype(np.float32) * np.float32(np.sqrt(6 / 7168)))
        w2 = CTensor.from_numpy(rng.uniform(-1, 1, (1, 1, 768, 3072)).astype(np.float32) * np.float32(np.sqrt(6 / 3840)))
        b1, b2 = CTensor.from_numpy(np.full((1, 1, 3072, 1), 0.1, np.float32)), CTensor.from_numpy(np.full((1, 1, 768, 1), 0.1, np.float32))
        h, out = CTensor(256, 1, 3072, 1), CTensor(256, 1, 768, 1)
        flop = {"linear": 2.0 * 256 * (4096 * 3072 + 3072 * 768)}

        def step():
            Fused.LinearForward(h, w1, x, b1, "relu")
            Fused.LinearForward(out, w2, h, b2)
    elif args.workload == "gan":
        import gan_generator as GG
        batch, name = GG.BATCH, ("the reference's shipped GAN generator (cmodel_gan.cu.h), batch 32: Linear 1024 -> 3*4*512, six times (up-sampling x2, "
                                 "conv 3x3, BN, leaky ReLU) 512 -> 512 -> 256 -> 128 -> 64 -> 32 -> 16, conv 3x3 -> 3, tanh: 192x256 images; "
                                 + ("layer by layer" if args.literal else "up-sampling + convolution in one call"))
        net = GG.GanGenerator(batch)
        net.set_noise(GG.make_noise(batch))
        layers = GG.conv_flops(batch)
        # the one-call path multiplies 4 taps per output pixel where the layers multiply 9 (sums of coefficients)
        executed = sum(layers) if args.literal else sum(layers[:6]) * 4.0 / 9.0 + layers[6]
        flop = {"conv_executed": executed, "linear": 2.0 * batch * 1024 * 6144}
        extra = {"conv_gflop_as_the_layers_count_it": sum(layers) / 1e9}
        step = (lambda: net.forward(False)) if args.literal else (lambda: net.forward(True))
    else:
        import vae
        batch, name = 64, ("configs[3]: VAE forward, batch 64: conv 3x3 s2 p1 3->32->64->128->256 with BN + leaky ReLU, Linear 16384->128 x2, "
                           "reparameterisation + KL, Linear 128->16384, transposed conv 4x4 s2 p1 256->128->64->32->3, sigmoid")
        net = vae.Vae(batch)
        net.set_batch(*vae.make_batch(batch))
        flop = vae.flops(batch)
        step = net.forward
    if args.workload != "gan":
        extra = {}
    stream = mt.get_stream()
    create, record, elapsed_ms = hip_events()
    for _ in range(max(args.warmup, 1)):
        step()
    mt.synchronize()
    graph = mt.Graph(step)
    for _ in range(3):
        graph.launch()
    mt.synchronize()
    e0, e1 = create(), create()
    t0 = time.perf_counter()
    record(e0, stream)
    for _ in range(args.steps):
        graph.launch()
    record(e1, stream)
    mt.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = elapsed_ms(e0, e1)
    # the same steps issued call by call: a node of a replayed graph starts about 3 us after the one before it, launches
    # queued back to back on the stream follow each other more closely, as long as the host keeps ahead of the GPU
    for _ in range(max(args.warmup, 1)):
        step()
    mt.synchronize()
    e2, e3 = create(), create()
    t0 = time.perf_counter()
    record(e2, stream)
    for _ in range(args.steps):
        step()
    record(e3, stream)
    mt.synchronize()
    eager_wall_ms = (time.perf_counter() - t0) * 1e3
    eager_gpu_ms = elapsed_ms(e2, e3)
    mt.profile_enable(True)
    for _ in range(args.steps):
        step()
    prof = mt.profile_report()
    mt.profile_enable(False)
    graph_ms, eager_ms = max(gpu_ms, wall_ms) / args.steps, max(eager_gpu_ms, eager_wall_ms) / args.steps
    ms_per_step = min(graph_ms, eager_ms)
    path = "step replayed as a HIP graph" if graph_ms <= eager_ms else "calls issued one by one from Python"
    if eager_ms < graph_ms:
        gpu_ms, wall_ms = eager_gpu_ms, eager_wall_ms
    kernel_ms = sum(v[1] for v in prof.values()) / args.steps
    total = sum(flop.values())
    return ({
        "metric": "images/sec, forward fp32 (secondary workload)" if args.workload != "c2" else "samples/sec, forward fp32 (secondary workload)",
        "value": batch / (ms_per_step * 1e-3), "unit": "images/s" if args.workload != "c2" else "samples/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic", "config": {"workload": name, "global_batch": batch, "path": "fused C-ABI entry points, " + path},
        "ms_per_step_graph_replay": graph_ms, "ms_per_step_calls_from_python": eager_ms,
        "gpu_ms_per_step_events": gpu_ms / args.steps, "host_ms_per_step_wall": wall_ms / args.steps, "kernel_ms_per_step_sum": kernel_ms,
        "gflop_per_step": dict({k: v / 1e9 for k, v in flop.items()}, **extra),
        "tflops_over_the_step": total / (ms_per_step * 1e-3) / 1e12,
        "frac_of_fp32_mfma_peak_over_the_step": total / (ms_per_step * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS,
        "kernels_ms_per_step": {k: v[1] / args.steps for k, v in sorted(prof.items(), key=lambda kv: -kv[1][1])}})


def secondary_workloads(steps, warmup):
    """The other configurations and the shipped GAN generator, a few hundred steps each, in this process after the
    measured workload: {name: {ms_per_step, tflops, frac_of_fp32_mfma_peak, ...}} for the `secondary` object of the
    default run's JSON line.  Algorithmic FLOP over the whole step, convolution kernels beside it where they dominate."""
    out = {}
    for wl in ("c1", "c2", "c4", "c5", "gan"):
        a = argparse.Namespace(workload=wl, steps=steps, warmup=warmup, literal=False)
        full = discriminator_step(a) if wl == "c5" else secondary_forward(a)
        brief = {"workload": full["config"]["workload"], "steps": steps, "warmup": warmup, "ms_per_step": full["ms_per_step"],
                 "value": full["value"], "unit": full["unit"], "gflop_per_step": sum(v for k, v in full["gflop_per_step"].items() if not k.startswith("conv_gflop_as")),
                 "tflops": full["tflops_over_the_step"], "frac_of_fp32_mfma_peak": full["frac_of_fp32_mfma_peak_over_the_step"],
                 "path": full["config"]["path"]}
        if "conv_frac_of_fp32_mfma_peak" in full:
            brief["conv_kernels_frac_of_fp32_mfma_peak"] = full["conv_frac_of_fp32_mfma_peak"]
        top = sorted(full["kernels_ms_per_step"].items(), key=lambda kv: -kv[1])[:4]
        brief["largest_kernels_ms_per_step"] = {k: round(v, 5) for k, v in top}
        out[wl] = brief
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--cpu-sample-batch", type=int, default=40,
                    help="images of the CPU baseline sample (about 0.3 s each on one core)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="workload c3: leave out the `secondary` object (the other configurations, about 3 s)")
    ap.add_argument("--secondary-steps", type=int, default=200, help="steps per secondary workload inside the default run")
    ap.add_argument("--copy-mib", type=int, default=0,
                    help="also launch one plain copy (mt_set) of this many MiB before the timed region: the known-size kernel "
                         "that calibrates the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    ap.add_argument("--sustained-steps", type=int, default=0,
                    help="steps of the sustained region (default: at least 2000, about a second of GPU work; counter runs of "
                         "rocprofv3 --pmc, which intercept every dispatch, use a few hundred)")
    ap.add_argument("--graph", action="store_true",
                    help="time region 1 as replays of the step recorded once as a HIP graph (c5 does so by default: its step "
                         "is about a hundred short kernels and the Python host would be the bottleneck)")
    ap.add_argument("--ops-batch", type=int, default=256, help="workload ops: batch size of the [W,64,32,32] activation (1024: 268 MB per tensor)")
    ap.add_argument("--literal", action="store_true", help="workload gan: up-sampling and convolution as two layers")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="mt_set_option before the run (measurements: tconv_walk=0, pack_cache=0, igemm_tile=3 ...); may be repeated")
    ap.add_argument("--linear-bn", type=int, default=None, metavar="0|1",
                    help="workload c3: Linear layer and its batch norm as one launch (1) or two (0); default: the generator's own choice")
    ap.add_argument("--fold", default=None, metavar="LAYERS",
                    help="workload c3: batch norms folded into the convolutions around them, e.g. 3 or 1,2,3 or none (default: the generator's own choice)")
    ap.add_argument("--workload", choices=["c3", "c5", "ops", "c1", "c2", "c4", "gan"], default="c3",
                    help="c3 (default, the measured configuration): DCGAN-64 generator forward, batch 256; "
                         "c5 (secondary): DCGAN-64 discriminator training step, batch 128; "
                         "c1, c2, c4 (secondary): one convolution layer at batch 16, a two-layer MLP at batch 256, the VAE forward at batch 64; "
                         "gan (secondary): the reference's shipped GAN generator at batch 32 (--literal: up-sampling and convolution as two layers); "
                         "ops (secondary): every HBM-bound tensor operation on a [256,64,32,32] activation, GB/s each")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (--gpus 1); the path would shard along the batch axis, one all-reduce of the batch-norm sums per layer")
    if args.option:
        import mi355tensor as mt_
        mt_.init(0)
        for item in args.option:
            name, value = item.split("=")
            mt_.set_option(name, int(value))
    if args.workload == "c5":
        return print(json.dumps(discriminator_step(args)))
    if args.workload == "ops":
        return memory_bound_ops(args)
    if args.workload in ("c1", "c2", "c4", "gan"):
        return print(json.dumps(secondary_forward(args)))

    # The CPU baseline runs first (about 12 s of host work), so that everything that follows is GPU work back to back:
    # a coarse GPU-busy sample taken from outside during the second half of the run sees the GPU at work.
    baseline = None if args.no_cpu_baseline else cpu_baseline(args.cpu_sample_batch)

    import mi355tensor as mt
    import generator as G

    net = G.DcganGenerator(BATCH)
    if args.fold is not None:
        net.fold = () if args.fold == "none" else tuple(int(v) for v in args.fold.split(","))
    if args.linear_bn is not None:
        net.fuse_linear_bn = bool(args.linear_bn)
    net.set_latent(G.make_latent(BATCH))
    stream = mt.get_stream()
    create, record, elapsed_ms = hip_events()

    step = net.forward_fused
    if args.graph:
        step()                       # workspaces and kept weights exist before the recording
        mt.synchronize()
        graph = mt.Graph(net.forward_fused)
        step = graph.launch

    def timed_region(steps):
        """W untimed warm-up steps, then `steps` steps with one event per step boundary on the work stream and the host
        wall clock beside them.  Returns (milliseconds between first and last event, wall milliseconds, per-step list)."""
        for _ in range(args.warmup):
            step()
        marks = [create() for _ in range(steps + 1)]
        mt.synchronize()
        t0 = time.perf_counter()
        record(marks[0], stream)
        for i in range(steps):
            step()
            record(marks[i + 1], stream)
        mt.synchronize()
        wall = (time.perf_counter() - t0) * 1e3
        per_step = [elapsed_ms(marks[i], marks[i + 1]) for i in range(steps)]
        return elapsed_ms(marks[0], marks[steps]), wall, per_step

    # Region 0 (reported, not `value`): the first K steps of the process after W warm-up steps.  The GPU raises its
    # clocks over the first tens of milliseconds of load, so these steps run slower than the same steps of a job that
    # has been running for a moment.
    cold_gpu_ms, cold_wall_ms, _ = timed_region(args.steps)
    # Sustained load: long enough (about 1 s) for the clocks to settle, and for a GPU-busy sample from outside to
    # see the GPU working; its average is reported as ms_per_step_sustained.
    sustained_steps = args.sustained_steps if args.sustained_steps > 0 else max(2000, 4 * args.steps)
    # A counter run of rocprofv3 (--pmc sets ROCPROF_COUNTER_COLLECTION for the program it starts) serialises and
    # intercepts every dispatch; with tens of thousands of them its own tool library has ended in a segmentation fault.
    # The counters of a kernel do not depend on the number of steps: a few hundred are enough there.
    counters_on = os.environ.get("ROCPROF_COUNTER_COLLECTION", "").lower() not in ("", "0", "false")
    if counters_on and sustained_steps > 300:
        sustained_steps = 300
    s0, s1 = create(), create()
    record(s0, stream)
    for _ in range(sustained_steps):
        step()
    record(s1, stream)
    sustained_ms = elapsed_ms(s0, s1) / sustained_steps
    if args.copy_mib:
        n = args.copy_mib * 1024 * 1024 // 4
        src, dst = mt.CTensor(1, 1, n // 1024, 1024), mt.CTensor(1, 1, n // 1024, 1024)
        mt.CTensorMath.Fill(src, 1.0)
        mt.CTensorMath.Set(dst, src, 1.0, 0.0)   # reads and writes copy_mib MiB each
        mt.synchronize()

    # Timed region 1 (-> value): W warm-up steps, then exactly K steps between events on the work stream, host wall clock
    # beside it; the larger of the two counts.  The median of the per-step times is reported beside the mean.
    gpu_ms, wall_ms, per_step_ms = timed_region(args.steps)
    median_ms = sorted(per_step_ms)[len(per_step_ms) // 2]

    # The same K steps with the latents coming from the host: one 100 KB upload (mt_copy_h2d, which waits for the copy)
    # in front of every step, wall clock around the K steps.
    latent_host = G.make_latent(BATCH)
    mt.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.set_latent(latent_host)
        step()
    mt.synchronize()
    h2d_ms = (time.perf_counter() - t0) * 1e3

    # Timed region 2 (-> roofline, per-kernel times): the same K steps with every kernel launch bracketed by two HIP
    # events on the work stream.  The ~40 extra event records per step cost about 0.1 ms of stream time between the
    # kernels, which is why this region is not the one `value` is taken from; kernel durations themselves are unaffected.
    mt.profile_enable(True)
    mt.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.forward_fused()
    mt.synchronize()
    profiled_wall_ms = (time.perf_counter() - t0) * 1e3
    prof = mt.profile_report()
    mt.profile_enable(False)

    ms_per_step = max(gpu_ms, wall_ms) / args.steps
    flops = G.conv_flops(BATCH)
    conv_kernels = {k: v for k, v in prof.items() if k.startswith("mt_backward_convolution")}
    conv_ms = sum(v[1] for v in conv_kernels.values()) / args.steps
    conv_tflops = sum(flops) / (conv_ms * 1e-3) / 1e12

    # dominant kernel: the matrix-core implicit GEMM of the three large layers.  Its label carries the GEMM shape
    # "M<Cout> N<batch*pixels per phase> K<Cin*taps> x<phases>", i.e. 2*M*N*K*phases algorithmic FLOP per launch
    # (= 2*B*Cin*Hin*Win*Cout*16 of the layer: every phase multiplies only its own non-zero taps).
    import re
    big = []
    for k, v in conv_kernels.items():
        m = re.search(r"M(\d+) N(\d+) K(\d+) x(\d+)", k)
        if m:
            M_, N_, K_, X_ = (int(g) for g in m.groups())
            big.append((k, v[0], v[1], 2.0 * M_ * N_ * K_ * X_))
    dom_label = big[0][0].split(" M")[0] if big else None
    dom_launches = sum(b[1] for b in big)
    dom_ms = sum(b[2] for b in big)
    flop_per_launch = sum(b[1] * b[3] for b in big) / dom_launches if dom_launches else 0.0
    achieved = flop_per_launch / (dom_ms / dom_launches * 1e-3) / 1e12 if dom_launches else 0.0

    result = {
        "metric": "images/sec, DCGAN-64 generator fwd fp32 b=256 (conv GFLOP/s and % fp32 MFMA peak beside it)",
        "value": BATCH / (ms_per_step * 1e-3),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[2]: DCGAN-64 generator forward, batch 256, latent 100 -> 512x4x4 -> 256 -> 128 -> 64 -> 3x64x64, BN(batch stats)+ReLU, tanh",
                   "global_batch": BATCH, "path": "fused C-ABI entry points"},
        "conv_gflops": conv_tflops * 1e3,
        "conv_ms_per_step": conv_ms,
        "conv_frac_of_fp32_mfma_peak": conv_tflops / FP32_MFMA_PEAK_TFLOPS,
        "gpu_ms_per_step_events": gpu_ms / args.steps,
        "host_ms_per_step_wall": wall_ms / args.steps,
        "ms_per_step_median": median_ms,
        "ms_per_step_with_h2d": h2d_ms / args.steps,
        "ms_per_step_first_steps_of_the_process": max(cold_gpu_ms, cold_wall_ms) / args.steps,
        "ms_per_step_sustained": sustained_ms, "sustained_steps": sustained_steps,
        "ms_per_step_with_per_kernel_events": profiled_wall_ms / args.steps,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / FP32_MFMA_PEAK_TFLOPS, "traffic": measured_traffic(), "traffic_unit": "bytes per launch",
                     "traffic_source": "profiles/dcgan64_b256_forward_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, not measured in this run)",
                     "kernel": dom_label,
                     "launches_per_step": dom_launches / args.steps, "avg_launch_ms": dom_ms / dom_launches if dom_launches else None,
                     "flop_per_launch": flop_per_launch,
                     "per_layer": {b[0]: {"avg_launch_ms": b[2] / b[1], "tflops": b[3] / (b[2] / b[1] * 1e-3) / 1e12} for b in big}},
        "kernels_ms_per_step": {k: v[1] / args.steps for k, v in sorted(prof.items(), key=lambda kv: -kv[1][1])},
    }
    if baseline is not None:
        result["cpu_baseline"] = baseline
    if not args.no_secondary:
        # the other configurations, measured by the same process right after the measured workload (python bench.py --workload
        # c1|c2|c4|c5|gan prints each one's full line)
        result["secondary"] = secondary_workloads(args.secondary_steps, 20)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
