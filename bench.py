#!/usr/bin/env python3
"""Benchmark of the LogicLayer kernel path on one MI355X.

Headline workload (the one BASELINE.json's metric is quoted on): bit-packed inference of the
discretised net 784 -> 6 x 64000 -> GroupSum(k=10) on 2^20 synthetic samples.  One step is
one pass of the whole path over the batch, starting from a bool [B, 784] tensor resident in
HBM: PackBitsTensor (transpose + pack, 64-bit words) -> six LogicLayers (evaluated in fused
groups) -> GroupSum bit counts [B, 10] int32.

Prints ONE JSON line.  `roofline` describes the dominant launch (the one that takes the most
time per step): its algorithmic bytes (per layer 8*W*(in+out) + 17*out, summed over the layers a
fused launch replaces) divided by the launch duration measured with events on the launch stream
inside the timed region.  `cpu_baseline`
times the CPU oracle (single thread, like the reference's generated C) on a bounded sample.
`extra.train` reports the fp32 forward+backward path (784 -> 6 x 64000, B = 512).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch-log2", type=int, default=20)
    ap.add_argument("--width", type=int, default=64000)
    ap.add_argument("--layers", type=int, default=6)
    ap.add_argument("--features", type=int, default=784)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-train", action="store_true")
    ap.add_argument("--cpu-sample-log2", type=int, default=18)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 4 plain device copies of 1 GiB (for scaling rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    return ap.parse_args()


def eval_layer_bytes(in_dim, out_dim, words):
    return 8 * words * (in_dim + out_dim) + 17 * out_dim


def packed_bench(args, torch, dl):
    F, width, L, k = args.features, args.width, args.layers, 10
    B = 1 << args.batch_log2
    W = B // 64
    torch.manual_seed(0)
    mods, d = [torch.nn.Flatten()], F
    for _ in range(L):
        mods.append(dl.LogicLayer(d, width, connections="random"))
        d = width
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, 30.0)).eval()
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.rand(B, F, device="cuda", generator=g) < 0.2

    ext = dl.difflogic_cuda
    names = ("tensor_packbits_batch_major", "eval", "eval_fused", "eval_chained", "eval_fused_groupbitsum",
             "groupbitsum")
    real = {n: getattr(ext, n) for n in names}
    launches = []          # (kernel label, algorithmic bytes, start_event, end_event)
    record = {"on": False}

    def describe(name, a):
        """(label, algorithmic bytes): per layer 8*W*(in+out) + 17*out, the count 8*W*out + 4*k*B, the
        packing B*F + F*W*8; a fused launch is charged the sum over the layers it replaces."""
        if name == "tensor_packbits_batch_major":
            return "packbits_batch_major %dx%d" % tuple(a[0].shape), B * F + 8 * W * F
        if name == "groupbitsum":
            return "groupbitsum %d" % a[0].shape[0], 8 * W * a[0].shape[0] + 4 * k * B
        if name == "eval":
            return "eval %d->%d" % (a[0].shape[0], a[3].shape[0]), eval_layer_bytes(a[0].shape[0], a[3].shape[0], W)
        dims = [a[0].shape[0]] + [l[2].shape[0] for l in a[1]]
        by = sum(eval_layer_bytes(i, o, W) for i, o in zip(dims[:-1], dims[1:]))
        label = "%s x%d %s" % (name if name != "eval_fused_groupbitsum" else "eval_fused", len(a[1]),
                               "->".join(str(d) for d in dims))
        if name == "eval_fused_groupbitsum":
            by += 8 * W * dims[-1] + 4 * k * B
            label += " +groupbitsum"
        return label, by

    def timed(name):
        def wrapper(*a, **kw):
            if not record["on"]:
                return real[name](*a, **kw)
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            y = real[name](*a, **kw)
            e.record()
            launches.append(describe(name, a) + (s, e))
            return y
        return wrapper

    for n in names:
        setattr(ext, n, timed(n))

    def step():
        with torch.no_grad():
            return model(dl.PackBitsTensor(x, bit_count=64))

    try:
        for _ in range(args.warmup):
            out = step()
        torch.cuda.synchronize()
        record["on"] = True
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    finally:
        for n in names:
            setattr(ext, n, real[n])
        record["on"] = False

    ms_per_step = elapsed / args.steps * 1e3
    per_kernel = {}
    for label, by, s, e in launches:
        d = per_kernel.setdefault(label, {"n": 0, "ms": 0.0, "bytes": by})
        d["n"] += 1
        d["ms"] += s.elapsed_time(e)
    # dominant kernel = the launch kind that takes the most time in a step
    dom = max(per_kernel, key=lambda kk: per_kernel[kk]["ms"])
    avg_ms = per_kernel[dom]["ms"] / per_kernel[dom]["n"]
    alg = per_kernel[dom]["bytes"]
    achieved = alg / (avg_ms * 1e-3) / 1e9
    total_alg = sum(v["bytes"] * v["n"] for v in per_kernel.values()) / args.steps
    roofline = {
        "bound": "hbm", "kernel": dom,
        "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": load_traffic(dom), "algorithmic_bytes_per_launch": int(alg), "avg_launch_ms": round(avg_ms, 4),
        "launches_timed": per_kernel[dom]["n"],
    }
    info = {
        "kernels": {kk: {"avg_ms": round(v["ms"] / v["n"], 4), "launches_per_step": v["n"] / args.steps,
                         "algorithmic_GB": round(v["bytes"] / 1e9, 3),
                         "GBps_algorithmic": round(v["bytes"] / (v["ms"] / v["n"] * 1e-3) / 1e9, 1)}
                    for kk, v in per_kernel.items()},
        "path_algorithmic_GB_per_step": round(total_alg / 1e9, 2),
        "path_GBps_algorithmic": round(total_alg / (ms_per_step * 1e-3) / 1e9, 1),
        "checksum": int(out.sum().item()),
    }
    return B * args.steps / elapsed, ms_per_step, roofline, info, model, x


def load_traffic(kernel_label):
    """HBM-side bytes per launch of the dominant kernel from the committed rocprofv3 --pmc summary
    (profiles/packed_kernel_traffic.json, keyed by the launch label), or None when that launch
    has not been measured."""
    p = os.path.join(ROOT, "profiles", "packed_kernel_traffic.json")
    if os.path.exists(p):
        with open(p) as f:
            entry = json.load(f).get(kernel_label)
        if entry:
            return entry.get("hbm_bytes_per_launch")
    return None


def cpu_baseline(args, model, x, dl):
    """The oracle's table-driven C interpreter (same per-word arithmetic as the C the reference
    generates), one thread, on the first 2^cpu_sample_log2 samples of the batch."""
    import numpy as np

    from oracle import interp
    layers = [(m.indices[0].cpu().numpy(), m.indices[1].cpu().numpy(),
               m.weights.argmax(-1).to("cpu").numpy().astype(np.uint8)) for m in model if isinstance(m, dl.LogicLayer)]
    n = min(1 << args.cpu_sample_log2, x.shape[0])
    xs = x[:n].cpu().numpy()
    interp.net_eval(xs[:64], layers, 10)            # load the library, touch the tables
    t0 = time.perf_counter()
    want = interp.net_eval(xs, layers, 10, threads=1)
    dt = time.perf_counter() - t0
    with __import__("torch").no_grad():
        got = model(dl.PackBitsTensor(x[:n], bit_count=64)).cpu().numpy()
    return {"value": round(n / dt, 1), "unit": "samples/s", "cores": 1, "kind": "port",
            "sample": "first %d of %d samples, same net; oracle/c/packed_interp.c, 1 thread, %.1f s" % (n, x.shape[0], dt),
            "gpu_matches_cpu_on_sample": bool((got == want).all())}


def train_bench(args, torch, dl):
    """fp32 forward + backward of 784 -> 6 x 64000 -> GroupSum(10, tau 30), B = 512, 'unique'
    connections, grad_factor 1, CrossEntropy.  Reports the whole step (eager and replayed as one
    HIP graph) and each layer kernel timed alone (back-to-back launches on a 64000 -> 64000 layer,
    forward and backward_w in their chained form; backward_chained is the single pass the layer
    runs in place of backward_w + backward_x and is charged the bytes of both)
    against its algorithmic bytes: forward 4B(in+out)+80 out, backward_w 4B(in+out)+64 out,
    backward_x 4B(2 in+out)+64 out."""
    F, width, L, k, B = 784, 64000, 6, 10, 512
    torch.manual_seed(0)
    mods, d = [torch.nn.Flatten()], F
    for _ in range(L):
        mods.append(dl.LogicLayer(d, width, connections="unique"))
        d = width
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, 30.0)).train()
    g = torch.Generator(device="cuda").manual_seed(2)
    x = (torch.rand(B, F, device="cuda", generator=g) < 0.2).float()
    labels = torch.randint(0, k, (B,), device="cuda", generator=g)
    loss_fn = torch.nn.CrossEntropyLoss()
    steps, warmup = max(5, args.steps), max(3, args.warmup)

    def step():
        model.zero_grad(set_to_none=True)
        loss = loss_fn(model(x), labels)
        loss.backward()
        return loss

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    torch.cuda.synchronize()
    eager = (time.perf_counter() - t0) / steps
    eager_loss = loss.item()

    # each layer kernel alone, 20 launches back to back on one square layer
    ext = dl.difflogic_cuda
    layer = model[2]
    a, b = layer.indices
    xs = torch.rand(width, B, device="cuda", generator=g)
    gy = torch.randn(width, B, device="cuda", generator=g)
    logits = layer.weights.detach()
    _, probs = ext.forward_logits(xs, a, b, logits)
    start, idx = layer.given_x_indices_of_y_start, layer.given_x_indices_of_y
    sched = layer._train_schedule()
    calls = {
        "forward_logits": (lambda: ext.forward_logits(xs, a, b, logits, sched), 4 * B * 2 * width + 80 * width),
        "backward_logits": (lambda: ext.backward_logits(xs, a, b, gy, probs, sched), 4 * B * 2 * width + 64 * width),
        "backward_x": (lambda: ext.backward_x(xs, a, b, probs, gy, start, idx), 4 * B * 3 * width + 64 * width),
        # backward_logits + backward_x in one pass (what the layer runs when both gradients are needed)
        "backward_chained": (lambda: ext.backward_chained(xs, probs, gy, sched, 1.0, softmax_backward=True),
                             4 * B * 5 * width + 128 * width),
    }
    kernels = {}
    for name, (fn, by) in calls.items():
        for _ in range(3):
            fn()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(20):
            fn()
        e.record()
        torch.cuda.synchronize()
        us = s.elapsed_time(e) / 20 * 1e3
        kernels[name] = {"us_per_launch": round(us, 2), "GBps_algorithmic": round(by / (us * 1e-6) / 1e9, 1),
                         "frac_hbm": round(by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
    del xs, gy

    # Drop every reference to the eager autograd graph before capturing: gradient-accumulation
    # nodes kept alive by `loss` belong to the default stream and would be replayed into the
    # capture stream's backward.
    del loss
    model.zero_grad(set_to_none=True)
    import gc
    gc.collect()
    torch.cuda.synchronize()
    from difflogic_amd.graphs import GraphedTrainStep
    graphed = GraphedTrainStep(model, loss_fn, x, labels)
    for _ in range(warmup):
        graphed.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        gl = graphed.step()
    torch.cuda.synchronize()
    replay = (time.perf_counter() - t0) / steps

    dims = [F] + [width] * L
    alg = sum(4 * B * (i + o) + 80 * o + 4 * B * (i + o) + 64 * o for i, o in zip(dims[:-1], dims[1:]))
    alg += sum(4 * B * (2 * i + o) + 64 * o for i, o in zip(dims[1:-1], dims[2:]))     # no backward_x for layer 1
    neuron_samples = L * width * B
    return {
        "workload": "fp32 fwd+bwd 784->6x64000->GroupSum(10,tau=30), B=512, connections=unique, CrossEntropy",
        "dtype": "f32", "algorithmic_GB_per_step": round(alg / 1e9, 3),
        "graph_replay": {"neuron_samples_per_s": round(neuron_samples / replay, 1), "ms_per_step": round(replay * 1e3, 4),
                         "GBps_algorithmic": round(alg / replay / 1e9, 1),
                         "frac_hbm": round(alg / replay / 1e9 / HBM_PEAK_GBS, 4), "loss": round(gl.item(), 6)},
        "eager": {"neuron_samples_per_s": round(neuron_samples / eager, 1), "ms_per_step": round(eager * 1e3, 4),
                  "loss": round(eager_loss, 6)},
        "kernels_alone_64000x64000": kernels,
    }


def train_cpu_baseline(torch):
    """Full training step (forward, CrossEntropy, backward, Adam lr 0.01) of the python
    implementation restated in oracle/float_oracle.py: 784 -> 4 x 8000 -> GroupSum(10, tau 10),
    B = 128, 'random' connections; median of 5 steps after 2 warm-ups, at 1 thread (the figure
    reported) and at torch's default thread count."""
    from oracle import connections as oc
    from oracle import float_oracle as fo
    torch.manual_seed(0)
    layers, d = [], 784
    for _ in range(4):
        lg = torch.randn(8000, 16, requires_grad=True)
        a, b = oc.random_connections(d, 8000)
        layers.append((a, b, lg))
        d = 8000
    net = fo.PythonNet(layers, 10, 10.0)
    opt = torch.optim.Adam([l[2] for l in layers], lr=0.01)
    x = (torch.rand(128, 784) < 0.2).float()
    y = torch.randint(0, 10, (128,))

    def median_step():
        times = []
        for _ in range(7):
            t0 = time.perf_counter()
            loss = torch.nn.functional.cross_entropy(net(x), y)
            opt.zero_grad()
            loss.backward()
            opt.step()
            times.append(time.perf_counter() - t0)
        return statistics.median(times[2:])

    threads = torch.get_num_threads()
    all_threads = median_step()                      # torch's default thread count
    torch.set_num_threads(1)                         # what the reference's drivers pin (experiments/main.py:17)
    try:
        med = median_step()
    finally:
        torch.set_num_threads(threads)
    return {"value": round(4 * 8000 * 128 / med, 1), "unit": "neuron-samples/s", "cores": 1, "kind": "port",
            "sample": "784->4x8000 B=128 full step (fwd+CE+bwd+Adam), median of 5, %.3f s/step" % med,
            "default_threads": {"value": round(4 * 8000 * 128 / all_threads, 1), "cores": threads,
                                "s_per_step": round(all_threads, 4)}}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path shards along the batch without "
              "communication); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch

    import difflogic_amd as dl
    assert torch.cuda.is_available(), "bench.py needs the GPU"

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    value, ms, roofline, info, model, x = packed_bench(args, torch, dl)
    result = {
        "metric": "packed-eval samples/s (784->6x64k)", "value": round(value, 1), "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int64", "data": "synthetic",
        "config": {"workload": "packed inference %d->%dx%d->GroupSum(10), batch 2^%d, int64 words, bool input "
                               "resident in HBM; step = pack + %d gate layers + groupbitsum"
                               % (args.features, args.layers, args.width, args.batch_log2, args.layers),
                   "connections": "random", "seed": 0},
        "roofline": roofline,
    }
    result["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline(args, model, x, dl)
    extra = dict(info)
    del model, x
    torch.cuda.empty_cache()
    if not args.no_train:
        extra["train"] = train_bench(args, torch, dl)
        if not args.no_cpu_baseline:
            extra["train"]["cpu_baseline"] = train_cpu_baseline(torch)
    result["extra"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
