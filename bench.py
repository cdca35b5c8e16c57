#!/usr/bin/env python3
"""Benchmark of the LogicLayer kernel path on one MI355X.

Headline workload (the one BASELINE.json's metric is quoted on): bit-packed inference of the
discretised net 784 -> 6 x 64000 -> GroupSum(k=10) on 2^20 synthetic samples.  One step is
one pass of the whole path over the batch, starting from a bool [B, 784] tensor resident in
HBM: PackBitsTensor (transpose + pack, 64-bit words) -> six LogicLayers (evaluated in fused
groups) -> GroupSum bit counts [B, 10] int32.

Prints ONE JSON line.

`roofline` describes the dominant launch (the one that takes the most time per step), timed with
events on the launch stream inside the timed region.  A fused launch replaces several layers and
moves fewer bytes than their algorithmic sum, so two figures are kept apart:
  * `achieved` / `frac`: bytes the launch really moved between the L2 caches and the memory fabric
    (`traffic`, from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary of this very
    kernel source, see profiles/packed_kernel_traffic.json) divided by the launch time, against
    the 8 TB/s HBM peak; `bound` names the resource the counters show as binding;
  * `alg_GBps` / `alg_over_peak`: the algorithmic bytes (per layer 8*W*(in+out) + 17*out, summed
    over the layers the launch replaces, plus 8*W*out + 4*k*B for the count) divided by the same
    time.  This ratio can exceed 1 for a fused launch and is not a bandwidth.
When the committed traffic summary was taken from other kernel sources than the built ones,
`traffic` is null, a warning goes to stderr, and `achieved`/`frac` fall back to null.

`cpu_baseline` is the reference's CPU inference path: the C text CompiledLogicNet generates for the
headline net, gcc-compiled as the reference's driver does and timed single-threaded on a bounded sample.
gcc needs minutes for 384 000 gates, so it is started as a child process before anything touches the GPU
and collected after the GPU work; the table interpreter's figure is kept beside it.  `extra.configs` holds the other BASELINE configurations: C2 and C4 (packed inference,
checked bit-exactly against the CPU interpreter on the first 4096 samples of the full-batch
result), C3 and C5 (fp32 training forward+backward, with and without the Adam step, eager and as a
replayed HIP graph) and C1 on the GPU next to the CPU python-implementation step.

`python bench.py --ceilings` instead measures plain streaming and gather kernels (the practical
ceilings the kernels are compared with) and prints them as one JSON line.
"""
import argparse
import ctypes
import gc
import hashlib
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "packed_kernel_traffic.json")
TRAIN_TRAFFIC_JSON = os.path.join(ROOT, "profiles", "train_step_traffic.json")
# what the measured traffic of a training step depends on
TRAIN_TRAFFIC_SOURCES = ("difflogic_amd/csrc/train.hip", "difflogic_amd/csrc/schedule.cpp", "difflogic_amd/csrc/dl_common.h",
                         "difflogic_amd/difflogic.py")
# what the measured traffic of the packed launches depends on: the kernels and the launch plan
TRAFFIC_SOURCES = ("difflogic_amd/csrc/packed.hip", "difflogic_amd/csrc/lds_net.hip", "difflogic_amd/csrc/count_chain.h", "difflogic_amd/csrc/schedule.cpp",
                   "difflogic_amd/csrc/dl_common.h", "difflogic_amd/packbitstensor.py")


# seconds of untimed steps ahead of each warm-up (packed_run, train_config's timeit); --no-settle zeroes them
SETTLE_S = {"packed": 0.3, "train": 0.2}


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
    ap.add_argument("--no-train", action="store_true", help="skip the training configurations (C1, C3, C5)")
    ap.add_argument("--no-configs", action="store_true", help="skip the other packed configurations (C2, C4, other word widths)")
    ap.add_argument("--only", default="", help="comma list out of c1,c2,c3,c4,c5: run only these extra configurations")
    ap.add_argument("--skip-headline", action="store_true",
                    help="profiling aid: run only the configurations selected with --only and print their results")
    ap.add_argument("--gate-mix", default="uniform", choices=("uniform", "two_input_gates_only", "half_pass_through"),
                    help="profiling aid: run the headline with this gate mix (see GATE_MIXES) instead of the BASELINE config's")
    ap.add_argument("--train-eager-only", default="", choices=("", "written", "fused"),
                    help="profiling aid: of a training configuration run only the eager forward+backward loop of the model "
                         "as written for the reference, or of the fuse_for_training model (for whole-step counters)")
    ap.add_argument("--no-settle", action="store_true",
                    help="profiling aid: leave out the untimed steps ahead of each warm-up (counter runs record every "
                         "dispatch; per-launch figures do not depend on them)")
    ap.add_argument("--cpu-sample-log2", type=int, default=18)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 4 plain device copies of 1 GiB (for scaling rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--no-cpu-generated-c", action="store_true",
                    help="do not compile and time the reference's own CPU inference path (the generated C of the headline "
                         "net and of C2, gcc-compiled as experiments/main.py:362 does: minutes of gcc next to the GPU work); "
                         "cpu_baseline is then the table interpreter")
    ap.add_argument("--cpu-generated-c-sample-log2", type=int, default=18)
    ap.add_argument("--ceilings", action="store_true",
                    help="measure streaming read/write/copy and row-gather ceilings instead of the benchmark")
    return ap.parse_args()


def source_hash(sources=TRAFFIC_SOURCES):
    """sha256 over the sources the measured traffic depends on (default: the packed launches')."""
    h = hashlib.sha256()
    for rel in sources:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(rel.encode() + b"\0" + f.read() + b"\0")
    return h.hexdigest()[:16]


def eval_layer_bytes(in_dim, out_dim, words):
    return 8 * words * (in_dim + out_dim) + 17 * out_dim


# ------------------------------------------------------------------------------------------
# packed inference
# ------------------------------------------------------------------------------------------

def bernoulli_input(torch, B, F, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.rand(B, F, device="cuda", generator=g) < 0.2


def thresholded_input(torch, B, seed, as_float=False):
    """3x32x32 uniform values thresholded at 1/4, 2/4, 3/4 and concatenated on the channel axis
    (experiments/main.py:57 with 3 thresholds): [B, 9216]."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    out = torch.empty(B, 9216, dtype=torch.float32 if as_float else torch.bool, device="cuda")
    step = 1 << 14
    for s in range(0, B, step):
        u = torch.rand(min(step, B - s), 3, 32, 32, device="cuda", generator=g)
        bits = torch.cat([u > (i + 1) / 4 for i in range(3)], dim=1).flatten(1)
        out[s:s + step] = bits.float() if as_float else bits
    return out


LOGIT_SEED_OFFSET = 1000


def packed_model(torch, dl, F, widths, k, seed=0, connections="random"):
    """Flatten -> LogicLayer x L -> GroupSum as a user of the reference writes it.  The wiring is what LogicLayer
    draws after torch.manual_seed(seed); the gate logits are N(0,1) from a CPU generator of their own (seed +
    LOGIT_SEED_OFFSET) copied into the layers, so that the same net can be made without a GPU (cpu_side_net)."""
    torch.manual_seed(seed)
    mods, d = [torch.nn.Flatten()], F
    for w in widths:
        mods.append(dl.LogicLayer(d, w, connections=connections))
        d = w
    g = torch.Generator().manual_seed(seed + LOGIT_SEED_OFFSET)
    with torch.no_grad():
        for m in mods[1:]:
            m.weights.copy_(torch.randn(m.out_dim, 16, generator=g))
    return torch.nn.Sequential(*mods, dl.GroupSum(k, 30.0)).eval()


def cpu_side_net(torch, F, widths, seed=0, connections="random"):
    """[(a, b, gate ids)] (numpy) of the net packed_model builds from the same arguments, made on the CPU alone, so
    that the compile of its generated C can start before anything touches the GPU: the wiring as LogicLayer draws it
    (oracle.connections: the CPU default generator after torch.manual_seed(seed); the layers' initial weights come
    from the device's generator and do not advance it), the gate ids as the argmax of packed_model's logits.
    Part of the CPU-baseline leg; main() checks the GPU model's own tables against these."""
    import numpy as np
    from oracle import connections as oc
    draw = {"random": oc.random_connections, "unique": oc.unique_connections}[connections]
    torch.manual_seed(seed)
    wiring, d = [], F
    for w in widths:
        wiring.append(draw(d, w))
        d = w
    g = torch.Generator().manual_seed(seed + LOGIT_SEED_OFFSET)
    return [(a.numpy(), b.numpy(), torch.randn(len(a), 16, generator=g).argmax(-1).numpy().astype(np.uint8))
            for a, b in wiring]


def gate_mix(layers):
    """Share of gate ids, over all layers, that look at both inputs / one input / none."""
    import numpy as np
    ids = np.concatenate([np.asarray(l[2]) for l in layers])
    one = np.isin(ids, (3, 5, 10, 12)).mean()
    none = np.isin(ids, (0, 15)).mean()
    return {"two_input": round(float(1 - one - none), 4), "one_input": round(float(one), 4), "constant": round(float(none), 4)}


def packed_run(torch, dl, model, x, k, steps, warmup, graph=True):
    """Times `steps` passes of pack -> layers -> counts over x; returns (samples/s, ms per step,
    per-launch table, last output).  Every binding call of the path is bracketed by events on the
    launch stream."""
    B, F = x.shape
    W = B // 64
    ext = dl.difflogic_cuda
    names = ("tensor_packbits_batch_major", "tensor_packbits_batch_major_rows", "eval", "eval_fused", "eval_chained", "eval_fused_groupbitsum",
             "eval_chained_groupbitsum", "eval_net_lds", "eval_net_lds_bool", "groupbitsum")
    names = tuple(n for n in names if hasattr(ext, n))
    real = {n: getattr(ext, n) for n in names}
    launches = []          # (kernel label, algorithmic bytes, start_event, end_event)
    record = {"on": False}

    def describe(name, a):
        """(label, algorithmic bytes): per layer 8*W*(in+out) + 17*out, the count 8*W*out + 4*k*B, the
        packing B*F + F*W*8; a fused launch is charged the sum over the layers it replaces."""
        if name in ("tensor_packbits_batch_major", "tensor_packbits_batch_major_rows"):
            return "packbits_batch_major %dx%d" % tuple(a[0].shape), B * F + 8 * W * F
        if name == "groupbitsum":
            return "groupbitsum %d" % a[0].shape[0], 8 * W * a[0].shape[0] + 4 * k * B
        if name == "eval":
            return "eval %d->%d" % (a[0].shape[0], a[3].shape[0]), eval_layer_bytes(a[0].shape[0], a[3].shape[0], W)
        from_bool = name == "eval_net_lds_bool"           # x [B, F] bool: the packing happens inside the launch
        dims = [a[0].shape[1] if from_bool else a[0].shape[0]] + [l[2].shape[0] for l in a[1]]
        by = sum(eval_layer_bytes(i, o, W) for i, o in zip(dims[:-1], dims[1:])) + (B * F + 8 * W * F if from_bool else 0)
        counted = name in ("eval_fused_groupbitsum", "eval_chained_groupbitsum", "eval_net_lds", "eval_net_lds_bool")
        base = {"eval_fused_groupbitsum": "eval_fused", "eval_chained_groupbitsum": "eval_chained"}.get(name, name)
        label = "%s x%d %s" % (base, len(a[1]), "->".join(str(d) for d in dims))
        if from_bool:
            label = "packbits + " + label
        if counted:
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
        t_first = time.perf_counter()
        out = step()
        torch.cuda.synchronize()
        first_call_ms = (time.perf_counter() - t_first) * 1e3       # includes the host-side schedule / order builds
        # untimed: a third of a second of the same steps ahead of the warm-up proper, so that clocks and caches have
        # settled however few warm-up steps were asked for (the first launches of a process run up to 1.5x slower)
        # (back to back, as the timed steps run: launches that follow an idle GPU run slower for a while, so the host
        # waits for the stream every eighth step only, which bounds the queue)
        t_settle = time.perf_counter() + SETTLE_S["packed"]
        while time.perf_counter() < t_settle:
            for _ in range(8):
                out = step()
            torch.cuda.synchronize()
        for _ in range(max(0, warmup - 1)):
            out = step()
        torch.cuda.synchronize()
        # the timed region: exactly `steps` steps, nothing else on the stream
        t0 = time.perf_counter()
        for _ in range(steps):
            out = step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        # the same steps once more with a pair of events around every launch, for the per-launch durations: the
        # timing events drain the queue between kernels (about 8 % of a step), so they stay out of the pass above
        record["on"] = True
        t0 = time.perf_counter()
        for _ in range(steps):
            out = step()
        torch.cuda.synchronize()
        elapsed_with_events = time.perf_counter() - t0
    finally:
        for n in names:
            setattr(ext, n, real[n])
        record["on"] = False

    graph_info = None
    if graph:
        # the same step captured once into a HIP graph and replayed (difflogic_amd.graphs.GraphedPackedInference;
        # the batch sits in the graph's static input buffer, as the eager step's sits in x)
        from difflogic_amd.graphs import GraphedPackedInference
        graphed = GraphedPackedInference(model, x, bit_count=64)
        # (capturing leaves the GPU idle for milliseconds, after which launches run up to 1.3x slower for some twenty
        # steps: the replays get the warm-up the eager steps had)
        for _ in range(max(warmup, 20)):
            graphed()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            replayed = graphed()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) / steps * 1e3
        graph_info = {"ms_per_step": round(graph_ms, 4), "samples_per_s": round(B / graph_ms * 1e3, 1),
                      "equal_to_eager": bool(torch.equal(replayed, out)),
                      "eager_ms_per_step_with_launch_events": round(elapsed_with_events / steps * 1e3, 4)}
        del graphed, replayed

    per_kernel = {}
    for label, by, s, e in launches:
        d = per_kernel.setdefault(label, {"n": 0, "ms": 0.0, "bytes": by})
        d["n"] += 1
        d["ms"] += s.elapsed_time(e)
    return B * steps / elapsed, elapsed / steps * 1e3, per_kernel, out, first_call_ms, graph_info


def kernel_table(per_kernel, steps):
    return {kk: {"avg_ms": round(v["ms"] / v["n"], 4), "launches_per_step": v["n"] / steps,
                 "algorithmic_GB": round(v["bytes"] / 1e9, 3),
                 "alg_GBps": round(v["bytes"] / (v["ms"] / v["n"] * 1e-3) / 1e9, 1)}
            for kk, v in per_kernel.items()}


_TRAFFIC = None


def load_traffic():
    """The committed rocprofv3 --pmc summary of the packed launches, or ({}, note) when it was
    taken from other kernel sources than the ones in the tree."""
    global _TRAFFIC
    if _TRAFFIC is None:
        _TRAFFIC = read_traffic()
    return _TRAFFIC


def read_traffic():
    if not os.path.exists(TRAFFIC_JSON):
        return {}, "no traffic summary committed"
    with open(TRAFFIC_JSON) as f:
        table = json.load(f)
    have, want = table.get("_source_hash"), source_hash()
    if have != want:
        note = ("profiles/packed_kernel_traffic.json was measured on kernel sources %s, the tree has %s: traffic "
                "not reported; re-run the --pmc passes named in profiles/packed_path_hbm_traffic.txt" % (have, want))
        print("bench.py: WARNING: " + note, file=sys.stderr)
        return {}, note
    return table, None


def packed_headline(args, torch, dl):
    F, width, L, k = args.features, args.width, args.layers, 10
    B = 1 << args.batch_log2
    model = packed_model(torch, dl, F, [width] * L, k)
    if args.gate_mix != "uniform":
        apply_gate_mix(torch, dl, model, args.gate_mix)
    x = bernoulli_input(torch, B, F, 1)
    value, ms_per_step, per_kernel, out, first_ms, graph_info = packed_run(torch, dl, model, x, k, args.steps, args.warmup)

    table, note = load_traffic()
    prefix = "" if args.gate_mix == "uniform" else args.gate_mix + ": "
    kernels, roofline = launch_rooflines(per_kernel, args.steps, table, prefix)
    roofline["achieved_is"] = ("measured L2<->fabric bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a plain "
                               "copy) / launch time; reads served by the Infinity Cache are included")
    roofline["launches_timed_in"] = ("a second pass of the same steps with HIP events around every launch; the pass that "
                                     "yields `value` runs without them (timing events drain the queue between kernels)")
    roofline["fully_fused_floor_bytes_per_sample"] = F // 8 + 4 * k
    if note:
        roofline["traffic_note"] = note
    total_alg = sum(v["bytes"] * v["n"] for v in per_kernel.values()) / args.steps
    info = {
        "kernels": kernels,
        "path_algorithmic_GB_per_step": round(total_alg / 1e9, 2),
        "path_alg_GBps": round(total_alg / (ms_per_step * 1e-3) / 1e9, 1),
        "first_call_ms": round(first_ms, 1),
        "hip_graph_replay": graph_info,
        "checksum": int(out.sum().item()),
    }
    if not args.no_configs:
        info["other_word_widths"] = word_width_variants(torch, dl, model, x, out)
        if args.gate_mix == "uniform":
            info["other_gate_mixes"] = gate_mix_variants(torch, dl, model, x, table, not args.no_cpu_baseline)
    return value, ms_per_step, roofline, info, model, x, out


GATE_MIXES = {
    # name: (pool the gate ids are drawn from uniformly, what it stands for)
    "uniform": (list(range(16)), "N(0,1) gate logits: ids uniform over the 16 gates (the BASELINE config)"),
    "two_input_gates_only": ([1, 2, 4, 6, 7, 8, 9, 11, 13, 14],
                             "every gate looks at both of its inputs: nothing for the packed kernels to skip"),
    "half_pass_through": ([3, 5, 10, 12] * 4 + list(range(16)),
                          "half of the ids from {a, b, not a, not b}, the other half uniform over all 16: the "
                          "pass-through-rich end that trained nets are reported to lie towards"),
}


def apply_gate_mix(torch, dl, model, mix, seed=3):
    """Overwrites the gate logits of `model` with one-hot rows whose ids are drawn from GATE_MIXES[mix]."""
    pool = torch.tensor(GATE_MIXES[mix][0], device="cuda")
    g = torch.Generator(device="cuda").manual_seed(seed)
    with torch.no_grad():
        for m in model:
            if isinstance(m, dl.LogicLayer):
                ids = pool[torch.randint(0, len(pool), (m.out_dim,), device="cuda", generator=g)]
                m.weights.copy_(torch.nn.functional.one_hot(ids, 16).float())


def launch_rooflines(per_kernel, steps, table, prefix=""):
    """Per-launch table of a packed run, with the measured traffic of each launch where the committed --pmc summary
    has it (keys of profiles/packed_kernel_traffic.json: `prefix` + the launch label), and the roofline block of
    the launch kind that takes the most time."""
    kernels = kernel_table(per_kernel, steps)
    for label, row in kernels.items():
        e = table.get(prefix + label)
        if e and e.get("hbm_bytes_per_launch"):
            row["traffic_GB"] = round(e["hbm_bytes_per_launch"] / 1e9, 3)
            row["traffic_GBps"] = round(e["hbm_bytes_per_launch"] / (row["avg_ms"] * 1e-3) / 1e9, 1)
            row["frac_hbm_traffic"] = round(row["traffic_GBps"] / HBM_PEAK_GBS, 4)
            row["limited_by"] = e.get("bound")
    dom = max(per_kernel, key=lambda kk: per_kernel[kk]["ms"])
    avg_ms = per_kernel[dom]["ms"] / per_kernel[dom]["n"]
    alg = per_kernel[dom]["bytes"]
    alg_gbps = alg / (avg_ms * 1e-3) / 1e9
    entry = table.get(prefix + dom) or {}
    traffic = entry.get("hbm_bytes_per_launch")
    achieved = traffic / (avg_ms * 1e-3) / 1e9 if traffic else None
    roofline = {
        # `achieved`, `peak` and `frac` are HBM figures; what actually limits the launch is said in words beside them
        "bound": "hbm",
        "limited_by": entry.get("bound", "hbm") if traffic else "hbm (traffic of this build not measured)",
        "kernel": dom,
        "achieved": round(achieved, 1) if achieved else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4) if achieved else None,
        "traffic": traffic,
        "algorithmic_bytes_per_launch": int(alg), "alg_GBps": round(alg_gbps, 1),
        "alg_over_peak": round(alg_gbps / HBM_PEAK_GBS, 4),
        "avg_launch_ms": round(avg_ms, 4), "launches_timed": per_kernel[dom]["n"],
    }
    return kernels, roofline


def gate_mix_variants(torch, dl, model, x, table, check_cpu):
    """The headline net and batch with other gate mixes.  The packed kernels fetch, evaluate and write nothing that
    no gate looks at (six of the sixteen gates ignore an input, constants fold upwards), so the headline, whose gate
    ids are uniform over all sixteen, moves fewer bytes than a net without such gates.  Each variant gets the
    headline's treatment: samples/s, per-launch table with measured traffic, the roofline of its dominant launch,
    and the first 4096 samples of the full-batch result compared with the CPU interpreter."""
    import copy
    res = {}
    for mix in ("two_input_gates_only", "half_pass_through"):
        net = copy.deepcopy(model)
        apply_gate_mix(torch, dl, net, mix)
        value, ms, per_kernel, out, _, _ = packed_run(torch, dl, net, x, 10, steps=5, warmup=2, graph=False)
        kernels, roofline = launch_rooflines(per_kernel, 5, table, prefix=mix + ": ")
        r = {"gate_ids": GATE_MIXES[mix][1], "gate_mix": gate_mix(net_tables(net, dl)), "samples_per_s": round(value, 1),
             "ms_per_step": round(ms, 4), "kernels": kernels, "roofline": roofline, "checksum": int(out.sum().item())}
        if check_cpu:
            from oracle import interp
            n = 4096
            want = interp.net_eval(x[:n].cpu().numpy(), net_tables(net, dl), 10, threads=1)
            r["bit_exact_vs_cpu_interpreter"] = {"samples": n, "equal": bool((out[:n].cpu().numpy() == want).all())}
        res[mix] = r
        del net, out
    return res


def word_width_variants(torch, dl, model, x, want):
    """The same step with PackBitsTensor's other word widths (32 is the reference's default) and with a
    batch that fills neither the last word nor the last 16 bytes of a row: ms per step, and whether the
    counts equal the int64 run's."""
    res = {}
    ragged = x[:x.shape[0] - 37].contiguous()
    for name, inp, bits in (("int32", x, 32), ("int16", x, 16), ("int8", x, 8), ("int32, batch - 37", ragged, 32),
                            ("int64, batch - 37", ragged, 64)):
        def step():
            with torch.no_grad():
                return model(dl.PackBitsTensor(inp, bit_count=bits))
        for _ in range(24):                     # (steps that follow a pause run slower, for some twenty steps)
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            got = step()
        torch.cuda.synchronize()
        res[name] = {"ms_per_step": round((time.perf_counter() - t0) / 10 * 1e3, 4),
                     "equal_to_int64_run": bool(torch.equal(got, want[:inp.shape[0]]))}
    return res


def net_tables(model, dl):
    import numpy as np
    return [(m.indices[0].cpu().numpy(), m.indices[1].cpu().numpy(),
             m.weights.argmax(-1).to("cpu").numpy().astype(np.uint8)) for m in model if isinstance(m, dl.LogicLayer)]


def cpu_interpreter(args, model, x, out, dl):
    """The oracle's table-driven C interpreter (same per-word arithmetic as the C the reference
    generates), one thread, on the first 2^cpu_sample_log2 samples of the batch; the GPU's
    full-batch result is compared with it on those samples."""
    from oracle import interp
    layers = net_tables(model, dl)
    n = min(1 << args.cpu_sample_log2, x.shape[0])
    xs = x[:n].cpu().numpy()
    interp.net_eval(xs[:64], layers, 10)            # load the library, touch the tables
    t0 = time.perf_counter()
    want = interp.net_eval(xs, layers, 10, threads=1)
    dt = time.perf_counter() - t0
    got = out[:n].cpu().numpy()
    return {"value": round(n / dt, 1), "unit": "samples/s", "cores": 1, "kind": "port",
            "sample": "first %d of %d samples, same net; oracle/c/packed_interp.c (table interpreter), 1 thread, %.1f s"
                      % (n, x.shape[0], dt),
            "gpu_matches_cpu_on_sample": bool((got == want).all())}


def cpu_baseline(interpreter, compiled, xs, got, sample_note):
    """`cpu_baseline` of the line: the gcc-compiled generated C where it was started (and built), with the table
    interpreter's figure beside it; else the interpreter."""
    if compiled is None:
        return interpreter
    res = compiled.collect(xs, got, sample_note)
    if "error" in res:
        return dict(interpreter, generated_c_error=res["error"])
    res["table_interpreter"] = {kk: interpreter[kk] for kk in ("value", "unit", "cores", "sample", "gpu_matches_cpu_on_sample")}
    return res


class GeneratedC:
    """The reference's CPU inference path for one net on this host: the C text CompiledLogicNet generates
    (difflogic/compiled_model.py:159-239, restated by oracle/cgen.py), compiled the way the reference's driver does
    (experiments/main.py:362: gcc -O1 below 50 000 gates, else -O0), 64-bit words, one thread.  The constructor
    writes the text and starts gcc as a child process (minutes for 384 000 gates: call it before the GPU is
    initialised, so that the child is started from a process that has not touched it); collect() waits for the
    compiler and times the whole apply_logic_gate_net call (bool packing, gates, adders)."""

    # collect() gives the compiler this long, counted from its start (about 130 s for the headline's 384 000 gates on
    # the GPU box's host); a host that needs longer gets the table interpreter's figure instead of a run without end
    MAX_WAIT_S = 420.0

    def __init__(self, name, layers, num_inputs, k=10):
        import subprocess
        import tempfile
        import threading
        from oracle import cgen
        self.name, self.layers, self.k = name, layers, k
        self.gates = sum(len(l[2]) for l in layers)
        self.opt = 1 if self.gates < 50000 else 0
        self.work = tempfile.mkdtemp(prefix="dl_bench_cgen_")
        self.c_path, self.so_path = os.path.join(self.work, "net.c"), os.path.join(self.work, "net.so")
        with open(self.c_path, "w") as f:
            f.write(cgen.generate_c(layers, num_inputs, k, 64))
        self.t0 = time.perf_counter()
        self.t_end = None
        self.proc = subprocess.Popen(["gcc", "-shared", "-fPIC", "-O%d" % self.opt, "-o", self.so_path, self.c_path])

        def wait():
            self.proc.wait()
            self.t_end = time.perf_counter()
        self._waiter = threading.Thread(target=wait, daemon=True)
        self._waiter.start()

    def same_net(self, tables):
        import numpy as np
        return len(tables) == len(self.layers) and all(
            np.array_equal(u, v) for mine, theirs in zip(self.layers, tables) for u, v in zip(mine, theirs))

    def collect(self, xs, got, sample_note):
        """xs bool [n, F] (numpy): the sample; got int32 [n, k]: what the GPU computed for it."""
        from oracle import cgen
        while self._waiter.is_alive():
            self._waiter.join(timeout=30)
            if self._waiter.is_alive():
                waited = time.perf_counter() - self.t0
                print("bench.py: waiting for gcc -O%d on the %d gates of %s, %.0f s so far"
                      % (self.opt, self.gates, self.name, waited), file=sys.stderr, flush=True)
                if waited > self.MAX_WAIT_S:
                    self.proc.kill()
                    self._waiter.join()
                    return {"error": "gcc -O%d on %d gates not finished after %.0f s: stopped" % (self.opt, self.gates, waited)}
        if self.proc.returncode:
            return {"error": "gcc exited with %d" % self.proc.returncode}
        fn = cgen.load_apply_fn(self.so_path)
        cgen.call_apply_fn(fn, xs[:64], self.k, 64)
        t0 = time.perf_counter()
        want = cgen.call_apply_fn(fn, xs, self.k, 64)
        dt = time.perf_counter() - t0
        n = xs.shape[0]
        return {"value": round(n / dt, 1), "unit": "samples/s", "cores": 1, "kind": "generated-c",
                "gates": self.gates, "compiler": "gcc -shared -fPIC -O%d" % self.opt,
                "compile_s": round(self.t_end - self.t0, 1),
                "sample": "%s; the C text CompiledLogicNet generates for this net (restated by oracle/cgen.py), compiled as "
                          "experiments/main.py:362 does, one apply_logic_gate_net call, 1 thread, %.1f s; gcc ran as a child "
                          "process next to the GPU work" % (sample_note, dt),
                "gpu_matches_cpu_on_sample": bool((got == want).all())}

    def close(self):
        if self._waiter.is_alive():
            self.proc.kill()
            self._waiter.join()
        for path in (self.c_path, self.so_path):
            if os.path.exists(path):
                os.remove(path)
        if os.path.isdir(self.work):
            os.rmdir(self.work)


def packed_config(torch, dl, tag, name, F, widths, B, x, check_cpu, compiled=None):
    """One of the other packed configurations: samples/s, per-launch times, and the first 4096
    samples of the full-batch result compared with the CPU interpreter.  ``compiled``: the GeneratedC of this
    net started by main(), timed on the first 2^16 samples."""
    k = 10
    model = packed_model(torch, dl, F, widths, k)
    value, ms, per_kernel, out, first_ms, graph_info = packed_run(torch, dl, model, x, k, steps=5, warmup=2)
    W = B // 64
    dims = [F] + list(widths)
    alg = sum(eval_layer_bytes(i, o, W) for i, o in zip(dims[:-1], dims[1:])) + 8 * W * dims[-1] + 4 * k * B
    table, _ = load_traffic()
    kernels, roofline = launch_rooflines(per_kernel, 5, table, prefix=tag + ": ")
    res = {"workload": name, "dtype": "int64", "samples_per_s": round(value, 1), "ms_per_step": round(ms, 4),
           "algorithmic_GB_per_step_without_pack": round(alg / 1e9, 2),
           "alg_over_peak": round(alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           "first_call_ms": round(first_ms, 1), "hip_graph_replay": graph_info, "kernels": kernels, "roofline": roofline,
           "checksum": int(out.sum().item())}
    if check_cpu:
        from oracle import interp
        n = 4096
        t0 = time.perf_counter()
        want = interp.net_eval(x[:n].cpu().numpy(), net_tables(model, dl), k, threads=1)
        dt = time.perf_counter() - t0
        res["bit_exact_vs_cpu_interpreter"] = {"samples": n, "equal": bool((out[:n].cpu().numpy() == want).all()),
                                               "cpu_samples_per_s": round(n / dt, 1)}
    res["gate_mix"] = gate_mix(net_tables(model, dl))
    if compiled is not None:
        n = min(1 << 16, B)
        if compiled.same_net(net_tables(model, dl)):
            res["cpu_generated_c"] = compiled.collect(x[:n].cpu().numpy(), out[:n].cpu().numpy(), "first %d samples" % n)
        else:
            res["cpu_generated_c"] = {"error": "the net made on the CPU differs from the model's"}
        compiled.close()
    del model, out
    return res


# ------------------------------------------------------------------------------------------
# fp32 training
# ------------------------------------------------------------------------------------------

def train_alg_bytes(dims, B):
    """forward 4B(in+out)+80 out, backward_w 4B(in+out)+64 out per layer; backward_x 4B(2 in+out)+64 out
    for every layer but the first."""
    alg = sum(4 * B * (i + o) + 80 * o + 4 * B * (i + o) + 64 * o for i, o in zip(dims[:-1], dims[1:]))
    return alg + sum(4 * B * (2 * i + o) + 64 * o for i, o in zip(dims[1:-1], dims[2:]))


def load_train_traffic(config):
    """{variant: measured bytes between the L2s and the fabric per eager forward+backward step} of `config` from the
    committed rocprofv3 --pmc summary, or {} when it was taken from other kernel sources than the ones in the tree."""
    if not os.path.exists(TRAIN_TRAFFIC_JSON):
        return {}
    with open(TRAIN_TRAFFIC_JSON) as f:
        table = json.load(f)
    if table.get("_source_hash") != source_hash(TRAIN_TRAFFIC_SOURCES):
        print("bench.py: WARNING: profiles/train_step_traffic.json was measured on other kernel sources than the tree's: "
              "frac_hbm_traffic not reported", file=sys.stderr)
        return {}
    return table.get(config, {})


def train_config(torch, dl, name, F, widths, k, tau, B, connections, grad_factor, x, steps, warmup, other_dtypes=False,
                 eager_only="", config=""):
    """fp32 training step of one configuration with CrossEntropy: forward+backward and
    forward+backward+Adam(lr 0.01), each eager and replayed as one HIP graph; once for the model as
    the reference's user writes it (torch's fused Adam) and once with the training epilogue of this
    package (last layer fused with GroupSum, difflogic_amd.FusedAdam)."""
    from difflogic_amd.graphs import GraphedTrainStep
    torch.manual_seed(0)
    mods, d = [torch.nn.Flatten()], F
    for w in widths:
        mods.append(dl.LogicLayer(d, w, connections=connections, grad_factor=grad_factor))
        d = w
    model = torch.nn.Sequential(*mods, dl.GroupSum(k, tau)).train()
    g = torch.Generator(device="cuda").manual_seed(2)
    labels = torch.randint(0, k, (B,), device="cuda", generator=g)
    loss_fn = torch.nn.CrossEntropyLoss()
    neuron_samples = sum(widths) * B
    alg = train_alg_bytes([F] + list(widths), B)

    def timeit(fn):
        # untimed: a fifth of a second of the same steps, back to back as the timed ones run, ahead of the warm-up
        # proper (launches that follow an idle GPU run slower for some tens of milliseconds)
        t_settle = time.perf_counter() + SETTLE_S["train"]
        while time.perf_counter() < t_settle:
            for _ in range(8):
                fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            last = fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps, last

    traffic = load_train_traffic(config)

    def report(sec, loss, variant=None):
        r = {"neuron_samples_per_s": round(neuron_samples / sec, 1), "ms_per_step": round(sec * 1e3, 4),
             "alg_GBps": round(alg / sec / 1e9, 1), "frac_hbm_algorithmic": round(alg / sec / 1e9 / HBM_PEAK_GBS, 4),
             "loss": round(float(loss), 6)}
        t = traffic.get(variant)
        if t:
            # measured bytes between the L2 caches and the fabric per step (rocprofv3 FETCH_SIZE + WRITE_SIZE over the
            # same eager loop) over this run's time: the bandwidth; frac_hbm_algorithmic above is a ratio to compare
            # against the per-layer formula, not a bandwidth
            r["traffic_GB_per_step"] = round(t["hbm_bytes_per_step"] / 1e9, 3)
            r["traffic_GBps"] = round(t["hbm_bytes_per_step"] / sec / 1e9, 1)
            r["frac_hbm_traffic"] = round(t["hbm_bytes_per_step"] / sec / 1e9 / HBM_PEAK_GBS, 4)
        return r

    res = {"workload": name, "dtype": "f32", "algorithmic_GB_per_step": round(alg / 1e9, 3)}

    def measure(net, out, make_opt, variant):
        """forward+backward and forward+backward+Adam of `net`, eager and as a replayed HIP graph."""
        def fwd_bwd():
            net.zero_grad(set_to_none=True)
            loss = loss_fn(net(x), labels)
            loss.backward()
            return loss

        sec, loss = timeit(fwd_bwd)
        out["fwd_bwd_eager"] = report(sec, loss.item(), variant)
        if eager_only:
            return
        # Drop every reference to the eager autograd graph before capturing: gradient-accumulation
        # nodes kept alive by `loss` belong to the default stream and would be replayed into the
        # capture stream's backward.
        del loss
        net.zero_grad(set_to_none=True)
        gc.collect()
        torch.cuda.synchronize()
        graphed = GraphedTrainStep(net, loss_fn, x, labels)
        sec, loss = timeit(graphed.step)
        out["fwd_bwd_graph"] = report(sec, loss.item())
        del graphed, loss
        gc.collect()

        # with the optimizer step (experiments/main.py:169,174-181).  The weights move, so the loss differs per step.
        opt = make_opt(net.parameters())

        def full_step():
            opt.zero_grad(set_to_none=True)
            loss = loss_fn(net(x), labels)
            loss.backward()
            opt.step()
            return loss

        sec, loss = timeit(full_step)
        out["fwd_bwd_adam_eager"] = report(sec, loss.item())
        del loss
        opt.zero_grad(set_to_none=True)
        gc.collect()
        torch.cuda.synchronize()
        graphed = GraphedTrainStep(net, loss_fn, x, labels, optimizer=opt)
        sec, loss = timeit(graphed.step)
        out["fwd_bwd_adam_graph"] = report(sec, loss.item())
        del graphed, loss, opt
        gc.collect()

    # the model as a user of the reference writes it, then with the last LogicLayer and GroupSum merged
    # and the first two layers merged (difflogic_amd.fuse_for_training: same parameters; the Adam steps above moved
    # them, so the losses differ)
    if eager_only != "fused":
        measure(model, res, lambda ps: torch.optim.Adam(ps, lr=0.01, fused=True, capturable=True), "written")
        res["optimizer"] = "torch.optim.Adam(fused=True, capturable=True)"
    if eager_only != "written":
        res["fused_for_training"] = {"optimizer": "difflogic_amd.FusedAdam (one launch over all weight tensors)"}
        measure(dl.fuse_for_training(model).train(), res["fused_for_training"], lambda ps: dl.FusedAdam(ps, lr=0.01), "fused")

    if other_dtypes and not eager_only:
        # experiments/main.py:19-23,286 (--training-bit-count 16 / 64): the input is cast, the weights stay fp32
        res["other_input_dtypes"] = {}
        for key, dtype, size in (("f16", torch.float16, 2), ("f64", torch.float64, 8)):
            xd = x.to(dtype)

            def fwd_bwd():
                model.zero_grad(set_to_none=True)
                loss = loss_fn(model(xd), labels)
                loss.backward()
                return loss

            def report_dtype(sec, loss):
                r = report(sec, loss)
                r["alg_GBps"] = round(r["alg_GBps"] * size / 4, 1)
                r["frac_hbm_algorithmic"] = round(r["frac_hbm_algorithmic"] * size / 4, 4)
                return r

            out = res["other_input_dtypes"][key] = {}
            sec, loss = timeit(fwd_bwd)
            out["fwd_bwd_eager"] = report_dtype(sec, loss.item())
            del loss
            # the fuse_for_training model: its layers and the GroupSum as one autograd node (less host work per step)
            fused_model = dl.fuse_for_training(model).train()

            def fwd_bwd_fused():
                fused_model.zero_grad(set_to_none=True)
                loss = loss_fn(fused_model(xd), labels)
                loss.backward()
                return loss

            sec, loss = timeit(fwd_bwd_fused)
            out["fused_for_training_fwd_bwd_eager"] = report_dtype(sec, loss.item())
            del loss, fused_model
            model.zero_grad(set_to_none=True)
            gc.collect()
            torch.cuda.synchronize()
            graphed = GraphedTrainStep(model, loss_fn, xd, labels)
            sec, loss = timeit(graphed.step)
            out["fwd_bwd_graph"] = report_dtype(sec, loss.item())
            del graphed, loss, xd
            gc.collect()
    return res, model


def train_kernels_alone(torch, dl, model, B, width):
    """Each layer kernel timed alone (back-to-back launches on a 64000 -> 64000 layer, forward and
    backward_w in their chained form; backward_chained is the single pass the layer runs in place
    of backward_w + backward_x and is charged the bytes of both) against its algorithmic bytes."""
    ext = dl.difflogic_cuda
    g = torch.Generator(device="cuda").manual_seed(3)
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
        kernels[name] = {"us_per_launch": round(us, 2), "alg_GBps": round(by / (us * 1e-6) / 1e9, 1),
                         "frac_hbm_algorithmic": round(by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
    return kernels


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


# ------------------------------------------------------------------------------------------
# practical ceilings
# ------------------------------------------------------------------------------------------

def ceilings(torch):
    """Streaming read / write / copy over 8 GiB buffers and row gathers with the gate kernels'
    access pattern (64 lanes x 16 bytes per gathered row, column-tile-major dispatch) from an
    input that stays L2-resident per column tile (784 rows) and from one that does not (64000
    rows, served by the fabric / Infinity Cache).  GB/s, best of the grid sizes tried."""
    from difflogic_amd import build
    lib = ctypes.CDLL(build.CEILINGS_LIB_PATH)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.dlc_stream.argtypes = [i32, vp, vp, i64, i32, vp]
    lib.dlc_gather.argtypes = [vp, vp, i64, i64, i32, vp, vp]
    stream = vp(torch.cuda.current_stream().cuda_stream)

    def timed(fn, iters):
        for _ in range(2):
            fn()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(iters):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / iters * 1e-3

    nbytes = 8 << 30                            # also holds the 64000 x 128 KB matrix of the gather test
    a = torch.empty(nbytes, dtype=torch.uint8, device="cuda").fill_(1)
    b = torch.empty(nbytes, dtype=torch.uint8, device="cuda").fill_(2)
    res = {"buffer_GiB": nbytes >> 30}
    for mode, key, moved in ((0, "stream_read", nbytes), (1, "stream_write", nbytes), (2, "stream_copy", 2 * nbytes)):
        best = {}
        for grid in (2048, 8192, 32768):
            def fn():
                st = lib.dlc_stream(mode, vp(a.data_ptr()), vp(b.data_ptr()), nbytes, grid, stream)
                assert st == 0, st
            best[grid] = round(moved / timed(fn, 5) / 1e9, 1)
        res[key + "_GBps"] = max(best.values())
        res[key + "_by_grid"] = best
    t = timed(lambda: b[:1 << 30].copy_(a[:1 << 30]), 5)
    res["runtime_copy_1GiB_GBps"] = round(2 * (1 << 30) / t / 1e9, 1)
    del b

    W = 16384                                   # row = 128 KB, as in the headline workload
    out_rows = 64000
    g = torch.Generator(device="cuda").manual_seed(0)
    sink = torch.zeros(16, dtype=torch.uint8, device="cuda")
    for rows, key in ((784, "gather_l2_resident_784_rows"), (64000, "gather_fabric_64000_rows")):
        assert rows * W * 8 <= a.numel(), "the gathered matrix must fit the buffer"
        x = a[:rows * W * 8]
        for gathers in (2, 4, 8):
            if rows == 64000 and gathers == 8:
                continue
            idx = torch.randint(0, rows, (out_rows * gathers,), device="cuda", generator=g, dtype=torch.int32)
            assert 0 <= int(idx.min()) and int(idx.max()) < rows and x.numel() == rows * W * 8

            def fn():
                st = lib.dlc_gather(vp(x.data_ptr()), vp(idx.data_ptr()), out_rows, W * 8, gathers, vp(sink.data_ptr()), stream)
                assert st == 0, st
            sec = timed(fn, 3)
            res["%s_x%d_GBps" % (key, gathers)] = round(out_rows * gathers * W * 8 / sec / 1e9, 1)
    return res


def wanted(args, c, group_off):
    only = {c for c in args.only.lower().split(",") if c}
    return (c in only) if only else not group_off


def extra_configs(args, torch, dl, started):
    """The other BASELINE configurations (C1 .. C5), each optional.  ``started``: GeneratedC objects by name."""
    want = lambda c, group_off: wanted(args, c, group_off)      # noqa: E731
    configs = {}
    check = not args.no_cpu_baseline
    if want("c2", args.no_configs):
        B = 1 << 20
        configs["C2"] = packed_config(torch, dl, "C2", "packed inference 784->6x8000->GroupSum(10), batch 2^20, int64 words",
                                      784, [8000] * 6, B, bernoulli_input(torch, B, 784, 1), check,
                                      compiled=started.get("C2"))
        torch.cuda.empty_cache()
    if want("c4", args.no_configs):
        B = 1 << 18
        configs["C4"] = packed_config(torch, dl, "C4", "packed inference 9216->4x256000->GroupSum(10), batch 2^18, int64 words, "
                                      "thresholded-uniform input", 9216, [256000] * 4, B, thresholded_input(torch, B, 1),
                                      check)
        torch.cuda.empty_cache()
    steps, warmup = max(5, args.steps), max(3, args.warmup)
    if want("c3", args.no_train):
        B = 512
        x = bernoulli_input(torch, B, 784, 2).float()
        configs["C3"], model = train_config(
            torch, dl, "fp32 train 784->6x64000->GroupSum(10,tau=30), B=512, connections=unique, CrossEntropy",
            784, [64000] * 6, 10, 30.0, B, "unique", 1.0, x, steps, warmup, other_dtypes=True,
            eager_only=args.train_eager_only, config="C3")
        if not args.train_eager_only:
            configs["C3"]["kernels_alone_64000x64000"] = train_kernels_alone(torch, dl, model, B, 64000)
        del model, x
        gc.collect()
        torch.cuda.empty_cache()
    if want("c5", args.no_train):
        B = 1024
        x = thresholded_input(torch, B, 2, as_float=True)
        configs["C5"], model = train_config(
            torch, dl, "fp32 train 9216->12x128000->GroupSum(10,tau=100), B=1024, connections=random, grad_factor=2, "
            "thresholded-uniform input, CrossEntropy", 9216, [128000] * 12, 10, 100.0, B, "random", 2.0, x, steps, warmup,
            eager_only=args.train_eager_only, config="C5")
        del model, x
        gc.collect()
        torch.cuda.empty_cache()
    if want("c1", args.no_train):
        B = 128
        x = bernoulli_input(torch, B, 784, 2).float()
        configs["C1"], model = train_config(
            torch, dl, "fp32 train 784->4x8000->GroupSum(10,tau=10), B=128, connections=random, CrossEntropy",
            784, [8000] * 4, 10, 10.0, B, "random", 1.0, x, max(steps, 50), warmup, eager_only=args.train_eager_only,
            config="C1")
        del model, x
        if not args.no_cpu_baseline:
            configs["C1"]["cpu_baseline"] = train_cpu_baseline(torch)
    return configs


def main():
    args = parse()
    if args.no_settle:
        SETTLE_S.update(packed=0.0, train=0.0)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path shards along the batch without "
              "communication); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch                      # (importing it does not initialise the GPU)

    # The reference's CPU inference path (gcc on the generated C) takes minutes to compile: started here, as child
    # processes of a process that has not touched the GPU yet, and collected after the GPU work.
    started = {}
    if not (args.no_cpu_baseline or args.no_cpu_generated_c or args.ceilings):
        if not args.skip_headline and args.gate_mix == "uniform":
            started["headline"] = GeneratedC("the headline net", cpu_side_net(torch, args.features, [args.width] * args.layers),
                                             args.features)
        if wanted(args, "c2", args.no_configs):
            started["C2"] = GeneratedC("C2", cpu_side_net(torch, 784, [8000] * 6), 784)
    try:
        run(args, torch, started)
    finally:
        for c in started.values():
            c.close()


def run(args, torch, started):
    import difflogic_amd as dl
    assert torch.cuda.is_available(), "bench.py needs the GPU"

    if args.ceilings:
        print(json.dumps({"metric": "practical ceilings on this GPU", "unit": "GB/s", "hbm_peak_GBps": HBM_PEAK_GBS,
                          "device": torch.cuda.get_device_name(0), **ceilings(torch)}))
        return

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.skip_headline:
        print(json.dumps({"metric": "extra configurations only (--skip-headline)",
                          "extra": {"configs": extra_configs(args, torch, dl, started)}}))
        return
    value, ms, roofline, info, model, x, out = packed_headline(args, torch, dl)
    result = {
        "metric": "packed-eval samples/s (784->6x64k)", "value": round(value, 1), "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int64", "data": "synthetic",
        "config": {"workload": "packed inference %d->%dx%d->GroupSum(10), batch 2^%d, int64 words, bool input "
                               "resident in HBM; step = pack + %d gate layers + groupbitsum"
                               % (args.features, args.layers, args.width, args.batch_log2, args.layers),
                   "connections": "random", "seed": 0, "gate_ids": GATE_MIXES[args.gate_mix][1],
                   "gate_mix": gate_mix(net_tables(model, dl))},
        "roofline": roofline,
    }
    interpreter, compiled, sample = None, None, None
    if not args.no_cpu_baseline:
        interpreter = cpu_interpreter(args, model, x, out, dl)
        compiled = started.get("headline")
        if compiled is not None and not compiled.same_net(net_tables(model, dl)):
            interpreter["generated_c_error"] = "the net made on the CPU differs from the model's"
            compiled = None
        n = min(1 << args.cpu_generated_c_sample_log2, x.shape[0])
        sample = (x[:n].cpu().numpy(), out[:n].cpu().numpy(), "first %d of %d samples, same net" % (n, x.shape[0]))
    extra = dict(info)
    del model, x, out
    gc.collect()
    torch.cuda.empty_cache()

    extra["configs"] = extra_configs(args, torch, dl, started)
    # last, so that gcc's minutes on the headline net's C overlap with everything above
    result["cpu_baseline"] = None if interpreter is None else cpu_baseline(interpreter, compiled, *sample)
    result["extra"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
