#!/usr/bin/env python3
"""Benchmark of the tiled-dataflow hot path on one MI355X.

A step is one inference pass over one resident batch in the reference's own loop
(reference main.c:116-123): rpool_reset_queue -> rpool_reset_nasm -> dse_group_run ->
dse_wait_for_nasm_completion -> dse_group_stop.  Inputs and weights are in HBM before the timed
region starts.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50_b32] [--mode dataflow|layers]
"""
import argparse
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3      # MI355X dense fp32 matrix peak
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the persistent kernel, measured with rocprofv3 FETCH_SIZE / WRITE_SIZE passes
# calibrated on the library's copy kernel (summaries: profiles/dataflow_kernel_resnet50_b32_hbm_traffic.txt and
# profiles/dataflow_kernel_vgg16_co_inference_bert_gpt2_kernel_stats_hbm_traffic.txt); valid for these tuned configurations only
MEASURED_TRAFFIC_BYTES = {("resnet50_b32", "dataflow", 1536): 8.68e9, ("vgg16_b32", "dataflow", 1536): 17.36e9,
                          ("co_resnet50_vgg16_b16", "dataflow", 1536): 15.00e9, ("bert_base_b8_s128", "dataflow", 192): 2.89e9,
                          ("gpt2_b4_s512", "dataflow", 384): 8.77e9, ("resnet50_b1", "dataflow", 256): 0.414e9}

# algorithmic GEMM-class flops per unit (2*M*N*K with the reference's K: padding taps counted, full
# S x S attention): per image for the vision nets, per token for the transformers
FLOP_PER_UNIT = {
    "resnet50": 8.178369e9, "vgg16": 3.069326e10 + 2.47267e8,
    "bert_base": 1.7459e8, "gpt2": 1.8877e8,
}
from aspen_amd.models import WORKLOADS      # noqa: E402  (shared with the full-size parity tests)


def gemm_flops(nasm, api):
    total = 0
    for l in range(nasm.num_ldata):
        i = nasm.info(l)
        if i["type"] in (api.CONV_LAYER, api.FC_LAYER, api.MATMUL_LAYER, api.K_ATTENTION_LAYER, api.V_ATTENTION_LAYER):
            total += i["flops"]
    return total


def compulsory_bytes(nasm, api):
    """What one inference must move if every matrix is read once by each layer that consumes it and written once, and
    every weight matrix is read once: the yardstick for the measured traffic (which adds re-reads by several XCDs,
    window overlaps that have left the caches, and split-K partial sums).  Follows the graph as built: a matrix that
    is never written (the pre-shortcut sums of a fused shortcut, the probabilities of a fused attention) counts
    neither as output nor as input."""
    infos = [nasm.info(l) for l in range(nasm.num_ldata)]
    size = lambda i: 4 * i["H"] * i["W"]
    contraction = (api.CONV_LAYER, api.FC_LAYER, api.MATMUL_LAYER)
    total = 0
    for i in infos:
        t = i["type"]
        if t == api.INPUT_LAYER:
            continue
        no_tiles = i["num_ninst"] == 0
        if t == api.K_ATTENTION_LAYER and no_tiles:
            continue                                    # fused into the V-attention tiles: nothing written, nothing read here
        if not i.get("discarded"):
            total += size(i)
        parents = [infos[p] for p in (i["p0"], i["p1"]) if 0 <= p < len(infos)]
        if t == api.RESIDUAL_LAYER and no_tiles:
            parents = parents[1:]                       # computed in its producer's epilogue: only the other operand is read
        if t == api.V_ATTENTION_LAYER and parents and parents[0]["type"] == api.K_ATTENTION_LAYER and parents[0]["num_ninst"] == 0:
            k = parents[0]
            parents = [infos[p] for p in (k["p0"], k["p1"]) if 0 <= p < len(infos)] + parents[1:]     # Query, Key, Value
        total += sum(size(p) for p in parents)
        if t in contraction and i["flops"]:
            total += 4 * i["flops"] // (2 * i["W"])     # rows x K weights
    return total


def cpu_baseline(cfgname, budget_s=20.0):
    """Reference tile kernels (oracle/_ref, compiled from the reference's sources) timed on this host's
    cores; falls back to the oracle port when that library is absent.  Bounded sample of the workload."""
    from aspen_amd import models as M
    gen, style, batch, seq, seed, kind = M.CONFIGS[cfgname]
    threads = min(16, os.cpu_count() or 1)
    os.environ.setdefault("OMP_NUM_THREADS", str(threads))
    cfg = gen()
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, seed, style)
    x = M.synth_input(layers, seed, batch, seq, kind or "token_ids")
    units = batch * (seq if seq else 1)
    unit = "tokens/s" if seq else "img/s"
    try:
        from oracle import ref
        if not ref.available():
            raise OSError("oracle/_ref not built")
        wp = tempfile.mktemp(suffix=".bin")
        M.write_aspen_data(wp, tens)
        net = ref.RefNet(cfg, wp, batch, seq, threads=threads)
        os.unlink(wp)
        net.set_input(x)
        t0 = time.time()
        net.forward()                         # warm-up, also gives the per-pass cost
        one = time.time() - t0
        iters = int(max(1, min(10, budget_s / max(one, 1e-3))))
        sec = net.time_forward(iters)
        net.close()
        flops = FLOP_PER_UNIT.get(cfgname.split("_b")[0], 0.0) * units
        return {"value": units / sec, "unit": unit, "cores": threads, "kind": "reference",
                "scheduler": "reference kernels, layer-synchronous: the reference's tiled_* functions swept layer by layer "
                             "under an OpenMP parallel-for (a barrier per layer), NOT its DSE scheduler",
                "sample": f"{cfgname}: {iters} full passes after 1 warm-up, reference tiled_* kernels swept layer by "
                          f"layer with {threads} OpenMP threads (tile dependency discovery skipped)",
                "ms_per_step": sec * 1e3, "gflops": flops / sec / 1e9}
    except (OSError, RuntimeError) as exc:
        from oracle import cpu
        t0 = time.time()
        cpu.run_network(layers, tens, x, batch, seq, keep_all=False)
        sec = time.time() - t0
        return {"value": units / sec, "unit": unit, "cores": threads, "kind": "port",
                "sample": f"{cfgname}: 1 full pass of the oracle port ({exc})", "ms_per_step": sec * 1e3}


def cpu_baseline_dse(cfgname, min_ninst=100, iters=20):
    """The reference's own scheduler on this host's cores: apu_create_nasm (full tile-dependency search, affordable at
    batch 1) and the run loop of its main.c (reference main.c:105-123: rpool_reset_queue / rpool_reset_nasm /
    dse_group_run / dse_wait_for_nasm_completion / dse_group_stop) with one DSE thread per physical core, through
    oracle/_ref.  None where that library is absent."""
    from aspen_amd import models as M
    try:
        from oracle import ref
        if not ref.available():
            return None
        gen, style, batch, seq, seed, kind = M.CONFIGS[cfgname]
        cfg = gen()
        layers = M.parse_cfg(cfg)
        tens = M.synth_weights(layers, seed, style)
        x = M.synth_input(layers, seed, batch, seq, kind or "token_ids")
        cores = cpu_description()["physical_cores"] or min(16, os.cpu_count() or 1)
        cores = min(cores, 16)                 # the box's CPU share
        wp = tempfile.mktemp(suffix=".bin")
        M.write_aspen_data(wp, tens)
        net = ref.RefNet(cfg, wp, batch, seq, threads=1)
        os.unlink(wp)
        t0 = time.time()
        sec, out = net.time_dse(x, batch, seq, min_ninst, cores, 3, iters)
        wall = time.time() - t0
        net.close()
        units = batch * (seq if seq else 1)
        flops = FLOP_PER_UNIT.get(cfgname.split("_b")[0], 0.0) * units
        return {"value": units / sec, "unit": "tokens/s" if seq else "img/s", "cores": cores, "kind": "reference",
                "scheduler": "the reference's own: apu_create_nasm graph, dse_group_run loop of its main.c, one DSE thread per core",
                "sample": f"{cfgname}: {iters} inferences after 3 warm-up runs; graph built with the reference's dependency search "
                          f"(min_ninst_per_ldata {min_ninst}); {wall:.1f} s including the graph build",
                "ms_per_step": sec * 1e3, "gflops": flops / sec / 1e9}
    except (OSError, RuntimeError) as exc:
        return {"error": str(exc)}


def verify_final_layer(name, nasm):
    """Final layer of the graph that was just timed against the fixture the compiled reference wrote for this
    configuration (tests/golden/<name>.npz: strided samples, norm and per-column argmax).  Returns None when
    no fixture exists for the configuration."""
    path = os.path.join(ROOT, "tests", "golden", f"{name}.npz")
    if not os.path.exists(path):
        return None
    gold = np.load(path)
    l = int(gold["num_layers"]) - 1
    got = nasm.layer_output(l)
    flat = got.reshape(-1).astype(np.float64)
    ref_val = gold[f"val{l}"].astype(np.float64)
    err = float(np.linalg.norm(flat[gold[f"idx{l}"]] - ref_val) / max(np.linalg.norm(ref_val), 1e-30))
    norm = float(np.sqrt((flat ** 2).sum()))
    ref_norm = float(gold[f"l2_{l}"])
    ok = err <= 1e-4 and abs(norm - ref_norm) <= 1e-4 * ref_norm and bool((got.argmax(axis=1) == gold["argmax"]).all())
    return {"ok": ok, "sampled_rel_l2": err, "argmax_equal": bool((got.argmax(axis=1) == gold["argmax"]).all())}


def cpu_description():
    """CPU model, physical cores and hardware threads of this host (from /proc/cpuinfo)."""
    model, phys, threads = "unknown", set(), 0
    try:
        pid = cid = None
        for line in open("/proc/cpuinfo"):
            k, _, v = line.partition(":")
            k, v = k.strip(), v.strip()
            if k == "model name":
                model = v
            elif k == "physical id":
                pid = v
            elif k == "core id":
                cid = v
            elif k == "processor":
                threads += 1
            elif not k and pid is not None:
                phys.add((pid, cid)); pid = cid = None
        if pid is not None:
            phys.add((pid, cid))
    except OSError:
        pass
    return {"model": model, "physical_cores": len(phys) or None, "hardware_threads": threads or (os.cpu_count() or 0)}


def measure_workload(api, M, name, steps, warmup, flags=0):
    """One of the other benchmark configurations, in the same loop as the headline one: its tuned tile count and
    engine (models.WORKLOADS), inputs resident, `warmup` untimed + `steps` timed steps (more of both for steps of
    under a millisecond, so that the timed region is tens of milliseconds long), final layer checked against the
    compiled reference's fixture afterwards.  `flags`: engine flags for this workload's runs.  Everything is torn down
    again."""
    L = api.lib()
    L.aspen_hip_set_flags(flags)
    cfgs, unit, units_per_step, min_ninst, engine = WORKLOADS[name]
    pool = api.RPool()
    dse = api.DseGroup(1, api.MODE_DATAFLOW if engine.startswith("dataflow") else api.MODE_LAYERS)
    dse.set_rpool(pool)
    nets = []
    for cname in cfgs:
        cfg, layers, tens, x, batch, seq = M.make_config(cname)
        wp = tempfile.mktemp(suffix=".bin")
        M.write_aspen_data(wp, tens)
        dnn = api.Dnn(cfg, wp)
        os.unlink(wp)
        del tens
        nasm = api.Nasm(dnn, batch, seq, min_ninst)
        if engine == "dataflow-ordered":
            nasm.set_ordered(1)
        pool.add_nasm_raw_input(nasm, x)
        nets.append((cname, dnn, nasm))
    flops = sum(gemm_flops(n, api) for _, _, n in nets)

    done_ms = [0.0] * len(nets)          # per nasm: when its own wait returned, from the start of the run

    def one(first=False, timed=False):
        if not first:
            pool.reset_queue()
            for _, _, n in nets:
                pool.reset_nasm(n)
        t_run = time.perf_counter()
        dse.run()
        for i, (_, _, n) in enumerate(nets):
            dse.wait(n)                   # returns when THIS nasm's last tile has finished, whatever the others do
            if timed:
                done_ms[i] += (time.perf_counter() - t_run) * 1e3
        dse.stop()

    one(first=True)
    L.aspen_hip_sync()
    t0 = time.perf_counter()
    for _ in range(warmup):
        one()
    L.aspen_hip_sync()
    estimate_ms = (time.perf_counter() - t0) / max(warmup, 1) * 1e3
    if warmup and estimate_ms < 2.0:
        # a step of a few hundred microseconds: the clock settles over many of them, and 20 would be a 10 ms sample
        steps = max(steps, min(200, int(60.0 / estimate_ms)))
        for _ in range(steps // 4):
            one()
        L.aspen_hip_sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        one(timed=True)
    L.aspen_hip_sync()
    ms = (time.perf_counter() - t0) / steps * 1e3
    weight_stream = None
    if name == "vgg16_b32":
        # the layer that streams the most weights past the fewest columns (FC1 of VGG-16: 411 MB of weights, 32 columns),
        # launched alone five times: a memory-bound contraction, priced against the memory roofline
        nasm = nets[0][2]
        lms = pool.profile_layers(nasm.num_ldata, 5)
        infos = [nasm.info(l) for l in range(nasm.num_ldata)]
        fc = [l for l, i in enumerate(infos) if api.LAYER_TYPE_NAMES[i["type"]] == "fc"]
        if fc:
            l = max(fc, key=lambda l: infos[l]["flops"])
            i = infos[l]
            wbytes = i["flops"] / (2 * i["W"]) * 4          # rows x K floats
            gbs = wbytes / (float(lms[l]) * 1e-3) / 1e9
            weight_stream = {"layer": l, "rows": i["H"], "columns": i["W"], "tile": [i["tile_H"], i["tile_W"]], "tiles": i["num_ninst"],
                             "weight_bytes": wbytes, "us": float(lms[l]) * 1e3,
                             "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS}}
    checks = [verify_final_layer(cname, n) for cname, _, n in nets]
    have = [c for c in checks if c is not None]
    ach = flops / (ms * 1e-3) / 1e12
    traffic = MEASURED_TRAFFIC_BYTES.get((name, engine, min_ninst))
    compulsory = sum(compulsory_bytes(n, api) for _, _, n in nets)
    out = {"ms_per_step": ms, "value": units_per_step / (ms * 1e-3), "unit": unit, "engine": engine, "min_ninst_per_ldata": min_ninst,
           "traffic": traffic, "compulsory_bytes": compulsory, "traffic_over_compulsory": traffic / compulsory if traffic else None,
           "tiles_per_step": sum(n.num_ninst for _, _, n in nets), "flops_per_step": flops,
           "frac_of_fp32_mfma_peak": ach / PEAK_FP32_MFMA_TFLOPS, "verified": all(c["ok"] for c in have) if have else None}
    if engine.startswith("dataflow") and dse.last_run_ordered():
        out["engine"] = "dataflow-ordered"
    out["steps"] = steps
    if weight_stream:
        out["weight_streaming_layer"] = weight_stream
    if len(nets) > 1:
        out["nasm_completion_ms"] = {cname: done_ms[i] / steps for i, (cname, _, _) in enumerate(nets)}
    L.aspen_hip_set_flags(0)
    dse.destroy()
    for _, _, n in nets:
        n.destroy()
    pool.destroy()
    for _, d, _ in nets:
        d.destroy()
    return out


def quiet_stdout():
    """The C library reports what it parses on stdout, as the reference does.  The benchmark's stdout
    carries exactly one JSON line, so everything else written to file descriptor 1 goes to stderr; returns
    the function that writes the final line to the real stdout."""
    sys.stdout.flush()
    real = os.dup(1)
    os.dup2(2, 1)

    def emit(line: str) -> None:
        sys.stdout.flush()
        os.write(real, (line + "\n").encode())

    return emit


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="resnet50_b32", choices=list(WORKLOADS))
    ap.add_argument("--mode", default="auto", choices=["auto", "dataflow", "layers"],
                    help="auto: the engine the timing tuner picks for the workload (the persistent dataflow kernel except at batch 1)")
    ap.add_argument("--min-ninst", type=int, default=0, help="tiles wanted per layer (0: the workload's tuned value)")
    ap.add_argument("--workgroups", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-baseline-dse", default="", metavar="CONFIG",
                    help="also time the reference's own scheduler (apu_create_nasm + dse_group_run, through oracle/_ref) on this configuration; "
                         "its dependency search takes minutes beyond batch 1 (bert_base_b8_s128: about 2.5 minutes), so it is not part of the default run")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the `workloads` section (the other benchmark configurations, measured after the headline one)")
    ap.add_argument("--skip-tiles", action="store_true", help="scheduler-only run: dependency protocol with empty tiles")
    ap.add_argument("--no-handoff", action="store_true", help="every ready tile goes through the queue (no parent -> child hand-off)")
    ap.add_argument("--xcd-queues", action="store_true", help="one ready queue per XCD, tiles at home on a fixed eighth of the columns (less memory traffic, less balance)")
    ap.add_argument("--engine-profile", action="store_true", help="report where the persistent workgroups spend their time")
    ap.add_argument("--trace", default="", metavar="NPZ", help="write per-tile start/end stamps of the last timed step (dataflow mode)")
    ap.add_argument("--layer-profile", action="store_true", help="also time every layer's kernel (layer-launch mode)")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="instead of a workload: run the library's streaming copy kernel over MIB MiB (--steps launches); "
                         "under a profiler this calibrates the HBM byte counters")
    args = ap.parse_args()
    emit = quiet_stdout()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)

    from aspen_amd import api, models as M
    L = api.lib()
    if L.aspen_hip_init() != 0:
        print("bench.py: no HIP device: " + L.aspen_hip_last_error().decode(), file=sys.stderr)
        sys.exit(1)
    dev = api.device_info()
    if args.copy_probe:
        nbytes = args.copy_probe << 20
        src, dst = L.aspen_hip_alloc(nbytes), L.aspen_hip_alloc(nbytes)
        for _ in range(args.warmup):
            L.aspen_hip_copy(dst, src, nbytes)
        L.aspen_hip_event_record(0)
        for _ in range(args.steps):
            L.aspen_hip_copy(dst, src, nbytes)
        L.aspen_hip_event_record(1)
        L.aspen_hip_sync()
        ms = api.C.c_float()
        L.aspen_hip_event_elapsed_ms(0, 1, api.C.byref(ms))
        emit(json.dumps({"copy_probe_bytes_read": nbytes, "copy_probe_bytes_written": nbytes, "launches": args.steps,
                          "ms_per_launch": ms.value / args.steps,
                          "GB_per_s": 2 * nbytes * args.steps / (ms.value * 1e-3) / 1e9}))
        return
    L.aspen_hip_set_flags((1 if args.skip_tiles else 0) | (4 if args.engine_profile else 0) | (8 if args.trace else 0) | (16 if args.no_handoff else 0) | (32 if args.xcd_queues else 0))
    cfgs, unit, units_per_step, tuned_min_ninst, tuned_engine = WORKLOADS[args.workload]
    if args.min_ninst <= 0:
        args.min_ninst = tuned_min_ninst
    ask_ordered = False
    if args.mode == "auto":
        args.mode, ask_ordered = tuned_engine.split("-")[0], tuned_engine == "dataflow-ordered"

    pool = api.RPool()
    dse = api.DseGroup(1, {"auto": api.MODE_AUTO, "dataflow": api.MODE_DATAFLOW, "layers": api.MODE_LAYERS}[args.mode], args.workgroups)
    dse.set_rpool(pool)
    nets = []
    for name in cfgs:
        cfg, layers, tens, x, batch, seq = M.make_config(name)
        wp = tempfile.mktemp(suffix=".bin")
        M.write_aspen_data(wp, tens)
        dnn = api.Dnn(cfg, wp)
        os.unlink(wp)
        del tens
        nasm = api.Nasm(dnn, batch, seq, args.min_ninst)
        if ask_ordered:
            nasm.set_ordered(1)
        pool.add_nasm_raw_input(nasm, x)
        nets.append((name, dnn, nasm, layers))
    flops = sum(gemm_flops(n, api) for _, _, n, _ in nets)
    tiles = sum(n.num_ninst for _, _, n, _ in nets)

    def step():
        pool.reset_queue()
        for _, _, n, _ in nets:
            pool.reset_nasm(n)
        dse.run()
        for _, _, n, _ in nets:
            dse.wait(n)
        dse.stop()

    # first run happens with the freshly added input (no reset), then warm-up
    dse.run()
    for _, _, n, _ in nets:
        dse.wait(n)
    dse.stop()
    # what "auto" resolved to for this graph
    args.mode = "dataflow" if dse.last_mode() == api.MODE_DATAFLOW else "layers"
    ordered = dse.last_run_ordered()
    for _ in range(args.warmup):
        step()
    L.aspen_hip_sync()
    if args.engine_profile and args.mode == "dataflow":
        pool.dataflow_profile(reset=True)
    kernel_ms = []
    ms = api.C.c_float()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
        if args.mode == "dataflow" and L.aspen_hip_event_elapsed_ms(14, 15, api.C.byref(ms)) == 0:
            kernel_ms.append(ms.value)
    L.aspen_hip_sync()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = units_per_step * args.steps / dt

    out = {
        "metric": "ResNet-50 fp32 img/s at batch 1/32 on 1 MI355X; conv-tile MFMA util vs FP32 peak",
        "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "engine": args.mode + ("-ordered" if ordered else ""), "tiles_per_step": tiles,
                   "min_ninst_per_ldata": args.min_ninst, "device": dev["name"], "compute_units": dev["compute_units"]},
    }
    if args.mode == "dataflow" and kernel_ms:
        k_ms = float(np.mean(kernel_ms))
        ach = flops / (k_ms * 1e-3) / 1e12
        out["roofline"] = {"bound": "mfma", "kernel": "dataflow_kernel", "achieved": ach, "peak": PEAK_FP32_MFMA_TFLOPS,
                           "unit": "TFLOP/s", "frac": ach / PEAK_FP32_MFMA_TFLOPS,
                           "traffic": MEASURED_TRAFFIC_BYTES.get((args.workload, args.mode, args.min_ninst)),
                           "flops_per_launch": flops, "kernel_ms": k_ms}
        out["roofline"]["compulsory_bytes"] = sum(compulsory_bytes(n, api) for _, _, n, _ in nets)
        if out["roofline"]["traffic"]:
            out["roofline"]["traffic_over_compulsory"] = out["roofline"]["traffic"] / out["roofline"]["compulsory_bytes"]
    else:
        ach = flops / (ms_per_step * 1e-3) / 1e12
        out["roofline"] = {"bound": "mfma", "kernel": "layer_kernel (all layers of one step)", "achieved": ach,
                           "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": ach / PEAK_FP32_MFMA_TFLOPS,
                           "traffic": None, "flops_per_launch": flops, "kernel_ms": ms_per_step}

    # the same step with the host boundary inside: input upload before, logits download after
    # (PCIe-inclusive rate; reported beside `value`, never as `value`)
    if not args.skip_tiles:
        xs = [M.make_config(name)[3] for name in cfgs]
        t0 = time.perf_counter()
        io_steps = max(1, min(5, args.steps))
        for _ in range(io_steps):
            pool.reset_queue()
            for (_, _, n, _), x in zip(nets, xs):
                pool.reset_nasm(n)
                pool.add_nasm_raw_input(n, x)
            dse.run()
            for _, _, n, _ in nets:
                dse.wait(n)
            dse.stop()
            for _, _, n, _ in nets:
                n.result()
        dt_io = (time.perf_counter() - t0) / io_steps
        out["host_io_inclusive"] = {"value": units_per_step / dt_io, "unit": unit, "ms_per_step": dt_io * 1e3, "steps": io_steps,
                                    "note": "input copied from pageable host memory and final layer copied back every step"}

    if args.engine_profile and args.mode == "dataflow":
        prof = pool.dataflow_profile()
        out["engine_profile"] = {k: v / max(prof["total"], 1e-12) for k, v in prof.items() if k not in ("total", "engine_clock_mhz")}
        out["engine_profile"]["engine_clock_mhz"] = prof["engine_clock_mhz"]
        out["engine_profile"]["workgroup_seconds_per_step"] = prof["total"] / args.steps
    if args.trace and args.mode == "dataflow":
        stamps = pool.dataflow_trace()
        tile_layer, base = [], 0
        for _, _, n, _ in nets:
            tile_layer.append(n.graph()[0].astype(np.int64) + base)
            base += n.num_ldata
        types = [n.info(l)["type"] for _, _, n, _ in nets for l in range(n.num_ldata)]
        np.savez(args.trace, stamps=stamps, phases=pool.dataflow_trace_phases(), tile_layer=np.concatenate(tile_layer), layer_type=np.array(types))
    if args.layer_profile:
        # conv-tile MFMA utilisation and bandwidth of the elementwise tiles, one kernel per layer
        nl = sum(n.num_ldata for _, _, n, _ in nets)
        lms = pool.profile_layers(nl, 5)
        per_type, per_layer, base = {}, [], 0
        for name, _, n, _ in nets:
            infos = [n.info(l) for l in range(n.num_ldata)]
            for l, i in enumerate(infos):
                t = api.LAYER_TYPE_NAMES[i["type"]]
                d = per_type.setdefault(t, {"ms": 0.0, "flops": 0, "bytes": 0})
                d["ms"] += float(lms[base + l])
                contraction = t in ("conv", "fc", "matmul", "attn_k", "attn_v")
                d["flops"] += i["flops"] if contraction else 0
                # algorithmic bytes of a bandwidth tile layer: its output once and each parent's matrix once
                nbytes = 0
                if not contraction and t != "input" and i["num_ninst"]:
                    nbytes = 4 * (i["H"] * i["W"] + sum(infos[p]["H"] * infos[p]["W"] for p in (i["p0"], i["p1"]) if 0 <= p < len(infos)))
                d["bytes"] += nbytes
                per_layer.append({"net": name, "layer": l, "type": t, "rows": i["H"], "columns": i["W"], "tiles": i["num_ninst"],
                                  "splits": i["splits"], "bytes": nbytes, "flops": i["flops"] if contraction else 0,
                                  "ms": round(float(lms[base + l]), 5)})
            base += n.num_ldata
        for t, d in per_type.items():
            if d["flops"]:
                d["tflops"] = d["flops"] / max(d["ms"], 1e-9) / 1e9
                d["mfma_util"] = d["tflops"] / PEAK_FP32_MFMA_TFLOPS
            if d["bytes"]:
                d["gbs"] = d["bytes"] / max(d["ms"], 1e-9) / 1e6
                d["hbm_frac"] = d["gbs"] / PEAK_HBM_GBS
        out["layer_profile"] = per_type
        out["layers"] = per_layer

    # the graph that was timed must also have computed the right thing: its final layer against the
    # compiled reference's fixture (outside the timed region)
    if not args.skip_tiles:
        checks = {name: verify_final_layer(name, n) for name, _, n, _ in nets}
        have = [c for c in checks.values() if c is not None]
        out["verified"] = all(c["ok"] for c in have) if have else None
        out["verification"] = checks

    dse.destroy()
    for _, dnn, nasm, _ in nets:
        nasm.destroy()
    pool.destroy()
    for _, dnn, nasm, _ in nets:
        dnn.destroy()
    del nets

    # the other configurations of the benchmark, each on its own tuned graph (value stays the headline workload's)
    plain = not (args.skip_tiles or args.engine_profile or args.trace or args.layer_profile or args.no_handoff or args.xcd_queues)
    if not args.no_other_workloads and plain and args.workload == "resnet50_b32":
        L.aspen_hip_set_flags(0)
        out["workloads"] = {}
        for name in WORKLOADS:
            if name != args.workload:
                out["workloads"][name] = measure_workload(api, M, name, max(5, min(args.steps, 20)), args.warmup)
        co, a, b = (out["workloads"].get(k) for k in ("co_resnet50_vgg16_b16", "resnet50_b16", "vgg16_b16"))
        if co and a and b:
            # ASPEN's point about co-scheduling: one merged ready queue against the same two graphs run one after the other
            co["back_to_back_ms"] = a["ms_per_step"] + b["ms_per_step"]
            co["speedup_over_back_to_back"] = co["back_to_back_ms"] / co["ms_per_step"]
        if not all(w["verified"] is not False for w in out["workloads"].values()):
            out["verified"] = False

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfgs[0])
        out["cpu_baseline"]["cpu"] = cpu_description()
        if args.workload == "resnet50_b32":
            b1 = cpu_baseline_dse("resnet50_b1")
            if b1 is not None:
                out["cpu_baseline_b1"] = b1
    if args.cpu_baseline_dse:
        out["cpu_baseline_dse"] = cpu_baseline_dse(args.cpu_baseline_dse, iters=5)
    emit(json.dumps(out))
    if out.get("verified") is False:
        print("bench.py: the timed graph's output does not match the reference fixture", file=sys.stderr)
        sys.exit(3)


if __name__ == "__main__":
    main()
