#!/usr/bin/env python3
"""Benchmark of the W4A4 linear hot path on one MI355X.

A "step" is one pass over the seven linear layers of a Llama-2-7B decoder block at
M = 2048 tokens (the configuration the headline metric is quoted on): per-token activation scales, per-channel
weight scales, fp16 activations with 1 % outlier channels.  Per step, issued the way a decoder layer issues it
(--launches layer, the default):

    rotate+quantise x[2048, 4096]          -> q, k, v as three weight matrices of ONE launch     (3 x 4096 x 4096)
    rotate+quantise x[2048, 4096]          -> o_proj                                            (4096 x 4096)
    rotate+quantise x[2048, 4096]          -> gate and up in ONE launch that stores silu(gate) * up   (2 x 11008 x 4096)
    rotate+quantise x[2048, 11008] (172x64)-> down_proj                                         (4096 x 11008)

--launches seven issues one GEMM launch per linear instead; whichever form is not the headline is timed and reported
beside it.  `value` is integer tera-operations per second of the whole step (2*M*N*K summed over the seven
contractions, divided by the wall time of the step including the four rotate+quantise launches), inputs resident in
HBM.  The JSON line also carries the roofline of the dominant kernel (the GEMM, against the dense int8 MFMA peak), the
roofline of the fused Hadamard-quant kernel (against HBM bandwidth), and the CPU oracle timed on a bounded sample of the
same workload.

Rotation modes (--hadamard): "fast" (default) runs the matrix-core kernels for all four launches: K = 4096 differs
from the float32-butterfly codes in fewer than 1e-5 of the positions (measured live and reported; it is closer to the
reference's float64 transform than the float32 butterflies are), K = 11008 = 172 x 64 in about 4e-4 (no summation
order is defined by the reference for its dense factor).  "mixed" runs the bit-exact float32-butterfly kernel for
K = 4096, "exact" for all four.  All modes are timed per kernel and reported either way.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--hadamard fast] [--launches layer]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

PEAK_INT8_TOPS = 5033.0   # 256 CU x 8192 int8 op/clk/CU x 2.4 GHz (dense)
PEAK_HBM_GBS = 8000.0
# Measured HBM traffic per launch at M = 2048 (fetch + write) is not a constant of this file: it is read from the
# machine-readable line ("bench.py reads: {...}") of the counter summary committed next to the profiles, so that the
# figure in the JSON line is the one the committed counter run produced.
TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "llama7b_block_M2048_hbm_traffic.txt")


def measured_traffic():
    """{"gemm": {"layer": bytes, "seven": bytes}, "rotate_quant_K4096": bytes} from the counter summary, or None."""
    try:
        for line in open(TRAFFIC_FILE):
            if line.startswith("bench.py reads:"):
                return json.loads(line.split(":", 1)[1])
    except (OSError, ValueError):
        pass
    return None


# (name, N, K, activation source) -- activation sources are quantised once and shared
LAYERS = [("q", 4096, 4096, "attn_in"), ("k", 4096, 4096, "attn_in"), ("v", 4096, 4096, "attn_in"),
          ("o", 4096, 4096, "attn_out"), ("gate", 11008, 4096, "mlp_in"), ("up", 11008, 4096, "mlp_in"),
          ("down", 4096, 11008, "mlp_mid")]
SOURCES = {"attn_in": 4096, "attn_out": 4096, "mlp_in": 4096, "mlp_mid": 11008}


def quant_bytes(m, k):
    return 2 * m * k + m * k // 2 + 2 * m          # fp16 in, packed nibbles + one fp16 scale per row out


def gemm_ops(m, n, k):
    return 2 * m * n * k


def make_inputs(m, seed=0):
    from flh_amd import synthetic as syn
    acts = {name: syn.activations(m, k, seed=seed + i) for i, (name, k) in enumerate(SOURCES.items())}
    weights = {}
    for i, (name, n, k, _) in enumerate(LAYERS):
        weights[name] = (syn.pack_codes(syn.weight_codes(n, k, seed=100 + i)), syn.weight_scales(n, 1, seed=200 + i))
    return acts, weights


def cpu_baseline(m_sample, min_seconds=10.0, budget_s=30.0):
    """The numpy oracle (a port of the reference's torch path) on the same seven layers and four
    rotate+quantise calls, repeated until at least `min_seconds` of CPU work have been timed (and
    stopped at `budget_s`); all host threads that numpy's BLAS uses."""
    from oracle import linear as L
    from oracle import gemm as G
    acts, weights = make_inputs(m_sample, seed=0)
    t0 = time.perf_counter()
    ops, passes = 0, 0
    while True:
        packed = {name: L.rotate_and_quantize(x, "f32")[:2] for name, x in acts.items()}
        for name, n, k, src in LAYERS:
            ap, sa = packed[src]
            G.gemm_i4_dequant(ap, weights[name][0], sa, weights[name][1])
            ops += gemm_ops(m_sample, n, k)
            if time.perf_counter() - t0 > budget_s:
                break
        passes += 1
        if time.perf_counter() - t0 >= min_seconds:
            break
    dt = time.perf_counter() - t0
    return {"value": ops / dt / 1e12, "unit": "TOPS", "cores": int(os.environ.get("OMP_NUM_THREADS", os.cpu_count())),
            "kind": "port", "seconds": round(dt, 3),
            "sample": f"{passes} passes over the same 7 Llama-2-7B linears + 4 rotate-quantise calls at M={m_sample} "
                      "(numpy oracle, float32 BLAS matmul of unpacked codes)"}


def operand_activity(torch, ops, m, launches, smi):
    """The q / k / v-sized launch (m x 12288 x 4096, one scale per row) on operands of decreasing switching activity:
    what separates the power limit of the part from the structure of the kernel.  Per case: median HIP-event time of
    `launches` back-to-back launches, and -- from a second thread, while the same launch keeps running -- the engine
    clock and the socket power rocm-smi reports.  A counter run (rocprofv3 --pmc GRBM_GUI_ACTIVE
    SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES) of this mode sees `launches` dispatches per case, in the order of the
    cases, behind the warm-up dispatches."""
    import re
    import subprocess
    import threading
    dev = torch.device("cuda:0")
    n, k = 12288, 4096
    sa = torch.full((m, 1), 0.01, dtype=torch.float16, device=dev)
    sb = torch.full((n, 1), 0.01, dtype=torch.float16, device=dev)
    out = {"shape": f"{m}x{n}x{k}", "launches_per_case": launches, "cases": {}}

    def smi_reading():
        try:
            txt = subprocess.run(["rocm-smi", "--showclocks", "--showpower"], capture_output=True, text=True, timeout=30).stdout
        except Exception:  # noqa: BLE001 -- the reading is optional
            return None, None
        mc = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", txt)
        mp = re.search(r"Power \(W\): ([0-9.]+)", txt)
        watts = float(mp.group(1)) if mp else None
        if watts is None:                                 # the tool prints no power on some boxes: the driver's own file
            import glob
            for f in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average") + \
                    glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"):
                try:
                    watts = int(open(f).read().strip()) / 1e6
                    break
                except Exception:  # noqa: BLE001
                    pass
        return (int(mc.group(1)) if mc else None), watts

    for label, hi in (("uniform_random_codes", 256), ("every_other_code_zero", 16), ("all_zero_codes", 1)):
        a = torch.randint(0, hi, (m, k // 2), dtype=torch.uint8, device=dev)
        b = torch.randint(0, hi, (n, k // 2), dtype=torch.uint8, device=dev)
        for _ in range(300):                              # steady clocks for this data
            ops.gemm_i4_dequant_o16(a, b, sa, sb)
        torch.cuda.synchronize()
        pairs = []
        for _ in range(launches):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            ops.gemm_i4_dequant_o16(a, b, sa, sb)
            e1.record()
            pairs.append((e0, e1))
        torch.cuda.synchronize()
        us = float(np.median([x.elapsed_time(y) * 1e3 for x, y in pairs]))
        case = {"us": round(us, 2), "TOPS": round(gemm_ops(m, n, k) / (us * 1e-6) / 1e12, 1),
                "frac_of_peak": round(gemm_ops(m, n, k) / (us * 1e-6) / 1e12 / PEAK_INT8_TOPS, 4)}
        if smi:
            reading = [None, None]

            def sample():
                time.sleep(0.7)
                reading[0], reading[1] = smi_reading()
            th = threading.Thread(target=sample)
            th.start()
            t0 = time.perf_counter()
            while th.is_alive() and time.perf_counter() - t0 < 20.0:
                for _ in range(100):
                    ops.gemm_i4_dequant_o16(a, b, sa, sb)
                torch.cuda.synchronize()
            th.join()
            case["engine_MHz"], case["socket_W"] = reading
            if reading[0]:
                case["frac_of_peak_at_that_clock"] = round(case["frac_of_peak"] * 2400.0 / reading[0], 4)
        out["cases"][label] = case
        del a, b
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--tokens", type=int, default=2048)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-tokens", type=int, default=2048)
    ap.add_argument("--no-vendor-reference", action="store_true",
                    help="skip timing the vendor library's int8 / fp16 GEMM on the same shapes")
    ap.add_argument("--no-decode-model", action="store_true",
                    help="skip the 32-layer Llama-3-8B decode step (about 6 GB of random weights)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch three elementwise passes over 256 MiB (read 256 MiB, write 256 MiB): the "
                         "known-size kernel that hardware-counter readings (FETCH_SIZE / WRITE_SIZE) are scaled by")
    ap.add_argument("--hadamard", choices=["mixed", "exact", "fast"], default="fast")
    ap.add_argument("--launches", choices=["layer", "seven"], default="layer",
                    help="GEMM launches of the timed step: the four a decoder layer issues (q/k/v in one launch, gate and "
                         "up in one launch that stores silu(gate)*up), or one per linear; the other form is reported beside it")
    ap.add_argument("--operand-activity-only", type=int, default=0, metavar="LAUNCHES",
                    help="diagnostic mode: only the q/k/v-sized GEMM launch (2048 x 12288 x 4096) on uniform random codes, "
                         "on codes with every other one zero and on all-zero codes, LAUNCHES back-to-back launches each "
                         "(in that order; the run under rocprofv3 --pmc that profiles/ summarises reads its counters per "
                         "dispatch), with the engine clock and socket power rocm-smi reports during each case")
    ap.add_argument("--no-smi", action="store_true", help="with --operand-activity-only: do not start rocm-smi")
    ap.add_argument("--step-only", type=int, default=0, metavar="STEPS",
                    help="profiling aid: after the warm-up run exactly STEPS steps of the headline form and exit")
    ap.add_argument("--decode-step-only", type=int, default=0, metavar="REPLAYS",
                    help="profiling aid: only the 32-layer Llama-3-8B decode step (kv_len 2048) of --decode-batch sequences, "
                         "captured into a graph and replayed REPLAYS times after five warm replays")
    ap.add_argument("--decode-batch", type=int, default=1)
    ap.add_argument("--large-tokens", type=int, default=16384,
                    help="token count of the extra Hadamard-quant launches that amortise the launch floor")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every box of this build has a single MI355X and the path has no "
                 "cross-GPU part; run with --gpus 1")

    import torch
    import flh_amd
    from flh_amd import synthetic as syn
    ops = flh_amd._CUDA           # the PyTorch-ROCm extension in front of the C ABI (ctypes ops where it has no wrapper)
    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X (no CPU fallback for the product path)")
    M = args.tokens
    if args.operand_activity_only:
        print(json.dumps(operand_activity(torch, ops, M, args.operand_activity_only, not args.no_smi)))
        return
    if args.decode_step_only:
        from flh_amd.quantized_model import LlamaShape, W4A4LlamaModel
        with torch.no_grad():
            model = W4A4LlamaModel.random_init(LlamaShape.llama3_8b(num_layers=32), activation="token", weight_group_size=128,
                                               fused=True, seed=1)
        graph, state = model.capture_decode_step(args.decode_batch, 2048)
        for i in range(32):
            state["cache"].keys[i].normal_()
            state["cache"].values[i].normal_()
        for _ in range(5):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.decode_step_only):
            graph.replay()
        torch.cuda.synchronize()
        print(json.dumps({"mode": "decode-step-only", "batch": args.decode_batch, "replays": args.decode_step_only,
                          "ms_per_step": round((time.perf_counter() - t0) / args.decode_step_only * 1e3, 3)}))
        return
    acts_h, weights_h = make_inputs(M)
    dev = torch.device("cuda:0")
    acts = {k: torch.from_numpy(v).to(dev) for k, v in acts_h.items()}
    weights = {k: (torch.from_numpy(w).to(dev), torch.from_numpy(s).to(dev)) for k, (w, s) in weights_h.items()}

    def had_mode(k):
        if args.hadamard == "mixed":                    # what hadamard=True selects
            return "exact" if k & (k - 1) == 0 else "fast"
        return args.hadamard

    # The launches of one step.  "layer": what a decoder layer issues (flh_amd.quantized_model) -- q / k / v as three
    # weight matrices of one launch, o, gate and up as one launch that stores silu(gate) * up, down: the same seven
    # contractions in four GEMM launches.  "seven": one launch per linear.
    FORMS = {"layer": [("qkv", "attn_in", ["q", "k", "v"]), ("o", "attn_out", ["o"]),
                       ("gate_up_swiglu", "mlp_in", ["gate", "up"]), ("down", "mlp_mid", ["down"])],
             "seven": [(name, src, [name]) for name, _, _, src in LAYERS]}
    shape_of = {name: (n, k) for name, n, k, _ in LAYERS}

    def launch(parts, q, s):
        if len(parts) == 1:
            return ops.gemm_i4_dequant_o16(q, weights[parts[0]][0], s, weights[parts[0]][1])
        if parts == ["gate", "up"]:
            return ops.gemm_i4_swiglu(q, weights["gate"][0], weights["up"][0], s, weights["gate"][1], weights["up"][1])
        return ops.gemm_i4_dequant_multi(q, [weights[n][0] for n in parts], s, [weights[n][1] for n in parts])

    def make_step(form):
        def step(events=None):
            packed = {}
            for name in SOURCES:
                if events is not None:
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                packed[name] = ops.rotate_and_quantize_i4(acts[name], hadamard=had_mode(SOURCES[name]))
                if events is not None:
                    e1.record()
                    events.append(("quant", name, e0, e1))
            out = None
            for name, src, parts in FORMS[form]:
                q, s = packed[src]
                if events is not None:
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                out = launch(parts, q, s)
                if events is not None:
                    e1.record()
                    events.append(("gemm", name, e0, e1))
            return out
        return step

    warm_q, warm_s = ops.rotate_and_quantize_i4(acts["attn_in"], hadamard="exact")

    def warm_gpu():
        """Sustained matrix work until it stops getting faster: after a pause (host work, allocations, a comparison
        that synchronises) the part takes some ten milliseconds of load to return to its steady clocks, and a side
        figure measured in that time reads up to 40 % slow."""
        prev = float("inf")
        for batch in range(30):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                ops.gemm_i4_dequant_o16(warm_q, weights["gate"][0], warm_s, weights["gate"][1])
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            if batch >= 6 and ms > 0.985 * prev:
                break
            prev = ms

    def engine_clock_under_load(lead=0.5, limit=20.0):
        """The engine clock (MHz) the part sustains while one of the step's GEMMs runs back to back, as rocm-smi reports
        it from a second thread (None where the tool or the reading is not available): under dense matrix work these
        parts settle well below the 2400 MHz the published peak is quoted at, and the fraction of that peak inherits it."""
        import re
        import subprocess
        import threading
        reading = [None]

        def sample():
            time.sleep(lead)
            try:
                out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=30).stdout
                m = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", out)
                reading[0] = int(m.group(1)) if m else None
            except Exception:
                reading[0] = None
        th = threading.Thread(target=sample)
        th.start()
        t0 = time.perf_counter()
        while th.is_alive() and time.perf_counter() - t0 < limit:    # the load lasts as long as the reading takes
            for _ in range(100):
                ops.gemm_i4_dequant_o16(warm_q, weights["gate"][0], warm_s, weights["gate"][1])
            torch.cuda.synchronize()
        th.join()
        return reading[0]

    def run_form(form):
        """(ms per step over exactly --steps steps after --warmup, median us per launch from a second pass with HIP
        events on the launch stream around every launch)"""
        step = make_step(form)
        warm_gpu()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / args.steps * 1e3
        events = []
        for _ in range(args.steps):
            step(events)
        torch.cuda.synchronize()
        per = {}
        for kind, name, e0, e1 in events:
            per.setdefault((kind, name), []).append(e0.elapsed_time(e1) * 1e3)  # us
        return ms, {k: float(np.median(v)) for k, v in per.items()}

    if args.step_only:
        # profiling aid: warm up, then exactly this many steps of the headline form and nothing else, so that the last
        # 8 (layer form) / 11 (seven) dispatches per step of a kernel trace are the step's launches in order
        step = make_step(args.launches)
        warm_gpu()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.step_only):
            step()
        torch.cuda.synchronize()
        print(json.dumps({"mode": "step-only", "launches": args.launches, "steps": args.step_only,
                          "us_per_step": round((time.perf_counter() - t0) / args.step_only * 1e6, 1)}))
        return
    other_form = "seven" if args.launches == "layer" else "layer"
    # the other form first: the first few hundred launches of a process run below the steady rate (clocks and caches
    # settle for longer than a handful of warm-up steps), which would otherwise be charged to whichever form is timed first
    ms_other, med_other = run_form(other_form)
    ms_per_step, med = run_form(args.launches)      # the headline: --warmup untimed steps, then exactly --steps timed ones
    sclk = engine_clock_under_load()
    step = make_step("seven")

    # The same step with the weights of projections that share an input stored concatenated ([q; k; v] and
    # [gate; up], as a model loader may lay them out): identical outputs from four GEMM launches instead of
    # seven, through the same entry point.  Reported beside the headline figure, never as it.
    cat = {"qkv": ("attn_in", ["q", "k", "v"]), "o": ("attn_out", ["o"]), "gate_up": ("mlp_in", ["gate", "up"]),
           "down": ("mlp_mid", ["down"])}
    cat_w = {name: (torch.cat([weights[n][0] for n in parts]), torch.cat([weights[n][1] for n in parts]))
             for name, (_, parts) in cat.items()}

    def step_concatenated():
        packed = {name: ops.rotate_and_quantize_i4(acts[name], hadamard=had_mode(SOURCES[name])) for name in SOURCES}
        for name, (src, _) in cat.items():
            out = ops.gemm_i4_dequant_o16(*packed[src][:1], cat_w[name][0], packed[src][1], cat_w[name][1])
        return out

    for _ in range(args.warmup):
        step_concatenated()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_concatenated()
    torch.cuda.synchronize()
    ms_concat = (time.perf_counter() - t0) / args.steps * 1e3
    del cat_w


    # ... and with the weights left where they are: the projections that share an input go through the entry point
    # that takes several weight matrices (gemm_i4_dequant_multi), again four GEMM launches, identical outputs
    def step_shared_launches():
        packed = {name: ops.rotate_and_quantize_i4(acts[name], hadamard=had_mode(SOURCES[name])) for name in SOURCES}
        for name, (src, parts) in cat.items():
            out = ops.gemm_i4_dequant_multi(packed[src][0], [weights[n][0] for n in parts], packed[src][1],
                                            [weights[n][1] for n in parts])
        return out

    for _ in range(args.warmup):
        step_shared_launches()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_shared_launches()
    torch.cuda.synchronize()
    ms_shared = (time.perf_counter() - t0) / args.steps * 1e3
    pq, ps = ops.rotate_and_quantize_i4(acts["attn_in"], hadamard=had_mode(4096))
    qkv = ops.gemm_i4_dequant_multi(pq, [weights[n][0] for n in "qkv"], ps, [weights[n][1] for n in "qkv"])
    shared_equal = all(torch.equal(d, ops.gemm_i4_dequant_o16(pq, weights[n][0], ps, weights[n][1]))
                       for d, n in zip(qkv, "qkv"))
    del qkv, pq, ps

    # ... and with gate and up as ONE launch that stores only silu(gate) * up (gemm_i4_swiglu): what a SwiGLU MLP needs
    # in front of the down_proj rotation, without the two fp16 [M, 11008] intermediates and torch's two elementwise
    # kernels.  Same seven contractions, six GEMM launches.
    def step_swiglu():
        packed = {name: ops.rotate_and_quantize_i4(acts[name], hadamard=had_mode(SOURCES[name])) for name in SOURCES}
        for name, n, k, src in LAYERS:
            if name in ("gate", "up"):
                continue
            out = ops.gemm_i4_dequant_o16(packed[src][0], weights[name][0], packed[src][1], weights[name][1])
        return ops.gemm_i4_swiglu(packed["mlp_in"][0], weights["gate"][0], weights["up"][0], packed["mlp_in"][1],
                                  weights["gate"][1], weights["up"][1])

    for _ in range(args.warmup):
        step_swiglu()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_swiglu()
    torch.cuda.synchronize()
    ms_swiglu = (time.perf_counter() - t0) / args.steps * 1e3

    def timed(calls):
        """median duration in us over `calls` (a list of thunks, each one launch): HIP events on the
        launch stream around each launch, at steady clocks, with a few GEMMs queued first so that the host runs
        ahead of the GPU and the events do not measure host launch gaps"""
        warm_gpu()
        for _ in range(10 + len(calls)):
            ops.gemm_i4_dequant_o16(warm_q, weights["gate"][0], warm_s, weights["gate"][1])
        pairs = []
        for fn in calls:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            pairs.append((e0, e1))
        torch.cuda.synchronize()
        return float(np.median([a.elapsed_time(b) * 1e3 for a, b in pairs]))

    pq_m, ps_m = ops.rotate_and_quantize_i4(acts["mlp_in"], hadamard=had_mode(4096))
    wg_, wu_ = weights["gate"], weights["up"]

    def unfused_mlp_front():
        g_ = ops.gemm_i4_dequant_o16(pq_m, wg_[0], ps_m, wg_[1])
        u_ = ops.gemm_i4_dequant_o16(pq_m, wu_[0], ps_m, wu_[1])
        return torch.nn.functional.silu(g_) * u_

    swiglu = {"us_per_layer": round(ms_swiglu * 1e3, 1),
              "TOPS": round(sum(gemm_ops(M, n, k) for _, n, k, _ in LAYERS) / (ms_swiglu * 1e-3) / 1e12, 2),
              "gate_up_one_launch_us": round(timed([lambda: ops.gemm_i4_swiglu(pq_m, wg_[0], wu_[0], ps_m, wg_[1], wu_[1])] * 20), 2),
              "gate_up_two_launches_plus_torch_silu_mul_us": round(timed([unfused_mlp_front] * 10), 2),
              "launches": "4 rotate-quantise + 5 GEMM + 1 gate/up GEMM that stores silu(gate) * up only"}
    swiglu["gate_up_one_launch_TOPS"] = round(2 * gemm_ops(M, 11008, 4096) / (swiglu["gate_up_one_launch_us"] * 1e-6) / 1e12, 1)
    del pq_m, ps_m

    def time_quant(x, mode, reps=20):
        return timed([lambda: ops.rotate_and_quantize_i4(x, hadamard=mode)] * reps)

    modes = {}
    for k, src in ((4096, "attn_in"), (11008, "mlp_mid")):
        for mode in ("exact", "fast"):
            us = time_quant(acts[src], mode)
            modes[f"K={k}:{mode}"] = {"us": round(us, 2), "GB/s": round(quant_bytes(M, k) / (us * 1e-6) / 1e9, 1)}
    ML = args.large_tokens
    xl = torch.from_numpy(np.tile(acts_h["attn_in"], (ML // M + 1, 1))[:ML].copy()).to(dev)
    large = {}
    for mode in ("exact", "fast"):
        us = time_quant(xl, mode)
        large[mode] = {"us": round(us, 2), "GB/s": round(quant_bytes(ML, 4096) / (us * 1e-6) / 1e9, 1)}
    # what a launch of this size reaches when it only streams: a device copy of the same fp16 rows (it writes four
    # times the bytes the quantiser writes), timed the same way -- the launch floor is visible at M = 2048
    same_size_copy = {}
    for m_c, x_c in ((M, acts["attn_in"]), (ML, xl)):
        dst = torch.empty_like(x_c)
        us = timed([lambda: dst.copy_(x_c)] * 20)
        same_size_copy[f"M={m_c}"] = {"us": round(us, 2), "GB/s_read_plus_write": round(2 * x_c.numel() * 2 / (us * 1e-6) / 1e9, 1)}
        del dst

    # the reference's own kernels for the same activations: groups of 128 (had_and_quant / quant_and_pack /
    # in-place FWHT); bytes: fp16 in, nibbles + one fp16 scale per group out (FWHT: fp16 in and out)
    group = {}
    for m_g, xg in ((M, acts["attn_in"]), (ML, xl)):
        rows = xg.numel() // 128
        x128 = xg.view(rows, 128)
        scratch = x128.clone()
        byts = rows * (256 + 64 + 2)
        for label, fn, b in (("had_and_quant", lambda: ops.hadamard_and_quantize_i4(x128), byts),
                             ("quant_and_pack", lambda: ops.quant_and_pack_i4(x128), byts),
                             ("fwht_inplace", lambda: ops.hadamard_transform_half(scratch), rows * 512)):
            us = timed([fn] * 20)
            group[f"{label},M={m_g}"] = {"us": round(us, 2), "GB/s": round(b / (us * 1e-6) / 1e9, 1)}
        del scratch

    # the two elementwise producers of quantised activations fused into the group quantiser, beside the
    # unfused pair (torch's kernel writing the fp16 intermediate, then the group quantiser reading it);
    # bytes: fp16 inputs in, nibbles + one fp16 scale per group of 128 out
    fused = {}
    for m_g, xg in ((M, acts["attn_in"]), (ML, xl)):
        gate = torch.randn(m_g, 11008, dtype=torch.float16, device=dev)
        up = torch.randn(m_g, 11008, dtype=torch.float16, device=dev)
        wn = torch.rand(4096, dtype=torch.float16, device=dev) + 0.5
        unfused_mlp = lambda: ops.quant_and_pack_i4((torch.nn.functional.silu(gate) * up).view(-1, 128))
        unfused_norm = lambda: ops.quant_and_pack_i4(
            (xg.float() * torch.rsqrt(xg.float().pow(2).mean(-1, keepdim=True) + 1e-5) * wn).half().view(-1, 128))
        for label, fn, b in (("silu_mul_quant,K=11008", lambda: ops.silu_mul_and_quantize_i4_gs(gate, up, 128),
                              m_g * 11008 * 4.5 + m_g * 86 * 2),
                             ("silu_mul_quant,K=11008,unfused", unfused_mlp, None),
                             ("rmsnorm_quant,K=4096", lambda: ops.rmsnorm_and_quantize_i4_gs(xg, wn, 1e-5, 128),
                              m_g * 4096 * 2.5 + m_g * 32 * 2),
                             ("rmsnorm_quant,K=4096,unfused", unfused_norm, None),
                             ("rmsnorm_rotate_quant,K=4096", lambda: ops.rmsnorm_rotate_and_quantize_i4(xg, wn, 1e-5),
                              quant_bytes(m_g, 4096)),
                             ("rotate_quant,K=4096", lambda: ops.rotate_and_quantize_i4(xg, hadamard="exact"),
                              quant_bytes(m_g, 4096))):
            us = timed([fn] * 10)
            fused[f"{label},M={m_g}"] = {"us": round(us, 2)}
            if b:
                fused[f"{label},M={m_g}"]["GB/s"] = round(b / (us * 1e-6) / 1e9, 1)
        del gate, up
    del xl

    # Cold inputs, timed without host gaps: a graph of launches over distinct input / output buffers that together exceed
    # the 256 MB last-level cache (no launch finds its rows on chip), replayed; per-launch time = replay / launches.
    # For every shape: the float32-butterfly mode, the matrix-core mode, the same kernel without rotation (quantise only)
    # and a plain device copy of the same fp16 rows -- the two streaming floors a rotation kernel can be held against.
    def graph_us(fns, reps=10):
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for f in fns:
                f()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for f in fns:
                f()
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps / len(fns)

    side = torch.cuda.Stream()
    cold = {}
    for k_c, m_c in ((4096, M), (11008, M), (14336, M), (4096, ML)):
        n_buf = max(4, int(300e6 // (m_c * k_c * 2)) + 1)
        base = torch.from_numpy(syn.activations(min(m_c, 2048), k_c, seed=k_c)).to(dev)
        xs_c = [base.repeat(m_c // base.size(0), 1) if m_c > base.size(0) else base.clone() for _ in range(n_buf)]
        ys_c = [torch.empty_like(x) for x in xs_c[:2]]
        row = {"distinct_inputs": n_buf, "algorithmic_bytes": quant_bytes(m_c, k_c)}
        for label, fn in (("fast", lambda x, i: ops.rotate_and_quantize_i4(x, hadamard="fast")),
                          ("exact", lambda x, i: ops.rotate_and_quantize_i4(x, hadamard="exact")),
                          ("quantise_only", lambda x, i: ops.rotate_and_quantize_i4(x, hadamard=False)),
                          ("device_copy", lambda x, i: ys_c[i % 2].copy_(x))):
            if label == "exact" and k_c != 4096 and m_c > 2048:
                continue
            us = graph_us([(lambda x=x, i=i: fn(x, i)) for i, x in enumerate(xs_c)])
            byts = 2 * 2 * m_c * k_c if label == "device_copy" else quant_bytes(m_c, k_c)
            row[label] = {"us": round(us, 2), "GB/s": round(byts / (us * 1e-6) / 1e9, 1),
                          "frac_hbm": round(byts / (us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4)}
        row["fast_over_quantise_only"] = round(row["fast"]["us"] / row["quantise_only"]["us"], 3)
        cold[f"K={k_c},M={m_c}"] = row
        del xs_c, ys_c, base
    # how far the matrix-core mode is from the float32-butterfly codes (K = 4096: both against each other on the device)
    qe_, se_ = ops.rotate_and_quantize_i4(acts["attn_in"], hadamard="exact")
    qf_, sf_ = ops.rotate_and_quantize_i4(acts["attn_in"], hadamard="fast")
    nib = lambda t: torch.stack((t & 15, t >> 4), -1)
    cold["K=4096:fast_vs_exact_code_mismatch_rate"] = float((nib(qe_) != nib(qf_)).float().mean())
    cold["K=4096:fast_vs_exact_scale_mismatch_rate"] = float((se_ != sf_).float().mean())
    del qe_, se_, qf_, sf_

    # decode (M = 1): the whole step is launch-bound, so it is also recorded into a graph once and replayed
    # (the library allocates nothing and needs no set-up after flh_init, so it can be captured as it is)
    x1 = {name: acts[name][:1].contiguous() for name in SOURCES}

    def decode_step():
        packed = {name: ops.rotate_and_quantize_i4(x1[name], hadamard=had_mode(SOURCES[name])) for name in SOURCES}
        for name, n, k, src in LAYERS:
            out = ops.gemm_i4_dequant_o16(packed[src][0], weights[name][0], packed[src][1], weights[name][1])
        return out

    def wall_us(fn, reps=200):
        warm_gpu()
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e6

    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        decode_step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        decode_step()
    decode = {"eager_us_per_layer": round(wall_us(decode_step), 1), "graph_replay_us_per_layer": round(wall_us(graph.replay), 1),
              "launches": "4 rotate-quantise + 7 GEMM at M = 1", "weight_bytes": int(sum(n * k // 2 for _, n, k, _ in LAYERS))}
    decode["graph_GB/s"] = round(decode["weight_bytes"] / (decode["graph_replay_us_per_layer"] * 1e-6) / 1e9, 1)
    del graph

    # ... with the projections that share a token as several weight matrices of one launch (4 GEMM launches
    # instead of 7, weights stored separately), and with the K = 4096 quantisers inside their GEMMs on top
    # (rotate_quantize_gemm_i4[_multi]: same bits, a launch less per GEMM; the K = 11008 rotation keeps its own)
    def decode_step_shared():
        packed = {name: ops.rotate_and_quantize_i4(x1[name], hadamard=had_mode(SOURCES[name])) for name in SOURCES}
        for name, (src, parts) in cat.items():
            out = ops.gemm_i4_dequant_multi(packed[src][0], [weights[n][0] for n in parts], packed[src][1],
                                            [weights[n][1] for n in parts])
        return out

    def decode_step_quantiser_inside(shared):
        groups = [(src, parts) for _, (src, parts) in cat.items()] if shared else [(src, [n]) for n, _, _, src in LAYERS]
        for src, parts in groups:
            if SOURCES[src] == 4096:
                out = ops.rotate_quantize_gemm_i4_multi(x1[src], [weights[n][0] for n in parts], [weights[n][1] for n in parts])
            else:
                pq, ps = ops.rotate_and_quantize_i4(x1[src], hadamard=had_mode(SOURCES[src]))
                out = ops.gemm_i4_dequant_multi(pq, [weights[n][0] for n in parts], ps, [weights[n][1] for n in parts])
        return out

    for label, fn in (("graph_replay_us_per_layer_shared_launches", decode_step_shared),
                      ("graph_replay_us_per_layer_quantiser_inside_gemm", lambda: decode_step_quantiser_inside(False)),
                      ("graph_replay_us_per_layer_quantiser_inside_gemm_shared_launches",
                       lambda: decode_step_quantiser_inside(True))):
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        decode[label] = round(wall_us(graph.replay), 1)
        del graph

    def two_launches(name, src):
        pq, ps = ops.rotate_and_quantize_i4(x1[src], hadamard="exact")
        return ops.gemm_i4_dequant_o16(pq, weights[name][0], ps, weights[name][1])

    same = all(torch.equal(ops.rotate_quantize_gemm_i4(x1[src], weights[name][0], weights[name][1]), two_launches(name, src))
               for name, n, k, src in LAYERS if k == 4096)
    decode["quantiser_inside_gemm_equal_to_two_launches"] = bool(same)

    # the same three GEMM shapes through the 6-bit matrix instruction (operands re-encoded at 6 bits per code;
    # bit-identical outputs), and the re-encoding of the activations that path needs per call
    f6 = {}
    for name, n, k, src in (("qkvo", 4096, 4096, "attn_in"), ("gate_up", 11008, 4096, "mlp_in"),
                            ("down", 4096, 11008, "mlp_mid")):
        w, ws = weights["q" if name == "qkvo" else "gate" if name == "gate_up" else "down"]
        aq, asc = ops.rotate_and_quantize_i4(acts[src], hadamard=had_mode(k))
        w6, a6 = ops.encode_f6(w), ops.encode_f6(aq)
        same = bool(torch.equal(ops.gemm_f6_dequant_o16(a6, w6, asc, ws), ops.gemm_i4_dequant_o16(aq, w, asc, ws)))
        us = timed([lambda: ops.gemm_f6_dequant_o16(a6, w6, asc, ws)] * 20)
        us_enc = timed([lambda: ops.encode_f6(aq)] * 20)
        f6[f"{n}x{k}"] = {"us": round(us, 2), "TOPS": round(gemm_ops(M, n, k) / (us * 1e-6) / 1e12, 1),
                          "encode_activations_us": round(us_enc, 2), "equal_to_int8_path": same}
        del w6, a6
    # The headline step itself on the 6-bit matrix instruction (side figure, never `value`): the quantisers write the
    # 6-bit operand format directly (matrix-core rotation), weights re-encoded once, the same four launches as the layer
    # form -- q/k/v in one, o, gate and up in one that stores silu(gate) * up, down.  Same outputs bit for bit.
    w6_all = {name: ops.encode_f6(weights[name][0]) for name in weights}

    def step_6bit(events=None):
        out = None
        for src, parts in (("attn_in", ["q", "k", "v"]), ("attn_out", ["o"]), ("mlp_in", ["gate", "up"]), ("mlp_mid", ["down"])):
            a6, ps = ops.rotate_and_quantize_f6(acts[src], hadamard=(True if SOURCES[src] != 4096 else "fast"))
            if events is not None:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            if parts == ["gate", "up"]:
                out = ops.gemm_f6_swiglu(a6, w6_all["gate"], w6_all["up"], ps, weights["gate"][1], weights["up"][1])
            elif len(parts) == 1:
                out = ops.gemm_f6_dequant_o16(a6, w6_all[parts[0]], ps, weights[parts[0]][1])
            else:
                out = ops.gemm_f6_dequant_multi(a6, [w6_all[n] for n in parts], ps, [weights[n][1] for n in parts])
            if events is not None:
                e1.record()
                events.append((src, e0, e1))
        return out

    us_step6 = wall_us(step_6bit, reps=args.steps)
    ev6 = []
    for _ in range(args.steps):
        step_6bit(ev6)
    torch.cuda.synchronize()
    per6 = {}
    for src, e0, e1 in ev6:
        per6.setdefault(src, []).append(e0.elapsed_time(e1) * 1e3)
    gemm6_us = sum(float(np.median(v)) for v in per6.values())
    f6["step_in_layer_form"] = {
        "us_per_layer": round(us_step6, 1),
        "TOPS": round(sum(gemm_ops(M, n, k) for _, n, k, _ in LAYERS) / (us_step6 * 1e-6) / 1e12, 1),
        "gemm_launch_us": {src: round(float(np.median(v)), 2) for src, v in per6.items()},
        "gemm_TOP/s": round(sum(gemm_ops(M, n, k) for _, n, k, _ in LAYERS) / (gemm6_us * 1e-6) / 1e12, 1),
        "gemm_frac_of_int8_peak": round(sum(gemm_ops(M, n, k) for _, n, k, _ in LAYERS) / (gemm6_us * 1e-6) / 1e12 / PEAK_INT8_TOPS, 4),
        "note": "v_mfma_f32_32x32x64_f8f6f4 on int4 codes encoded as e3m2 (exact); the headline stays on the int8 instruction"}
    del w6_all
    # group scales of 128 on the weights, one scale per token (the Llama-3 weight-group configuration), both kernels
    for n, k in ((4096, 4096), (14336, 4096)):
        wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev)
        wsg = (torch.rand(n, k // 128, device=dev) * 0.015 + 0.005).half()
        aq, asc = ops.rotate_and_quantize_i4(acts["attn_in"], hadamard=had_mode(k))
        w6, a6 = ops.encode_f6(wq), ops.encode_f6(aq)
        same = bool(torch.equal(ops.gemm_f6_dequant_o16_gs(a6, w6, asc, wsg), ops.gemm_i4_dequant(aq, wq, asc, wsg, 128)))
        us6 = timed([lambda: ops.gemm_f6_dequant_o16_gs(a6, w6, asc, wsg)] * 20)
        us8 = timed([lambda: ops.gemm_i4_dequant(aq, wq, asc, wsg, 128)] * 20)
        f6[f"{n}x{k},weight_groups_of_128"] = {"us": round(us6, 2), "int8_kernel_us": round(us8, 2),
                                               "TOPS": round(gemm_ops(M, n, k) / (us6 * 1e-6) / 1e12, 1),
                                               "equal_to_int8_path": same}
        del wq, wsg, w6, a6
    # the group quantiser writing the 6-bit operand format itself (no separate encoding pass), beside the
    # same launch with nibble output; K = 4096 as groups of 128, with the transform
    x_g = acts["attn_in"]
    q6g, s6g = ops.group_quantize_f6(x_g, True)
    q4g, s4g = ops.hadamard_and_quantize_i4(x_g.view(-1, 128))
    f6["group_quantiser_6bit_output,K=4096"] = {
        "us": round(timed([lambda: ops.group_quantize_f6(x_g, True)] * 20), 2),
        "nibble_output_us": round(timed([lambda: ops.hadamard_and_quantize_i4(x_g.view(-1, 128))] * 20), 2),
        "equal_to_encoded_nibbles": bool(torch.equal(q6g, ops.encode_f6(q4g.view(M, -1))) and
                                         torch.equal(s6g.view(-1), s4g.view(-1)))}
    del q6g, s6g, q4g, s4g

    # the Llama-3-8B block of the same path: group-wise weight scales (g = 128), one activation scale per token, grouped
    # queries (k / v 1024 wide), intermediate 14336 with the 28 x 512 online rotation; per layer, weights on the device
    L3 = [("q", 4096, 4096, "attn_in"), ("k", 1024, 4096, "attn_in"), ("v", 1024, 4096, "attn_in"), ("o", 4096, 4096, "attn_out"),
          ("gate", 14336, 4096, "mlp_in"), ("up", 14336, 4096, "mlp_in"), ("down", 4096, 14336, "mlp_mid")]
    L3_SRC = {"attn_in": 4096, "attn_out": 4096, "mlp_in": 4096, "mlp_mid": 14336}
    acts3 = {name: (acts[name] if k == 4096 else torch.from_numpy(syn.activations(M, k, seed=31)).to(dev)) for name, k in L3_SRC.items()}
    w3 = {name: (torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev),
                 (torch.rand(n, k // 128, device=dev) * 0.015 + 0.005).half()) for name, n, k, _ in L3}
    groups3 = [("attn_in", ["q", "k", "v"]), ("attn_out", ["o"]), ("mlp_in", ["gate", "up"]), ("mlp_mid", ["down"])]

    def llama3_step(shared):
        packed = {name: ops.rotate_and_quantize_i4(acts3[name], hadamard=had_mode(L3_SRC[name])) for name in L3_SRC}
        for src, parts in groups3:
            if shared:
                out = ops.gemm_i4_dequant_multi(packed[src][0], [w3[n][0] for n in parts], packed[src][1], [w3[n][1] for n in parts])
            else:
                for n in parts:
                    out = ops.gemm_i4_dequant(packed[src][0], w3[n][0], packed[src][1], w3[n][1], 128)
        return out

    ops3 = sum(gemm_ops(M, n, k) for _, n, k, _ in L3)
    llama3 = {}
    for label, shared_form in (("seven_launches", False), ("shared_activation_launches", True)):
        us = wall_us(lambda: llama3_step(shared_form), reps=args.steps)
        llama3[label] = {"us_per_layer": round(us, 1), "TOPS": round(ops3 / (us * 1e-6) / 1e12, 1)}
    # ... and on the 6-bit matrix instruction: weights re-encoded once, activations re-encoded after each quantiser
    w3_6 = {name: ops.encode_f6(w3[name][0]) for name in w3}

    def llama3_step_6bit():
        for src, parts in groups3:
            pq, ps = ops.rotate_and_quantize_i4(acts3[src], hadamard=had_mode(L3_SRC[src]))
            a6 = ops.encode_f6(pq)
            for n in parts:
                out = ops.gemm_f6_dequant_o16_gs(a6, w3_6[n], ps, w3[n][1])
        return out

    us = wall_us(llama3_step_6bit, reps=args.steps)
    llama3["six_bit_matrix_instruction"] = {"us_per_layer": round(us, 1), "TOPS": round(ops3 / (us * 1e-6) / 1e12, 1)}

    # ... with the quantisers writing the 6-bit format themselves (no encoding pass; K = 4096 in the run's rotation mode,
    # matrix cores for K = 14336) and the projections that share an input in one launch: what a token-configuration layer
    # with group-scaled weights issues for 256 rows or more
    def llama3_step_6bit_direct():
        for src, parts in groups3:
            a6, ps = ops.rotate_and_quantize_f6(acts3[src], hadamard=(True if L3_SRC[src] != 4096 else had_mode(4096)))
            out = ops.gemm_f6_dequant_multi(a6, [w3_6[n] for n in parts], ps, [w3[n][1] for n in parts])
        return out

    us = wall_us(llama3_step_6bit_direct, reps=args.steps)
    llama3["six_bit_direct_format,shared_launches"] = {"us_per_layer": round(us, 1),
                                                       "TOPS": round(ops3 / (us * 1e-6) / 1e12, 1)}
    # the same block at decode sizes (the linears of one layer of a Llama-3-8B decode step, batch x 1 token): graph
    # replays of 4 rotate-quantise + 4 GEMM launches (q/k/v and gate/up share their tokens), weights read once per step
    w3_bytes = int(sum(n * k // 2 + n * (k // 128) * 2 for _, n, k, _ in L3))
    llama3_decode = {"weight_and_scale_bytes_per_layer": w3_bytes}
    for batch in (1, 8, 16):
        xb = {name: acts3[name][:batch].contiguous() for name in L3_SRC}

        def llama3_decode_step():
            for src, parts in groups3:
                pq, ps = ops.rotate_and_quantize_i4(xb[src], hadamard=had_mode(L3_SRC[src]))
                out = ops.gemm_i4_dequant_multi(pq, [w3[n][0] for n in parts], ps, [w3[n][1] for n in parts], 128)
            return out

        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            llama3_decode_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            llama3_decode_step()
        us = wall_us(graph.replay)
        llama3_decode[f"batch={batch}"] = {"graph_replay_us_per_layer": round(us, 1),
                                           "GB/s": round(w3_bytes / (us * 1e-6) / 1e9, 1),
                                           "frac_hbm": round(w3_bytes / (us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4)}
        del graph
        if batch == 1:   # the K = 4096 quantisers inside their GEMMs (5 launches instead of 8)
            def llama3_decode_step_fused():
                for src, parts in groups3:
                    if L3_SRC[src] == 4096:
                        out = ops.rotate_quantize_gemm_i4_multi(xb[src], [w3[n][0] for n in parts], [w3[n][1] for n in parts])
                    else:
                        pq, ps = ops.rotate_and_quantize_i4(xb[src], hadamard=had_mode(L3_SRC[src]))
                        out = ops.gemm_i4_dequant_multi(pq, [w3[n][0] for n in parts], ps, [w3[n][1] for n in parts], 128)
                return out

            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                llama3_decode_step_fused()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                llama3_decode_step_fused()
            us = wall_us(graph.replay)
            llama3_decode["batch=1"]["quantiser_inside_gemm_us_per_layer"] = round(us, 1)
            del graph
        del xb
    del acts3, w3, w3_6

    # a whole W4A4 decoder layer of the Llama-2-7B shape (flh_amd.quantized_model: norms, group quantisers without
    # rotation as the reference's model uses them, the seven linears, RoPE, torch's attention, residuals), module by
    # module as the reference sequences it and in the fused form (same codes; see tests/test_gpu_decoder_layer.py)
    from flh_amd.quantized_model import W4A4DecoderLayer, rotary_tables
    from flh_amd.nn import LinearFLH
    gen = torch.Generator(device="cpu").manual_seed(11)
    lw = {n: (torch.randn(shape, generator=gen) / shape[1] ** 0.5).half().to(dev)
          for n, shape in (("q_proj", (4096, 4096)), ("k_proj", (4096, 4096)), ("v_proj", (4096, 4096)),
                           ("o_proj", (4096, 4096)), ("gate_proj", (11008, 4096)), ("up_proj", (11008, 4096)),
                           ("down_proj", (4096, 11008)))}
    layer_fig = {}
    xs = torch.randn(1, M, 4096, generator=gen).half().to(dev)
    cos, sin = rotary_tables(torch.arange(M, device=dev), 128)
    with torch.no_grad():
        for label, fused_form, six in (("module_by_module", False, False), ("fused", True, False),
                                       ("fused,6bit_matrix_instruction", True, True)):
            layer = W4A4DecoderLayer.from_float(lw, 32, 32, fused=fused_form, six_bit=six)
            layer_fig[f"prefill_T={M},{label}_us"] = round(wall_us(lambda: layer(xs, cos, sin), reps=20), 1)
            if six:
                del layer
                continue
            _, cache = layer(xs[:, :M - 1], cos[:M - 1], sin[:M - 1])
            layer_fig[f"decode_T=1,past={M - 1},{label}_eager_us"] = round(
                wall_us(lambda: layer(xs[:, M - 1:], cos[M - 1:], sin[M - 1:], cache), reps=50), 1)
            del layer, cache
    # ... and the per-token configuration (whole-row online rotation, per-channel weight scales) of the same layer at
    # batch 8 x 512 tokens
    xs8 = torch.randn(8, 512, 4096, generator=gen).half().to(dev)
    cos8, sin8 = rotary_tables(torch.arange(512, device=dev), 128)
    with torch.no_grad():
        for label, fused_form in (("module_by_module", False), ("fused", True)):
            layer = W4A4DecoderLayer.from_float(lw, 32, 32, fused=fused_form, activation="token")
            layer_fig[f"token_configuration,prefill_8x512,{label}_us"] = round(wall_us(lambda: layer(xs8, cos8, sin8), reps=20), 1)
            if fused_form:
                # ... with the rows of 4096 channels rotated on the matrix cores (the headline's rotation mode; the
                # default keeps the bit-exact float32 butterflies in the layer)
                layer.fast_rotation = True
                layer_fig["token_configuration,prefill_8x512,fused,matrix_core_rotation_us"] = round(
                    wall_us(lambda: layer(xs8, cos8, sin8), reps=20), 1)
                # ... and with the seven linears on the 6-bit matrix instruction as well (a second encoding of the weights)
                layer.set_six_bit(True)
                layer_fig["token_configuration,prefill_8x512,fused,matrix_core_rotation,6bit_matrix_instruction_us"] = round(
                    wall_us(lambda: layer(xs8, cos8, sin8), reps=20), 1)
            del layer
    del lw, xs, xs8
    # the causal attention kernel of the prefill path alone, beside torch's fused attention on the same tensors
    attn_fig = {}
    for (ab, at, ahq, ahkv) in ((8, 512, 32, 32), (1, 2048, 32, 32), (1, 2048, 32, 8)):
        aq = torch.randn(ab, at, ahq, 128, generator=gen).half().to(dev)
        ak = torch.randn(ab, ahkv, at, 128, generator=gen).half().to(dev)
        av = torch.randn(ab, ahkv, at, 128, generator=gen).half().to(dev)
        aqt = aq.transpose(1, 2)
        us_own = timed([lambda: ops.prefill_attention(aq, ak, av, 0)] * 20)
        us_torch = timed([lambda: torch.nn.functional.scaled_dot_product_attention(aqt, ak, av, is_causal=True,
                                                                                   enable_gqa=ahq != ahkv)] * 20)
        flops = 4 * ab * ahq * at * at * 128 / 2
        attn_fig[f"{ab}x{at}_tokens,{ahq}/{ahkv}_heads"] = {"us": round(us_own, 1), "TFLOP/s": round(flops / us_own / 1e6, 1),
                                                         "torch_fused_attention_us": round(us_torch, 1)}
        del aq, ak, av, aqt
    layer_fig["prefill_attention_kernel"] = attn_fig

    # The Llama-3-8B decode step (32 layers, batch x 1 token, attention over 2048 cached positions, grouped queries 32 / 8,
    # intermediate 14336 with the 28 x 512 online rotation, group-of-128 weight scales, fp16 head of 128 256 rows), random
    # weights, captured into one graph and replayed.  The int4 linears and their quantisers (with the norms, residual
    # additions and SiLU inside), the rotary embedding, the cache write and attention are this library's kernels; the
    # embedding, the final norm and the fp16 head are torch's.  "everything else" = whole step minus the same step's
    # linears-and-quantisers graph.  Lower bound of the step:
    # all int4 weights and scales + the fp16 head + the cached keys / values once over HBM.
    from flh_amd.quantized_model import LlamaShape, W4A4LlamaModel
    decode_model = {}
    if not args.no_decode_model:
        shape5 = LlamaShape.llama3_8b(num_layers=32)
        with torch.no_grad():
            model5 = W4A4LlamaModel.random_init(shape5, activation="token", weight_group_size=128, fused=True, seed=1)
        w_bytes = 32 * int(sum(n * k // 2 + n * (k // 128) * 2 for _, n, k, _ in L3))
        head_bytes = shape5.vocab_size * shape5.hidden_size * 2
        for batch in (1, 8, 16):
            kv_bytes = 32 * 2 * batch * shape5.num_kv_heads * 2048 * shape5.head_dim * 2
            graph5, st5 = model5.capture_decode_step(batch, 2048)
            for i in range(32):
                st5["cache"].keys[i].normal_()
                st5["cache"].values[i].normal_()
            ms = wall_us(graph5.replay, reps=30) / 1e3
            bound_ms = (w_bytes + head_bytes + kv_bytes) / (PEAK_HBM_GBS * 1e9) * 1e3
            # the linears (and their quantisers) of the same step alone, as a graph over the model's own modules
            xb5 = torch.randn(batch, 4096, dtype=torch.float16, device=dev)
            xb5b = torch.randn(batch, 4096, dtype=torch.float16, device=dev)

            def linears_only():
                for layer in model5.layers:
                    nw = layer._norm_weight16("input_layernorm", layer.input_layernorm)
                    if batch <= 2:      # residual addition, norm, quantiser and q / k / v in one launch
                        qkv = [layer.q_proj, layer.k_proj, layer.v_proj]
                        ops.rmsnorm_rotate_quantize_gemm_i4_multi(
                            xb5, xb5b, nw, 1e-5, [l.w_packed.view(l.out_features, l.in_features // 2) for l in qkv],
                            [l.w_scale.view(l.out_features, -1) for l in qkv])
                    else:
                        _, q5, s5 = ops.add_rmsnorm_rotate_and_quantize_i4(xb5, xb5b, nw, 1e-5)
                        LinearFLH.forward_many([layer.q_proj, layer.k_proj, layer.v_proj], q5, s5)
                    if batch <= 2:
                        layer.o_proj.forward_online(xb5, hadamard="exact")
                    else:
                        q5, s5 = ops.rotate_and_quantize_i4(xb5, hadamard="exact")
                        layer.o_proj(q5, s5, None, x_is_packed=True)
                    _, q5, s5 = ops.add_rmsnorm_rotate_and_quantize_i4(xb5, xb5b, nw, 1e-5)
                    g5, u5 = LinearFLH.forward_many([layer.gate_proj, layer.up_proj], q5, s5)
                    q5, s5 = ops.silu_mul_rotate_and_quantize_i4(g5, u5)
                    layer.down_proj(q5, s5, None, x_is_packed=True)

            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side), torch.no_grad():
                linears_only()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph_l = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph_l), torch.no_grad():
                linears_only()
            ms_lin = wall_us(graph_l.replay, reps=30) / 1e3
            decode_model[f"batch={batch}"] = {
                "ms_per_step_graph_replay": round(ms, 3), "hbm_lower_bound_ms": round(bound_ms, 3),
                "frac_of_bound": round(bound_ms / ms, 4),
                "linears_and_quantisers_ms": round(ms_lin, 3), "everything_else_ms": round(ms - ms_lin, 3),
                "linears_GB/s": round(w_bytes / (ms_lin * 1e-3) / 1e9, 1),
                "linears_frac_hbm": round(w_bytes / (ms_lin * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                "bytes": {"int4_weights_and_scales": w_bytes, "fp16_head": head_bytes, "kv_cache_read": kv_bytes}}
            del graph5, st5, graph_l
        del model5

    # the same linears at the other token counts of the configuration: decode (weight streaming,
    # judged against HBM bandwidth) and a short prefill
    small = {}
    for m_small in (1, 16, 256):
        xq = {k: torch.randint(0, 256, (m_small, k // 2), dtype=torch.uint8, device=dev) for k in (4096, 11008)}
        xs = torch.full((m_small, 1), 0.05, dtype=torch.float16, device=dev)
        row = {}
        for name, n, k in (("qkvo", 4096, 4096), ("gate_up", 11008, 4096), ("down", 4096, 11008)):
            w, ws = weights["q" if name == "qkvo" else "gate" if name == "gate_up" else "down"]
            us = timed([lambda: ops.gemm_i4_dequant_o16(xq[k], w, xs, ws)] * 20)
            byts = n * k // 2 + m_small * k // 2 + 2 * m_small * n + 2 * (n + m_small)
            row[f"{n}x{k}"] = {"us": round(us, 2), "TOPS": round(gemm_ops(m_small, n, k) / (us * 1e-6) / 1e12, 2),
                               "GB/s": round(byts / (us * 1e-6) / 1e9, 1),
                               "frac_hbm": round(byts / (us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4)}
        small[f"M={m_small}"] = row

    # calibration, not product: the vendor library's int8 GEMM (hipBLASLt through torch._int_mm: int8 operands,
    # int32 output, no nibble unpacking and no dequantisation) and fp16 GEMM on the same shapes, as a measure
    # of what fraction of the nominal matrix-core peak a tuned GEMM sustains on this device at these sizes
    # Diagnostic, not product: the q / k / v-sized launch on operands of less switching activity.  The part is at its power
    # limit under this kernel (rocm-smi reads the cap, 1400 W, and a lowered engine clock), and how fast it runs depends on
    # how many operand bits toggle: all-zero codes run at the full 2400 MHz and show what the kernel's structure alone
    # allows, a zero in every other code lies in between; codes quantised from normal data run within 2 % of uniform
    # random ones.  The launch takes the same number of engine cycles in all three cases (counter run in profiles/).
    n_act, k_act = 12288, 4096
    activity = operand_activity(torch, ops, M, 20, True)["cases"]   # time, engine clock and socket power per case
    vendor = None
    if not args.no_vendor_reference:
        vendor = {}
        for n, k in ((4096, 4096), (11008, 4096), (4096, 11008)):
            a8 = torch.randint(-8, 8, (M, k), dtype=torch.int8, device=dev)
            b8 = torch.randint(-8, 8, (n, k), dtype=torch.int8, device=dev).t()
            a16, b16 = a8.to(torch.float16), b8.to(torch.float16)
            try:
                torch._int_mm(a8, b8)
                us8 = timed([lambda: torch._int_mm(a8, b8)] * 20)
            except Exception as exc:  # noqa: BLE001 -- the calibration is optional
                us8 = None
                vendor["int8_error"] = repr(exc)[:120]
            torch.matmul(a16, b16)
            us16 = timed([lambda: torch.matmul(a16, b16)] * 20)
            vendor[f"{M}x{n}x{k}"] = {
                "int8_us": round(us8, 2) if us8 else None,
                "int8_TOPS": round(gemm_ops(M, n, k) / (us8 * 1e-6) / 1e12, 1) if us8 else None,
                "fp16_us": round(us16, 2), "fp16_TFLOPS": round(gemm_ops(M, n, k) / (us16 * 1e-6) / 1e12, 1)}
            del a8, b8, a16, b16

    # The step's four GEMM launches on weights that come from HBM: every launch takes the next of several sets of random
    # weights, more bytes in all than the 256 MB last-level cache holds (the state a model's layers are in), beside the
    # same launch on one set launched back to back (cached).  int8 kernel, 6-bit kernel with its automatic tile, and the
    # 6-bit kernel's 128 x 128 tile forced (flh_gemm_set_tuning, the tests' hook).
    cold_w = {}
    a4q, a4s = ops.rotate_and_quantize_i4(acts["attn_in"], hadamard=had_mode(4096))
    a11q, a11s = ops.rotate_and_quantize_i4(acts["mlp_mid"], hadamard=had_mode(11008))
    a4q6, a11q6 = ops.encode_f6(a4q), ops.encode_f6(a11q)
    sc4 = (torch.rand(4096, 1, device=dev) * 0.015 + 0.005).half()
    sc11 = (torch.rand(11008, 1, device=dev) * 0.015 + 0.005).half()

    def cycle_us(run, sets, reps=36):
        at = [0]

        def once():
            at[0] = (at[0] + 1) % len(sets)
            run(sets[at[0]])
        for _ in range(40):
            once()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                once()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / reps
            best = us if best is None else min(best, us)
        return best

    rand_w = lambda n, k: torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev)
    for name, copies, shapes, k in (("qkv_one_launch", 10, [(4096, 4096)] * 3, 4096), ("o", 30, [(4096, 4096)], 4096),
                                    ("gate_up_swiglu", 6, [(11008, 4096)] * 2, 4096), ("down", 10, [(4096, 11008)], 11008)):
        sets8 = [[rand_w(n, kk) for n, kk in shapes] for _ in range(copies)]
        sets6 = [[ops.encode_f6(w) for w in ws] for ws in sets8]
        aq, a_s, aq6 = (a4q, a4s, a4q6) if k == 4096 else (a11q, a11s, a11q6)
        scs = [sc11 if n == 11008 else sc4 for n, _ in shapes]
        if name == "gate_up_swiglu":
            run8 = lambda ws: ops.gemm_i4_swiglu(aq, ws[0], ws[1], a_s, scs[0], scs[1])
            run6 = lambda ws: ops.gemm_f6_swiglu(aq6, ws[0], ws[1], a_s, scs[0], scs[1])
        elif len(shapes) > 1:
            run8 = lambda ws: ops.gemm_i4_dequant_multi(aq, ws, a_s, scs, -1)
            run6 = lambda ws: ops.gemm_f6_dequant_multi(aq6, ws, a_s, scs)
        else:
            run8 = lambda ws: ops.gemm_i4_dequant_o16(aq, ws[0], a_s, scs[0])
            run6 = lambda ws: ops.gemm_f6_dequant_o16(aq6, ws[0], a_s, scs[0])
        fig = {"int8_us": round(cycle_us(run8, sets8), 1), "int8_cached_us": round(cycle_us(run8, sets8[:1]), 1),
               "six_bit_us": round(cycle_us(run6, sets6), 1), "six_bit_cached_us": round(cycle_us(run6, sets6[:1]), 1)}
        ops.gemm_set_tuning(128, 0)
        fig["six_bit_128x128_tile_us"] = round(cycle_us(run6, sets6), 1)
        fig["six_bit_128x128_tile_cached_us"] = round(cycle_us(run6, sets6[:1]), 1)
        ops.gemm_set_tuning(0, 0)
        fig["weight_sets"] = copies
        cold_w[name] = fig
        del sets8, sets6
    del a4q6, a11q6

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.bitwise_not(src, out=dst)      # its own kernel name: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    traffic = measured_traffic()
    copy_cold = cold[f"K=4096,M={M}"]["device_copy"]
    total_ops = sum(gemm_ops(M, n, k) for _, n, k, _ in LAYERS)
    launches = FORMS[args.launches]
    gemm_us = sum(med[("gemm", name)] for name, *_ in launches)
    gemm_tops = total_ops / (gemm_us * 1e-6) / 1e12

    def launch_table(form, m):
        out = {}
        for name, _, parts in FORMS[form]:
            o = sum(gemm_ops(M, *shape_of[n]) for n in parts)
            out[name] = {"us": round(m[("gemm", name)], 2), "TOPS": round(o / (m[("gemm", name)] * 1e-6) / 1e12, 1)}
        return out
    other_us = sum(med_other[("gemm", name)] for name, *_ in FORMS[other_form])
    quant_detail = {}
    for name, k in SOURCES.items():
        us = med[("quant", name)]
        quant_detail[f"K={k}:{name}"] = {"us": round(us, 2), "GB/s": round(quant_bytes(M, k) / (us * 1e-6) / 1e9, 1)}
    q4096_us = float(np.mean([med[("quant", n)] for n, k in SOURCES.items() if k == 4096]))
    q4096_gbs = quant_bytes(M, 4096) / (q4096_us * 1e-6) / 1e9

    result = {
        "metric": "int4 GEMM+dequant TOPS (Llama-2-7B linears incl. online Hadamard-quant)",
        "value": round(total_ops / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 codes on int8 MFMA, int32 accumulate, fp32/fp16 epilogue",
        "data": "synthetic",
        "config": {"workload": "Llama-2-7B decoder-block linears, M=2048, per-token x per-channel scales "
                               "(the configuration the headline metric is quoted on)", "tokens": M,
                   "launches": args.launches, "hadamard": args.hadamard,
                   "notes": ("the step is issued as a decoder layer issues it: " +
                             ("FOUR GEMM launches for the seven contractions (q/k/v as three weight matrices of one launch; "
                              "gate and up as one launch that stores silu(gate)*up instead of the two fp16 outputs), "
                              if args.launches == "layer" else "one GEMM launch per linear, ") +
                             f"rotation mode '{args.hadamard}' ('fast' = matrix cores; its code mismatch rates against the "
                             "exactly rounded transform are reported in roofline_hadamard_quant), and every timed region "
                             "starts at steady clocks (sustained GEMMs until a batch stops getting faster, then --warmup "
                             "steps).  The form comparable with one-launch-per-linear figures is 'launches=seven', "
                             "reported beside this one.  The headline runs on the int8 matrix instruction; the same step "
                             "on the 6-bit one (bit-identical outputs, a second encoding of the weights) is "
                             "gemm_on_6bit_matrix_instruction.step_in_layer_form.")},
        "roofline": {"bound": "mfma",
                     "kernel": "gemm_i4_kernel (row-scale epilogue), " +
                               ("4 launches per step: q/k/v in one, o, gate and up in one (stores silu(gate)*up), down"
                                if args.launches == "layer" else "7 launches per step"),
                     "achieved": round(gemm_tops, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": round(gemm_tops / PEAK_INT8_TOPS, 4),
                     # HBM bytes per launch averaged over the seven launches (rocprofv3 --pmc FETCH_SIZE and
                     # WRITE_SIZE runs of this script, calibrated on a 256 MiB copy; summary under profiles/)
                     "traffic": traffic["gemm"][args.launches] if (traffic and M == 2048) else None,
                     "avg_launch_us": round(gemm_us / len(launches), 2),
                     "per_launch": launch_table(args.launches, med),
                     # what the part clocks at under this load, and the fraction of the peak at that clock
                     "engine_MHz_under_gemm_load": sclk,
                     "frac_of_peak_at_that_clock": (round(gemm_tops / (PEAK_INT8_TOPS * sclk / 2400.0), 4) if sclk else None),
                     },
        f"launches={other_form}": {"us_per_layer": round(ms_other * 1e3, 1),
                                   "TOPS": round(total_ops / (ms_other * 1e-3) / 1e12, 2),
                                   "gemm_TOP/s": round(total_ops / (other_us * 1e-6) / 1e12, 1),
                                   "gemm_frac_of_peak": round(total_ops / (other_us * 1e-6) / 1e12 / PEAK_INT8_TOPS, 4),
                                   "per_launch": launch_table(other_form, med_other)},
        "roofline_hadamard_quant": {"bound": "hbm",
                                    "kernel": ("rotate_quant_mfma4096_kernel" if had_mode(4096) == "fast" else
                                               "rotate_quant_wave_kernel<8>") + f" (K=4096, M={M}, inside the step)",
                                    "achieved": round(q4096_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                    "frac": round(q4096_gbs / PEAK_HBM_GBS, 4),
                                    # what a plain device copy of the same rows reaches on this box in this run (cold
                                    # inputs, graph replays: no host gaps): the practical ceiling of a streaming launch
                                    # of this size, and the same kernel's own cold figure against it
                                    "practical_peak_GB/s": copy_cold["GB/s"],
                                    "frac_of_practical_peak": round(q4096_gbs / copy_cold["GB/s"], 4),
                                    "cold_launch_frac_of_practical_peak": round(
                                        cold[f"K=4096,M={M}"]["fast" if had_mode(4096) == "fast" else "exact"]["GB/s"] / copy_cold["GB/s"], 4),
                                    f"K=4096,M={ML},cold_frac_of_practical_peak": round(
                                        cold[f"K=4096,M={ML}"]["fast" if had_mode(4096) == "fast" else "exact"]["GB/s"] /
                                        cold[f"K=4096,M={ML}"]["device_copy"]["GB/s"], 4),
                                    "note": "per-launch HIP events around a 7 us kernel also time about 2 us of dispatch: the "
                                            "profiler's duration of these same launches is 7.2-7.5 us (profiles/)",
                                    "traffic": traffic["rotate_quant_K4096"] if (traffic and M == 2048) else None,
                                    "avg_launch_us": round(q4096_us, 2), "per_launch": quant_detail,
                                    "hadamard_mode": args.hadamard, "modes_alone": modes,
                                    f"K=4096,M={ML}": large, "cold_inputs_K=4096": cold,
                                    "device_copy_of_the_same_rows": same_size_copy,
                                    "group_kernels_G=128,K=4096": group, "fused_prologues_G=128": fused},
        "gemm_other_token_counts": small,
        "gemm_on_6bit_matrix_instruction": f6,
        "decode_step_M=1": decode,
        "decoder_layer_llama2_7b": layer_fig,
        "llama3_8b_decode_step_32_layers,kv_len=2048": decode_model,
        f"llama3_8b_block_M={M},weight_groups_of_128": llama3,
        "llama3_8b_decode_linears,weight_groups_of_128": llama3_decode,
        "vendor_gemm_reference": vendor,
        "gemm_launches_on_weights_from_hbm": cold_w,
        f"gemm_{n_act}x{k_act}_by_operand_activity": activity,
        "us_per_layer": round(ms_per_step * 1e3, 1),
        "shared_activation_launches": {"us_per_layer": round(ms_shared * 1e3, 1),
                                       "TOPS": round(sum(gemm_ops(M, n, k) for _, n, k, _ in LAYERS) / (ms_shared * 1e-3) / 1e12, 2),
                                       "launches": "4 rotate-quantise + 4 GEMM; q/k/v and gate/up as several weight "
                                                   "matrices of one launch, weights stored separately",
                                       "equal_to_separate_launches": bool(shared_equal)},
        "gate_up_swiglu_in_one_launch": swiglu,
        "concatenated_qkv_gate_up": {"us_per_layer": round(ms_concat * 1e3, 1),
                                     "TOPS": round(total_ops / (ms_concat * 1e-3) / 1e12, 2),
                                     "launches": "4 rotate-quantise + 4 GEMM (N = 12288, 4096, 22016, 4096)"},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.cpu_sample_tokens)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
