#!/usr/bin/env python3
"""Benchmark of the routed-expert layer (pack -> grouped SwiGLU FFN -> combine).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c4|c1|c2]

One "step" is one ek_layer_forward over one synthetic batch whose inputs and
weights are already resident in HBM, enqueued on a non-default stream.  Prints
ONE JSON line: whole-job token-expert pairs/s of the decode configuration the
metric is quoted on (c3), the roofline of its dominant kernel (per-phase HIP
events recorded on the launch stream inside the timed region), `parity` (the
CPU oracle's output gate on the timed input, sampled tokens), `prefill` (the
8192-token configuration c4 measured on the same experts in the same run, with
its MFMA roofline and a CPU baseline of its own), `c1` / `c2` / `c5` (the other
three benchmark configurations, each built, gated, timed and freed in turn: time
per call, pairs/s, the roof that binds and the fraction reached), `peaks` (copy /
non-temporal read / MFMA ceilings measured by the library's microkernels) and
`cpu_baseline` (the reference-equivalent CPU backend timed on this box's host
cores on a bounded sample of the workload).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "expert-kit_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK = 8.0e12        # B/s, MI355X HBM3E
MFMA_PEAK_16 = 2.5e15    # FLOP/s, bf16/fp16 dense


def measured_traffic(workload: str, stage: int, decode: bool):
    """HBM bytes per launch of the dominant kernel, from the committed rocprofv3 --pmc
    summary (FETCH_SIZE + WRITE_SIZE, scaled by a 1 GiB copy): profiles/pmc_traffic.json.
    None when no profile of this workload has been committed."""
    path = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    if not os.path.exists(path):
        return None
    table = json.load(open(path)).get(workload, {})
    # kernel names in the profile end in <..., E, NMAT, ...>: NMAT = 2 is stage 1, 1 is stage 2;
    # the stage's time covers both kernel families, so does its traffic
    tag = "E, 2" if stage == 1 else "E, 1"
    total, seen = 0.0, False
    for name, t in table.items():
        if ("ffn_stream_kernel" in name or "ffn_tile_kernel" in name) and (tag + ",") in name.replace(">", ","):
            total += t["fetch_bytes"] + t["write_bytes"]
            seen = True
    return total if seen else None


def kernel_stage(name: str):
    """(family, stage) of one of the library's FFN kernels from its name as the profiler prints it,
    demangled (`ek::ffn_tile_kernel<..., E, NMAT, ...>`) or not (`..kernelIDF16bLi<WM>ELi<NMAT>E..`):
    NMAT = 2 is stage 1 (up + gate), 1 is stage 2 (down)."""
    import re
    fam = "stream" if "ffn_stream_kernel" in name else "tile" if "ffn_tile_kernel" in name else None
    if fam is None:
        return None, None
    m = re.search(r"E, (\d),", name.replace(">", ",")) or re.search(r"Li\d+ELi(\d)E", name)
    return fam, (1 if m and m.group(1) == "2" else 2 if m else None)


def live_traffic(n_calls: int):
    """HBM traffic of the FFN kernels measured in this run: two child runs of this file (the decode
    configuration and, on the same experts, the prefill configuration, 3 timed calls each) under
    `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`, each counter scaled by what it reads for a
    1 GiB device copy launched in the same child.  Returns {"c3": {stage: bytes}, "c4": {...}} (both
    kernel families of a stage added up, mean per call) or None when the profiler is not there or a
    child fails; never raises."""
    import collections, csv, glob, shutil, subprocess, tempfile
    if shutil.which("rocprofv3") is None:
        return None
    per = {}
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            d = tempfile.mkdtemp(prefix="ek_pmc_", dir="/tmp")
            cmd = ["timeout", "-s", "KILL", "170", "rocprofv3", "--pmc", counter, "-d", d, "-o", "p", "--output-format", "csv",
                   "--", sys.executable, os.path.abspath(__file__), "--workload", "c3", "--steps", "3", "--warmup", "1",
                   "--cpu-experts", "0", "--no-parity", "--no-peaks", "--no-live-traffic", "--calib-copy-mib", "1024"]
            r = subprocess.run(cmd, cwd="/tmp", env={**os.environ, "TMPDIR": "/tmp"}, stdout=subprocess.DEVNULL,
                               stderr=subprocess.DEVNULL, timeout=200)
            files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
            if r.returncode != 0 or not files:
                if os.environ.get("EK_BENCH_DEBUG"): print("live_traffic: child rc", r.returncode, "files", files, file=sys.stderr)
                shutil.rmtree(d, ignore_errors=True)
                return None
            rows = [x for x in csv.DictReader(open(files[0])) if x["Counter_Name"] == counter]
            shutil.rmtree(d, ignore_errors=True)
            copies = [float(x["Counter_Value"]) for x in rows if "copyBuffer" in x["Kernel_Name"]]
            if not copies:
                if os.environ.get("EK_BENCH_DEBUG"): print("live_traffic: no copy kernel among", sorted(set(x["Kernel_Name"][:40] for x in rows)), file=sys.stderr)
                return None
            unit = 1048576.0 * 1024.0 / max(copies)                     # bytes per counter unit: a 1 GiB copy reads and writes 1 GiB
            # the child launches the calibration copy (three dispatches) before each configuration's calls:
            # the decode configuration's kernels lie between the two groups of copies, the prefill
            # configuration's after the second
            # (the 1 GiB copies stand out by their size among the small copies of weight loading)
            copy_ids = sorted(int(x["Dispatch_Id"]) for x in rows
                              if "copyBuffer" in x["Kernel_Name"] and float(x["Counter_Value"]) > 0.5 * max(copies))
            if len(copy_ids) != 6:
                if os.environ.get("EK_BENCH_DEBUG"): print("live_traffic: calibration copies", copy_ids, file=sys.stderr)
                return None
            for x in rows:
                fam, stage = kernel_stage(x["Kernel_Name"])
                did = int(x["Dispatch_Id"])
                if stage is None or did < copy_ids[2]:
                    continue
                cfg = "c3" if did < copy_ids[3] else "c4"
                c = per.setdefault(cfg, {}).setdefault(stage, {})
                c[counter] = c.get(counter, 0.0) + float(x["Counter_Value"]) * unit / n_calls
        return {cfg: {st: sum(c.values()) for st, c in stages.items() if len(c) == 2} for cfg, stages in per.items()}
    except Exception:
        return None


def cpu_baseline(w, ws_sample, x, ids, gw, target_s=12.0, max_runs=15):
    """Reference-equivalent CPU backend (libtorch ops of ffn/expert_torch.rs:81-84,
    grouped per expert, weighted sum of qwen3_moe.py:102-104) on the pairs routed to
    a sample of experts; weights pre-cast to the compute dtype as load_module does."""
    import torch
    from oracle import oracle
    E = w.n_experts
    wu, wg, wd = [None] * E, [None] * E, [None] * E
    for e, ew in ws_sample.items():
        if w.fp8_block:
            def blk(t, sc):     # w8a16_activate's arithmetic: fp32 product, one rounding
                full = sc.repeat_interleave(128, 0)[:t.shape[0]].repeat_interleave(128, 1)[:, :t.shape[1]]
                return (t.float() * full).to(w.act_dtype)
            wu[e], wg[e], wd[e] = blk(ew.up_w, ew.up_scale), blk(ew.gate_w, ew.gate_scale), blk(ew.down_w, ew.down_scale)
        elif w.w8:
            wu[e] = oracle.torch_dequant_channel(ew.up_w, ew.up_scale)
            wg[e] = oracle.torch_dequant_channel(ew.gate_w, ew.gate_scale)
            wd[e] = oracle.torch_dequant_channel(ew.down_w, ew.down_scale)
        else:
            wu[e], wg[e], wd[e] = ew.up_w.cpu(), ew.gate_w.cpu(), ew.down_w.cpu()
    sample = set(ws_sample)
    times, pairs = [], 0
    t_all = time.time()
    while len(times) < max_runs and (time.time() - t_all < target_s or not times):
        t0 = time.time()
        _, pairs = oracle.torch_layer_forward(x, ids, gw, wu, wg, wd, experts=sample)
        times.append(time.time() - t0)
    med = sorted(times)[len(times) // 2]
    return pairs / med, pairs, len(times)


def calibration_copy(args, dev):
    """A plain device copy of --calib-copy-mib MiB: a kernel of known traffic for the profiler's counters."""
    import torch
    if not args.calib_copy_mib:
        return
    src = torch.empty(args.calib_copy_mib << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def bench_chain(args, w, dev):
    """The ragged continuous-batching mix over n_layers consecutive layers, one hipGraph.
    Returns the JSON object of the run."""
    import torch
    import ek_hip
    from ek_hip import workloads as wl
    layers = []
    for l in range(w.n_layers):
        layer = ek_hip.HipLayer(w.hidden, w.inter, w.n_experts, w.top_k, act_dtype=w.act_dtype,
                                w_dtype=torch.int8 if w.w8 else w.act_dtype, max_tokens=w.tokens)
        for e in range(w.n_experts):
            layer.set_expert(e, wl.make_expert(w, e, layer=l, device="cuda"))
        layers.append(layer)
    routing = [wl.make_routing(w, layer=l) for l in range(w.n_layers)]
    ids = torch.stack([r[0] for r in routing]).to(dev)
    gw = torch.stack([r[1] for r in routing]).to(dev)
    xd = wl.make_x(w).to(dev)
    y = torch.empty_like(xd)
    chain = ek_hip.HipChain(layers)
    stream = torch.cuda.Stream()          # enqueue-only calls on a stream of the caller's
    # gates on the timed input: the first layer's routing tables against a CPU stable sort, its output
    # on sampled tokens against the oracle (the later layers' inputs are the library's own outputs)
    x0 = wl.make_x(w)
    w0 = w
    y0, rt0 = layers[0].forward(xd, ids[0].contiguous(), gw[0].contiguous(), return_route=True)
    assert torch.equal(rt0.perm.cpu(), torch.argsort(routing[0][0].reshape(-1).long(), stable=True).to(torch.int32)), \
        "routing permutation mismatch"
    parity = None
    if args.parity:
        from dataclasses import replace
        parity = parity_on_timed_input(replace(w0, n_layers=1), xd, routing[0][0], routing[0][1], y0, x0)
    y_eager = chain.forward(xd, ids, gw, use_graph=False).clone()
    calibration_copy(args, dev)
    res = {}
    for mode, use_graph in (("eager", False), ("graph", True)):
        for _ in range(args.warmup):
            chain.forward(xd, ids, gw, use_graph=use_graph, stream=stream, out=y)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record(stream)
        for _ in range(args.steps):
            chain.forward(xd, ids, gw, use_graph=use_graph, stream=stream, out=y)
        ev1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        res[mode] = max(time.perf_counter() - t0, ev0.elapsed_time(ev1) * 1e-3) / args.steps
        assert torch.equal(y.view(torch.int16), y_eager.view(torch.int16)), f"{mode} chain output changed"
    step_s = res["graph"]
    pairs = w.pairs * w.n_layers
    counts = [torch.bincount(r[0].reshape(-1).long(), minlength=w.n_experts) for r in routing]
    b = sum(wl.algorithmic_bytes(w, c) for c in counts)
    f = pairs * w.flops_per_pair()
    out = {
        "metric": "token-expert pairs/s on 1 MI355X (DSv3 W8A16 layer); % HBM / MFMA roofline",
        "value": pairs / step_s, "unit": "pairs/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": step_s * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"bfloat16": "bf16", "float16": "f16"}[str(w.act_dtype).replace("torch.", "")], "data": "synthetic",
        "config": {"workload": w.name, "hidden": w.hidden, "moe_intermediate": w.inter, "experts": w.n_experts,
                   "top_k": w.top_k, "tokens": w.tokens, "pairs_per_layer": w.pairs, "layers": w.n_layers,
                   "requests": len(wl.request_lengths()), "zipf_s": w.zipf_s, "launch": "one hipGraph per chain"},
        "roofline": {"bound": "mfma" if f / MFMA_PEAK_16 > b / HBM_PEAK else "hbm",
                     "achieved": f / step_s / 1e12, "peak": MFMA_PEAK_16 / 1e12, "unit": "TFLOP/s",
                     "frac": f / step_s / MFMA_PEAK_16, "traffic": None, "kernel": "whole chain"},
        "layer": {"algorithmic_bytes": b, "algorithmic_flops": f, "hbm_frac": b / step_s / HBM_PEAK,
                  "mfma_frac": f / step_s / MFMA_PEAK_16, "eager_ms_per_step": res["eager"] * 1e3,
                  "graph_ms_per_step": res["graph"] * 1e3},
    }
    if parity is not None:
        out["parity"] = parity
        out["parity"]["of"] = "the first layer's output on the chain's input (later layers consume the library's own outputs)"
    chain.close()
    for layer in layers:
        layer.close()
    return out


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def parity_on_timed_input(w, xd, ids, gw, y, x):
    """The output gate on the very input that is timed: sampled tokens recomputed by the CPU oracle
    (test infrastructure, outside every timed region).  Returns the plain figures; raises if an
    output lies outside 2e-2 * rms plus the storage quanta of the 16-bit tensors."""
    import torch
    from ek_hip import workloads as wl
    from oracle import sampled
    tokens = sampled.choose_tokens(ids, w.n_experts)
    r = sampled.check(y[tokens], x[tokens], ids[tokens], gw[tokens], w.n_experts,
                      lambda e: wl.make_expert(w, e, device="cuda"))      # (the generator gives the loaded weights again)
    ref, y3 = r.pop("ref"), r.pop("y3")
    bits = 7 if w.act_dtype == torch.bfloat16 else 10
    ulp = lambda v: torch.exp2(torch.floor(torch.log2(v.float().abs().clamp_min(1e-30))) - bits)
    rms = float(ref.pow(2).mean().sqrt())
    quanta = 0.5 * ulp(ref) * 1.0001 + ulp((gw[tokens].float().unsqueeze(-1) * y3.float()).abs().amax(dim=1))
    assert bool(((y[tokens].float().cpu() - ref).abs() <= 2e-2 * rms + quanta).all()), f"output parity failed: {r}"
    r["tokens"] = tokens
    r["y_ref"] = "CPU oracle, reference-rounded form before its last storage rounding"
    return r


def time_layer(layer, w, args, dev, stream, graph=False):
    """Parity gates on the workload's input, then warm-up and K timed enqueue-only layer calls on
    `stream` (a stream of the caller's, not the default one).  Returns the measurements."""
    import torch
    from ek_hip import workloads as wl
    ids, gw = wl.make_routing(w)
    counts = torch.bincount(ids.reshape(-1).long(), minlength=w.n_experts)
    x = wl.make_x(w)
    xd, idd, gwd = x.to(dev), ids.to(dev), gw.to(dev)
    y = torch.empty_like(xd)

    # parity gates on this very input: routing tables vs a CPU stable sort, outputs vs the oracle
    y0, rt = layer.forward(xd, idd, gwd, return_route=True)
    ref_perm = torch.argsort(ids.reshape(-1).long(), stable=True).to(torch.int32)
    assert torch.equal(rt.perm.cpu(), ref_perm), "routing permutation mismatch"
    parity = parity_on_timed_input(w, xd, ids, gw, y0, x) if args.parity else None

    torch.cuda.synchronize()
    for _ in range(args.warmup):
        layer.forward(xd, idd, gwd, stream=stream, out=y)
    stream.synchronize()
    torch.cuda.synchronize()
    # per-phase events on every fourth timed call: five event records cost a decode-sized call ~15 us
    # of gaps on the device, which is measurement, not the library
    every = 4 if args.steps >= 8 else 1
    layer.profile(every)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(args.steps):
        layer.forward(xd, idd, gwd, stream=stream, out=y)
    ev1.record(stream)
    stream.synchronize()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_s = ev0.elapsed_time(ev1) * 1e-3
    st = layer.stats()
    layer.profile(False)
    assert torch.equal(y.view(torch.int16), y0.view(torch.int16)), "timed calls changed the output"
    step_s = max(wall, dev_s) / args.steps
    n_prof = max(st["profiled_calls"], 1)
    graph_s = None
    if graph:
        # the same call captured once into a graph of the caller's and replayed: what a serving loop that
        # replays its decode step pays (no launch gaps, no fork / join on the host)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(g, stream=stream):
                layer.forward(xd, idd, gwd, stream=torch.cuda.current_stream(), out=y)
        torch.cuda.synchronize()
        for _ in range(args.warmup):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(args.steps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        graph_s = max(time.perf_counter() - t0, e0.elapsed_time(e1) * 1e-3) / args.steps
        assert torch.equal(y.view(torch.int16), y0.view(torch.int16)), "graph replays changed the output"
        del g
    return {"w": w, "x": x, "ids": ids, "gw": gw, "counts": counts, "step_s": step_s, "dev_s": dev_s / args.steps,
            "k_us": [v / n_prof for v in st["kernel_us"]], "parity": parity, "phase_calls": st["profiled_calls"],
            "graph_s": graph_s}


def decode_sweep(layer, base, dev, stream, token_counts):
    """The decode layer at other batch sizes (uniform routing, as the configuration's): enqueue-only
    calls on `stream` (200 of them up to 8 tokens, 50 up to 64, 30 beyond: ~15-50 ms of device time per
    size), the whole call's algorithmic bytes against the HBM peak.  The routing tables of each size are
    checked against a stable sort first; the timed calls must reproduce that call's output."""
    import torch
    from dataclasses import replace
    from ek_hip import workloads as wl
    rows = []
    for T in token_counts:
        w = replace(base, tokens=T)
        ids, gw = wl.make_routing(w)
        counts = torch.bincount(ids.reshape(-1).long(), minlength=w.n_experts)
        xd, idd, gwd = wl.make_x(w).to(dev), ids.to(dev), gw.to(dev)
        y0, rt = layer.forward(xd, idd, gwd, return_route=True)
        assert torch.equal(rt.perm.cpu(), torch.argsort(ids.reshape(-1).long(), stable=True).to(torch.int32)), T
        y = torch.empty_like(xd)
        calls = 200 if T <= 8 else 50 if T <= 64 else 30
        for _ in range(5):
            layer.forward(xd, idd, gwd, stream=stream, out=y)
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(calls):
            layer.forward(xd, idd, gwd, stream=stream, out=y)
        e1.record(stream)
        stream.synchronize()
        step_s = max(time.perf_counter() - t0, e0.elapsed_time(e1) * 1e-3) / calls
        assert torch.equal(y.view(torch.int16), y0.view(torch.int16)), T
        rows.append({"tokens": T, "calls": calls, "ms_per_step": step_s * 1e3, "pairs_per_s": w.pairs / step_s,
                     "active_experts": int((counts > 0).sum()),
                     "hbm_frac": wl.algorithmic_bytes(w, counts) / step_s / HBM_PEAK})
    return rows


def roofline_of(m):
    """Roofline of the dominant kernel of one measured workload, and the layer-level figures."""
    w, counts, step_s, k_us = m["w"], m["counts"], m["step_s"], m["k_us"]
    from ek_hip import workloads as wl
    active = int((counts > 0).sum())
    wsz = 1 if w.w8 else 2
    a = 2
    # algorithmic bytes of each phase (weights of active experts once, activations in/out once)
    nblk = ((w.inter + 127) // 128) * ((w.hidden + 127) // 128)
    s_ffn1 = 2 * nblk * 4 if w.fp8_block else 2 * w.inter * 2 if w.w8 else 0      # scale bytes per expert and stage
    s_ffn2 = nblk * 4 if w.fp8_block else w.hidden * 2 if w.w8 else 0
    b_ffn1 = active * (2 * w.hidden * w.inter * wsz + s_ffn1) + w.tokens * w.hidden * a + w.pairs * w.inter * a
    b_ffn2 = active * (w.hidden * w.inter * wsz + s_ffn2) + w.pairs * w.inter * a + w.pairs * w.hidden * a
    b_layer = wl.algorithmic_bytes(w, counts)
    f_layer = w.pairs * w.flops_per_pair()
    hbm_frac = b_layer / step_s / HBM_PEAK
    mfma_frac = f_layer / step_s / MFMA_PEAK_16
    dom = 1 if k_us[1] >= k_us[2] else 2
    fam = "ffn_stream_kernel" if hbm_frac >= mfma_frac else "ffn_tile_kernel (+ ffn_stream_kernel for items of <= 16 rows)"
    dom_name = fam + (", stage 1: up/gate + SwiGLU" if dom == 1 else ", stage 2: down")
    dom_bytes = b_ffn1 if dom == 1 else b_ffn2
    dom_flops = w.pairs * (4 if dom == 1 else 2) * w.hidden * w.inter
    dom_s = k_us[dom] * 1e-6
    if hbm_frac >= mfma_frac:
        roof = {"bound": "hbm", "achieved": dom_bytes / dom_s / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                "frac": dom_bytes / dom_s / HBM_PEAK, "traffic": None}
    else:
        roof = {"bound": "mfma", "achieved": dom_flops / dom_s / 1e12, "peak": MFMA_PEAK_16 / 1e12, "unit": "TFLOP/s",
                "frac": dom_flops / dom_s / MFMA_PEAK_16, "traffic": None}
    roof.update({"kernel": dom_name, "kernel_us": k_us[dom], "algorithmic_bytes": dom_bytes,
                 "algorithmic_flops": dom_flops})
    roof["traffic"] = measured_traffic(w.name, dom, decode=hbm_frac >= mfma_frac)
    roof["traffic_source"] = ("profiles/pmc_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, "
                              "committed; not measured in this run") if roof["traffic"] is not None else None
    layer = {"algorithmic_bytes": b_layer, "algorithmic_flops": f_layer, "hbm_frac": hbm_frac, "mfma_frac": mfma_frac,
             "phase_us": {"pack": k_us[0], "ffn_up_gate": k_us[1], "ffn_down": k_us[2], "combine": k_us[3]},
             "phase_events": f"HIP events around the four phases on {m['phase_calls']} of the timed calls (every fourth)",
             "device_ms_per_step": m["dev_s"] * 1e3}
    config = {"workload": w.name, "hidden": w.hidden, "moe_intermediate": w.inter, "experts": w.n_experts,
              "top_k": w.top_k, "tokens": w.tokens, "pairs": w.pairs, "active_experts": active, "zipf_s": w.zipf_s,
              "weights": "fp8 e4m3fn, 128x128 block scales" if w.fp8_block else "int8 per-channel" if w.w8 else "16-bit"}
    return roof, layer, config


def build_layer(w, max_tokens, keep=()):
    """The workload's layer with every expert resident; CPU copies of the experts named in `keep`."""
    import torch
    import ek_hip
    from ek_hip import workloads as wl
    w_dtype = torch.float8_e4m3fn if w.fp8_block else torch.int8 if w.w8 else w.act_dtype
    layer = ek_hip.HipLayer(w.hidden, w.inter, w.n_experts, w.top_k, act_dtype=w.act_dtype, w_dtype=w_dtype,
                            max_tokens=max_tokens)
    kept = {}
    for e in range(w.n_experts):
        ew = wl.make_expert(w, e, device="cuda")
        layer.set_expert(e, ew)
        if e in keep:
            kept[e] = ek_hip.ExpertWeight(*[None if t is None else t.cpu() for t in
                                            (ew.up_w, ew.gate_w, ew.down_w, ew.up_scale, ew.gate_scale, ew.down_scale)])
        del ew
    return layer, kept


def sample_experts(w, n):
    """n experts spread evenly over the workload's experts ordered by load."""
    import torch
    from ek_hip import workloads as wl
    if n <= 0:
        return []
    ids, _ = wl.make_routing(w)
    counts = torch.bincount(ids.reshape(-1).long(), minlength=w.n_experts)
    order = torch.argsort(counts, descending=True, stable=True).tolist()
    return sorted(order[:: max(1, w.n_experts // n)][:n])


def compact(m, roof, layer_fig, config):
    """One of the other configurations as a short object: time, throughput, the roof that binds the whole
    call and the fraction of it reached, the dominant kernel's own fraction, the gates that were held."""
    bound = "hbm" if layer_fig["hbm_frac"] >= layer_fig["mfma_frac"] else "mfma"
    out = {"config": config, "ms_per_step": m["step_s"] * 1e3, "value": m["w"].pairs / m["step_s"], "unit": "pairs/s",
           "bound": bound, "frac": layer_fig[bound + "_frac"], "hbm_frac": layer_fig["hbm_frac"], "mfma_frac": layer_fig["mfma_frac"],
           "dominant_kernel": {"kernel": roof["kernel"], "us": roof["kernel_us"], "frac": roof["frac"], "bound": roof["bound"]},
           "phase_us": layer_fig["phase_us"], "routing_bit_exact": True}
    if m["graph_s"] is not None:
        out["graph_replay_ms_per_step"] = m["graph_s"] * 1e3
        out["graph_replay_frac"] = out["frac"] * m["step_s"] / m["graph_s"]
    if m["parity"] is not None:
        out["parity"] = {k: m["parity"][k] for k in ("max_err_over_rms", "over_frac", "elements", "tokens")}
    return out


def cpu_cores():
    return os.cpu_count() if not os.environ.get("OMP_NUM_THREADS") else int(os.environ["OMP_NUM_THREADS"])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all", choices=["all", "c1", "c2", "c3", "c4", "c5"],
                    help="all (default): c3 as the headline, c4 on the same experts as `prefill`, then c1, c2 and c5 "
                         "as short objects; one name: that configuration alone")
    ap.add_argument("--weights", choices=["config", "fp8", "bf16"], default="config",
                    help="fp8: the c3 / c4 layer with fp8 e4m3fn weights and 128x128 block scales kept as a "
                         "DeepSeek-V3 checkpoint stores them, instead of the configuration's int8 per channel; "
                         "bf16: the same layer with 16-bit weights")
    ap.add_argument("--cpu-experts", type=int, default=96, help="experts in the CPU-baseline sample (0 = skip)")
    ap.add_argument("--cpu-experts-prefill", type=int, default=16,
                    help="experts in the prefill configuration's CPU-baseline sample (0 = skip)")
    ap.add_argument("--tokens", type=int, default=0,
                    help="run the workload's layer at another token count (a parity-test style variation, e.g. other "
                         "decode batch sizes of c3; implies --no-prefill)")
    ap.add_argument("--no-prefill", dest="prefill", action="store_false",
                    help="with --workload c3: do not also measure the c4 prefill call on the same experts")
    ap.add_argument("--no-parity", dest="parity", action="store_false", help="skip the oracle's output gate before timing")
    ap.add_argument("--no-peaks", dest="peaks", action="store_false", help="skip the copy / read / MFMA microbenchmarks")
    ap.add_argument("--graph", action="store_true", help="also time the call replayed from a graph of the caller's")
    ap.add_argument("--no-live-traffic", dest="live_traffic", action="store_false",
                    help="with the default workload: do not measure `roofline.traffic` in this run (two child runs under "
                         "rocprofv3 --pmc); the figure of the committed profile is reported instead, and labelled so")
    ap.add_argument("--no-sweep", dest="sweep", action="store_false",
                    help="with --workload all: skip the decode layer's other batch sizes (decode_sweep)")
    ap.add_argument("--calib-copy-mib", type=int, default=0,
                    help="also launch a plain device copy of this many MiB (a kernel of known traffic, "
                         "used to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import ek_hip
    from ek_hip import workloads as wl
    from dataclasses import replace

    ek_hip.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    everything = args.workload == "all"
    w = wl.resolve(wl.CONFIGS["c3" if everything else args.workload])
    if args.weights == "fp8":
        assert w.w8, "--weights fp8 applies to the W8A16 configurations (c3, c4)"
        w = replace(w, fp8_block=True)
    if args.weights == "bf16":
        assert w.w8, "--weights bf16 applies to the W8A16 configurations (c3, c4)"
        w = replace(w, w8=False)
    if args.tokens > 0:
        assert w.n_layers == 1, "--tokens applies to the single-layer configurations"
        w = replace(w, tokens=args.tokens, name=f"{w.name}_T{args.tokens}")
        args.prefill = False
    if w.n_layers > 1:
        print(json.dumps(bench_chain(args, w, dev)))
        return
    # the decode configuration the metric is quoted on and the prefill configuration hold the same
    # 256 experts: both are measured on one layer object, decode first
    also = None
    if w.name.startswith("c3") and args.prefill:
        also = replace(wl.C4, fp8_block=w.fp8_block, w8=w.w8)
    sample_ids = sample_experts(w, args.cpu_experts)
    sample_ids_p = sample_experts(also, args.cpu_experts_prefill) if also is not None else []
    layer, kept = build_layer(w, max(w.tokens, also.tokens if also else 0), keep=set(sample_ids) | set(sample_ids_p))
    stream = torch.cuda.Stream()          # the calls are enqueue-only on a stream of the caller's
    calibration_copy(args, dev)
    m = time_layer(layer, w, args, dev, stream, graph=args.graph)
    roof, layer_fig, config = roofline_of(m)
    out = {
        "metric": "token-expert pairs/s on 1 MI355X (DSv3 W8A16 layer); % HBM / MFMA roofline",
        "value": w.pairs / m["step_s"], "unit": "pairs/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": m["step_s"] * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        # the type the MFMAs multiply in (int8 weights are dequantised to it in registers); fp32 accumulation
        "dtype": {"bfloat16": "bf16", "float16": "f16"}[str(w.act_dtype).replace("torch.", "")],
        "data": "synthetic",
        "config": config,
        "timed": "enqueue-only ek_layer_forward calls (device pointers) on a non-default stream; HIP events on that stream",
        "roofline": roof,
        "layer": layer_fig,
    }
    if m["graph_s"] is not None:
        out["graph_replay_ms_per_step"] = m["graph_s"] * 1e3
    if m["parity"] is not None:
        out["parity"] = m["parity"]
    if everything and args.sweep:
        out["decode_sweep"] = {"what": f"{w.name}'s layer at other batch sizes, 30 to 200 enqueue-only calls each, whole call against "
                                       "8 TB/s; outputs equal the routing-checked call's bit for bit",
                               "rows": decode_sweep(layer, w, dev, stream, (1, 2, 4, 8, 16, 32, 64, 256, 512))}
    torch.set_num_threads(cpu_cores())
    if also is not None:
        calibration_copy(args, dev)              # (a marker between the two configurations for the profiler's counters)
        mp = time_layer(layer, also, args, dev, stream)
        roof_p, layer_p, config_p = roofline_of(mp)
        out["prefill"] = {"config": config_p, "value": also.pairs / mp["step_s"], "unit": "pairs/s",
                          "ms_per_step": mp["step_s"] * 1e3, "steps": args.steps, "warmup": args.warmup,
                          "roofline": roof_p, "layer": layer_p}
        # the north-star figure of the prefill regime: the whole call's FLOPs against the bf16 dense peak
        out["prefill"]["roofline_whole_call"] = {"bound": "mfma", "achieved": layer_p["algorithmic_flops"] / mp["step_s"] / 1e12,
                                                 "peak": MFMA_PEAK_16 / 1e12, "unit": "TFLOP/s", "frac": layer_p["mfma_frac"]}
        if mp["parity"] is not None:
            out["prefill"]["parity"] = mp["parity"]
        if sample_ids_p:
            v, pairs, iters = cpu_baseline(also, {e: kept[e] for e in sample_ids_p}, mp["x"], mp["ids"], mp["gw"], max_runs=1)
            out["prefill"]["cpu_baseline"] = {
                "value": v, "unit": "pairs/s", "cores": torch.get_num_threads(), "kind": "port", "cpu_model": cpu_model(),
                "sample": f"pairs routed to {len(sample_ids_p)} of {also.n_experts} experts spread evenly over the experts "
                          f"ordered by load ({pairs} of {also.pairs} pairs), one run, libtorch CPU ops, weights pre-cast to "
                          f"{str(also.act_dtype).replace('torch.', '')}"}
    if args.peaks:
        from ek_hip import _capi as C
        import ctypes
        pk = C.ek_peaks()
        C.check(C.load().ek_measure_peaks(0, ctypes.byref(pk)))
        out["peaks"] = {"copy_GBps": pk.copy_gbps, "nontemporal_read_GBps": pk.read_nt_gbps,
                        "mfma_bf16_TFLOPs": pk.mfma_bf16_tflops,
                        "mfma_bf16_random_operands_TFLOPs": pk.mfma_bf16_random_tflops,
                        "mfma_bf16_with_int8_dequant_TFLOPs": pk.mfma_bf16_dequant_tflops,
                        "source": "in-library microkernels (csrc/ek_peaks.hip), measured in this run",
                        "published": {"hbm_GBps": HBM_PEAK / 1e9, "mfma_bf16_TFLOPs": MFMA_PEAK_16 / 1e12}}
    if sample_ids:
        v, pairs, iters = cpu_baseline(w, {e: kept[e] for e in sample_ids}, m["x"], m["ids"], m["gw"])
        out["cpu_baseline"] = {"value": v, "unit": "pairs/s", "cores": torch.get_num_threads(), "kind": "port",
                               "cpu_model": cpu_model(),
                               "sample": f"pairs routed to {len(sample_ids)} of {w.n_experts} experts ({pairs} pairs), "
                                         f"median of {iters} runs, libtorch CPU ops, weights pre-cast to "
                                         f"{str(w.act_dtype).replace('torch.', '')}"}
    layer.close()
    del layer, kept, m
    if everything and args.live_traffic and also is not None:
        # `traffic` of the two dominant kernels measured now, with the GPU otherwise idle
        torch.cuda.empty_cache()
        live = live_traffic(1 + 1 + 3)          # calls per configuration in a child: the gate call, 1 warm-up, 3 timed
        for cfg, roof_x in (("c3", out["roofline"]), ("c4", out["prefill"]["roofline"])):
            stage = 1 if "stage 1" in roof_x["kernel"] else 2
            if live and live.get(cfg, {}).get(stage):
                roof_x["traffic_committed_profile"] = roof_x["traffic"]
                roof_x["traffic"] = live[cfg][stage]
                roof_x["traffic_source"] = ("measured in this run: child runs of this file under rocprofv3 --pmc FETCH_SIZE and "
                                            "--pmc WRITE_SIZE (3 timed calls), each counter scaled by a 1 GiB device copy")
    if everything:
        # the other three configurations, each built, gated, timed and freed in turn
        torch.cuda.empty_cache()
        for name in ("c1", "c2"):
            wo = wl.resolve(wl.CONFIGS[name])
            lo, _ = build_layer(wo, wo.tokens)
            mo = time_layer(lo, wo, args, dev, stream, graph=True)
            out[name] = compact(mo, *roofline_of(mo))
            lo.close()
            del lo, mo
            torch.cuda.empty_cache()
        c5 = bench_chain(args, wl.resolve(wl.CONFIGS["c5"]), dev)
        out["c5"] = {"config": c5["config"], "ms_per_step": c5["ms_per_step"], "value": c5["value"], "unit": "pairs/s",
                     "bound": c5["roofline"]["bound"], "frac": c5["roofline"]["frac"], "hbm_frac": c5["layer"]["hbm_frac"],
                     "mfma_frac": c5["layer"]["mfma_frac"], "eager_ms_per_step": c5["layer"]["eager_ms_per_step"],
                     "graph_equals_eager_bitwise": True, "routing_bit_exact": True}
        if "parity" in c5:
            out["c5"]["parity"] = {k: c5["parity"][k] for k in ("max_err_over_rms", "over_frac", "elements", "tokens", "of")}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
