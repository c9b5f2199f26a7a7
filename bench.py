#!/usr/bin/env python3
"""Headline benchmark: NCN forward + backward of the full stage stack on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg3|cfg2|cfg4|cfg5] [--no-cpu]
                    [--grouping closed|stride-table|radix-table|ragged|radix] [--save-every K] [--scalar-heads]
                    [--no-surface]
    python bench.py --record-traffic <dir>      (turns rocprofv3 counter files into profiles/traffic.json, see there)

One step = forward of all L stages (each stage saving its outputs, like the reference's autograd
node) + reversible backward of all L stages producing dx, dxa and every dW_l, on inputs that are
already resident in HBM.  The default workload is the configuration the metric is quoted on:
B=16384, D=4096, g=16, bf16 storage / float32 arithmetic, i.e. [batch=128, N=4096, E=128],
4 heads of 32, n_cache=16, 3 stages.

Prints ONE JSON line.  `roofline` describes the dominant kernel (the backward stage kernel, or the
backward call over a segment of stages where several stages run per launch) against the roof that binds
it: float32 vector arithmetic for groups of 8 rows and more (each element takes n_cache sequential tanh
steps per stage), HBM bandwidth for smaller groups.  Its duration is measured with HIP events on the
launch stream inside the timed region; the figures for the other roof ride along as hbm_* / valu_*.
`roofline.frac` is against the published peak (157.3 TFLOP/s; 8 TB/s); what this GPU sustains is measured in the
same run and quoted beside it: `attainable_valu_TFLOPs` (a stream of independent v_fma_f32 on vector registers, the
library's ncn_probe_issue; the library is built without packed FP32) and `attainable_copy_GBps` (a 1 GiB device copy).
`stack.autograd_*` time the same workload through the reference's own surface (NCNNetTestCuda + yi.backward(dyi),
grad_test_bench.py:116-134) and through the one-node form of the stack, `stack.graph_ms_per_step` replays the timed
step from a HIP graph; all three outside the headline timed region.
`roofline.traffic` is read from profiles/traffic.json (rocprofv3 FETCH_SIZE + WRITE_SIZE of that kernel,
recorded for one library version) and is null when that file has no entry for this library version.
`cpu_baseline` times the checker's plain C restatement (and, beside it, the PyTorch one) on a bounded
batch slice of the same workload on the host cores.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# config label -> (batch, N, E, n_head, n_cache, L, io dtype, w_scale)   (B = batch*E tokens, D = N, g = n_cache)
CONFIGS = {
    "cfg2": dict(batch=32, N=1024, E=128, C=4, n=4, L=5, dtype="f32", w_scale=1.0),
    "cfg3": dict(batch=128, N=4096, E=128, C=4, n=16, L=3, dtype="bf16", w_scale=1.0),
    "cfg4": dict(batch=128, N=8192, E=128, C=4, n=2, L=13, dtype="f32", w_scale=1.0),
    "cfg5": dict(batch=64, N=2048, E=128, C=4, n=8, L=4, dtype="f32", w_scale=0.1),
}
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
VALU_PEAK_TFLOPS = 157.3   # MI355X FP32 vector peak
# float32 operations per element and step of the kernels as written in ncn_stage_kernels.h (FMA = 2, exp2 and
# rcp = 1 each), without the per-row and per-lane bookkeeping: forward 5 FMA (row sum, z, two for xa, x) + the
# +1 before the reciprocal + exp2 + rcp = 13; backward 12 FMA (inversion of x, row sum, z, two for xa, F'/4, the
# row's <U, x_j>, the pivot row's sum, two for G, dWi, P) + the +1 + P F'/4 + exp2 + rcp = 28.  (Heads of one feature,
# ncn_headwise_kernels.h: the same 13, and 29 with the products that are no longer shared by a row; counted as 28.)
FLOPS_FWD_PER_ELEM_STEP = 13.0
FLOPS_BWD_PER_ELEM_STEP = 28.0
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def traffic_key(config, grouping, scalar_heads=False):
    return f"{config}/{grouping}" + ("/scalar-heads" if scalar_heads else "")


def measured_traffic(config, grouping, version, scalar_heads=False):
    """HBM bytes per launch (or per backward call over a segment) of the dominant kernel, from the profile record of
    this library version; None when there is none."""
    try:
        with open(TRAFFIC_FILE) as fh:
            rec = json.load(fh)
    except (OSError, ValueError):
        return None
    entry = rec.get("entries", {}).get(traffic_key(config, grouping, scalar_heads))
    if not entry or entry.get("ncn_version") != version:
        return None
    return entry.get("bytes")


def record_traffic(prof_dir):
    """Turns the counter files of two rocprofv3 runs of this script into the entry of profiles/traffic.json that
    `roofline.traffic` is read from.  prof_dir holds f/ and w/ (the output directories of
        rocprofv3 --pmc FETCH_SIZE --output-format csv -d <prof_dir>/f -o p -- python3 bench.py --config C --steps 2
                  --warmup 1 --no-cpu --no-surface --copy-probe > <prof_dir>/f.log
    and the same with WRITE_SIZE and w) and the two logs.  Each counter is scaled by what it reads for the 1 GiB copy
    of --copy-probe (1048576 KiB read and written).  The library version, build id and workload of the entry are those
    the profiled runs printed, so an entry can only claim what was measured."""
    import csv
    import glob

    runs = {}
    for d in ("f", "w"):
        with open(os.path.join(prof_dir, d + ".log")) as fh:
            lines = [l for l in fh if l.startswith("{")]
        runs[d] = json.loads(lines[-1])
    meta = runs["f"]
    for key in ("ncn_version", "build_id", "kernel"):
        if runs["w"]["roofline"][key] != meta["roofline"][key]:
            raise SystemExit(f"the two runs disagree on {key}")
    workload = meta["config"]["workload"]
    config = workload.split(":")[0]
    grouping = workload.rsplit("grouping ", 1)[1]
    key = traffic_key(config, grouping, " heads of 1," in workload)
    one_stage = ("stage_backward_kernel", "headwise_backward_kernel")
    steps = meta["steps"] + meta["warmup"]
    per_call = "backward call" in meta["roofline"]["kernel"]
    sizes, factors, names = {}, {}, {}
    for d, counter in (("f", "FETCH_SIZE"), ("w", "WRITE_SIZE")):
        rows = []
        for f in glob.glob(os.path.join(prof_dir, d, "**", "*counter_collection.csv"), recursive=True):
            with open(f) as fh:
                rows += [r for r in csv.DictReader(fh) if r["Counter_Name"] == counter]
        copy = max(float(r["Counter_Value"]) for r in rows if "copyBuffer" in r["Kernel_Name"])
        factors[d] = 1048576.0 / copy
        per_dispatch = {}
        for r in rows:   # one row per dispatch and XCD set: sum what belongs to one dispatch
            if "ncn::" in r["Kernel_Name"]:
                k = (r["Kernel_Name"], r["Dispatch_Id"])
                per_dispatch[k] = per_dispatch.get(k, 0.0) + float(r["Counter_Value"])
        if per_call:    # every backward-side launch of a call (passes, one-stage launches, dW reduction), per call
            mine = {k: v for k, v in per_dispatch.items() if "backward" in k[0] or "reduce_" in k[0]}
            n_calls = steps * meta["config"]["backward_calls_per_step"]
            sizes[d] = sum(mine.values()) / n_calls * factors[d] * 1024.0
            counts = {}
            for (name, _), _v in mine.items():
                counts[name] = counts.get(name, 0) + 1
            short = lambda n: n.replace("(anonymous namespace)::", "").split("(")[0].replace("void ", "")
            names[d] = ", ".join(f"{c / n_calls:g} x {short(n)}" for n, c in sorted(counts.items()))
        else:           # the one-stage backward kernel, per launch
            mine = [v for k, v in per_dispatch.items() if any(o in k[0] for o in one_stage)]
            sizes[d] = sum(mine) / len(mine) * factors[d] * 1024.0
            names[d] = sorted({k[0] for k in per_dispatch if any(o in k[0] for o in one_stage)})[0].split("(")[0].replace("void ", "")
    try:
        with open(TRAFFIC_FILE) as fh:
            rec = json.load(fh)
    except (OSError, ValueError):
        rec = {"entries": {}}
    rec["comment"] = ("HBM bytes per launch (or per backward call over a segment) of the dominant kernel of bench.py, from "
                      "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, written by `python bench.py --record-traffic <dir>` from the "
                      "counter files and logs of the profiled runs; bench.py reports an entry only for the library version "
                      "it was measured on")
    rec["entries"][key] = {
        "ncn_version": meta["roofline"]["ncn_version"], "build_id": meta["roofline"]["build_id"],
        "kernel": names["f"], "bytes": round(sizes["f"] + sizes["w"]), "read_bytes": round(sizes["f"]),
        "written_bytes": round(sizes["w"]), "fetch_size_factor": round(factors["f"], 4),
        "write_size_factor": round(factors["w"], 4), "workload": workload}
    with open(TRAFFIC_FILE, "w") as fh:
        json.dump(rec, fh, indent=1)
        fh.write("\n")
    print(json.dumps(rec["entries"][key]))


def main():
    if len(sys.argv) == 3 and sys.argv[1] == "--record-traffic":
        record_traffic(sys.argv[2])
        return
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="cfg3", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--grouping", default="closed", choices=["closed", "stride-table", "radix-table", "ragged", "lengths", "radix"],
                    help="closed: the stride permutation in closed form (the headline path).  The others go through "
                         "the *_indexed entry points, one call per stage: the same permutation as a table, the "
                         "radix-n digit grouping as a table, or the stride table with one context length per batch "
                         "entry (N - 1 - b mod n_cache live rows).  lengths: the closed-form permutation with the same "
                         "lengths and no table, whole segments per call (multi-stage LDS passes for small groups).  radix: levels 0 .. L-1 of the radix-n digit grouping "
                         "through ncn_forward_radix / ncn_backward_radix (needs n_cache^L to divide N; several levels "
                         "per LDS pass for n_cache 2 and 4; float32 between calls)")
    ap.add_argument("--save-every", type=int, default=0,
                    help="stages per saved checkpoint (0: what the whole-net autograd node chooses, "
                         "modules.default_save_every)")
    ap.add_argument("--scalar-heads", action="store_true",
                    help="the literal scalar reading of x[B, D]: one feature per head (n_head = E), a different shape "
                         "from the one the metric is quoted on; register kernels that hold four heads per lane")
    ap.add_argument("--no-surface", action="store_true",
                    help="skip the legs outside the timed region that go through the autograd surface and a HIP graph")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 1 GiB device copy, so that a rocprofv3 --pmc run has a kernel of known "
                         "traffic to calibrate FETCH_SIZE / WRITE_SIZE against")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the layer shards over batch; "
              "only dW [L,2E] would need an all-reduce). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    from ncn_cuda_amd import ncn_cuda_module as M

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    cfg = CONFIGS[args.config]
    batch, N, E, C, n, L = cfg["batch"], cfg["N"], cfg["E"], cfg["C"], cfg["n"], cfg["L"]
    if args.scalar_heads:
        C = E
    io_dtype = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    alpha = 0.9
    tokens = batch * E
    P = batch * N * E
    sbytes = 2 if cfg["dtype"] == "bf16" else 4

    # synthetic inputs, seeded on the CPU: x ~ N(0,1), xa = 0 (as the reference's script starts it), W_l ~ N(0, 1/g)
    # (times the configuration's scale), upstream gradient ~ N(0,1) on yi only
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(batch, N, E, generator=gen).to(io_dtype)
    xa = torch.zeros(batch, N, E, dtype=io_dtype)
    Ws = [(torch.randn(2 * E, generator=gen) * (cfg["w_scale"] / math.sqrt(n))).to(io_dtype) for _ in range(L)]
    dyi = torch.randn(batch, N, E, generator=gen).to(io_dtype)
    dev = torch.device("cuda:0")
    gx, gxa, gdyi = x.to(dev), xa.to(dev), dyi.to(dev)
    gWs = [w.to(dev) for w in Ws]
    bf16 = io_dtype == torch.bfloat16

    # Stages per saved checkpoint: 1 for the headline shape (every stage saves its outputs, like the reference's
    # autograd node); small groups run whole segments per call (multi-stage LDS passes) and reverse them from the
    # segment's outputs: rounding grows like (1/m)^(n_cache * stages), kept below 16x.
    from ncn_cuda_amd.modules import default_save_every
    save_every = 1   # tables run stage by stage
    if args.grouping in ("closed", "radix", "lengths"):
        save_every = args.save_every if args.save_every > 0 else default_save_every(n, L, batch * N * E)
    tables = lens = None
    if args.grouping == "lengths":   # the closed-form permutation with one context length per batch entry
        lens = (N - 1 - torch.arange(batch, device=dev) % n).to(torch.int32)
    elif args.grouping not in ("closed", "radix"):
        from ncn_cuda_amd import chunk_linear as CL
        if args.grouping == "radix-table":
            levels = 1
            while n ** (levels + 1) <= N and N % n ** (levels + 1) == 0:
                levels += 1
            tables = [CL.radix_group_table(N, n, l % levels, device=dev) for l in range(L)]
        else:
            tables = [CL.stride_group_table(N, n, l, device=dev) for l in range(L)]
        if args.grouping == "ragged":
            lens = (N - 1 - torch.arange(batch, device=dev) % n).to(torch.int32)
    segs = [(a, min(save_every, L - a)) for a in range(0, L, save_every)]
    Wst = torch.stack([w.to(torch.float32) for w in gWs])

    def step(events=None):
        saved = []
        cx, cxa = gx, gxa
        for a, cnt in segs:
            if args.grouping == "radix":
                cx, cxa = M.forward_radix(cx, cxa, Wst[a:a + cnt], alpha, 0, n, C, a, cnt)
                saved.append((cx, cxa))
            elif tables is not None:
                # what the table-grouped autograd node keeps: two bf16 planes for bf16 storage, the outputs otherwise
                cx, cxa, sy, sya = M.forward_stages_saving(cx, cxa, Wst[a], alpha, 0, n, C, a, group_index=tables[a],
                                                           ctx_len=lens, check_tables=False)
                saved.append((sy, sya))
            elif bf16 and cnt == 1:
                # bf16 outputs plus what their rounding took away (a second bf16 plane): what the backward inverts
                # (float32 copies instead where only the generic kernels take the shape)
                cx, cxa, ys, yas = M.forward_stages_saving(cx, cxa, Wst[a], alpha, 0, n, C, a, ctx_len=lens)
                saved.append((ys, yas))
            else:
                cx, cxa = M.forward_stages(cx, cxa, Wst[a:a + cnt], alpha, 0, n, C, a, cnt, out_dtype=torch.float32,
                                           ctx_len=lens)
                saved.append((cx, cxa))
        dy, dya_ = gdyi, None  # the reference script back-propagates through yi only (grad_test_bench.py:121)
        dWs = [None] * len(segs)
        for k in range(len(segs) - 1, -1, -1):
            a, cnt = segs[k]
            if events is not None:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            extra = (dict(group_index=tables[a], ctx_len=lens, check_tables=False) if tables is not None else
                     dict(ctx_len=lens))
            if args.grouping == "radix":
                _, _, dy, dya_, dWs[k] = M.backward_radix(saved[k][0], saved[k][1], dy, dya_, Wst[a:a + cnt], alpha, 0,
                                                          n, C, a, cnt, want_inputs=False)
            else:
                _, _, dy, dya_, dWs[k] = M.backward_stages(saved[k][0], saved[k][1], dy, dya_, Wst[a:a + cnt], alpha,
                                                           0, n, C, a, cnt,
                                                           grad_dtype=io_dtype if cnt == 1 else torch.float32,
                                                           want_inputs=False, **extra)
            if events is not None:
                e1.record()
                events.append((e0, e1, cnt))
        return cx, cxa, dy, dya_, dWs

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = []
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for k in range(args.steps):
        out = step(events)
        marks[k + 1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = tokens / (ms_per_step * 1e-3)
    per_step_ms = sorted(marks[k].elapsed_time(marks[k + 1]) for k in range(args.steps))
    median_step_ms = per_step_ms[len(per_step_ms) // 2]

    # what a plain device-to-device copy reaches on this GPU (reads 1 GiB and writes 1 GiB per copy): quoted beside
    # the published 8 TB/s peak, outside the timed region
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    dst.copy_(src)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    for _ in range(5):
        dst.copy_(src)
    c1.record()
    torch.cuda.synchronize()
    copy_gbps = 5 * 2.0 * src.numel() * 4 / (c0.elapsed_time(c1) * 1e-3) / 1e9
    del src, dst

    # what this GPU sustains on float32 FMAs without packed instructions (as the library is built): a stream of
    # independent v_fma_f32 whose sources are vector registers, 8 waves per SIMD, timed with events on the launch stream
    from ncn_cuda_amd import probe
    lib = M._lib.load()
    attainable_valu = probe.fma_stream_tflops(device=dev)

    # The same workload through the autograd surface the reference times (NCNNetTestCuda(...)(x, xa); yi.backward(dyi),
    # grad_test_bench.py:116-134: one node per stage) and through the one-node form of the stack; then the timed step
    # replayed from a HIP graph (launch gaps taken out).  Medians of HIP-event brackets, outside the timed region.
    surface = {"autograd_per_stage_nodes_ms_per_step": None, "autograd_one_node_ms_per_step": None,
               "graph_ms_per_step": None}
    if not args.no_surface and args.grouping == "closed":
        import ncn_cuda_amd

        def timed_median(fn, reps):
            for _ in range(3):
                fn()
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
            ev[0].record()
            for k in range(reps):
                fn()
                ev[k + 1].record()
            torch.cuda.synchronize()
            t = sorted(ev[k].elapsed_time(ev[k + 1]) for k in range(reps))
            return t[len(t) // 2]

        ax, axa = gx.clone().requires_grad_(), gxa.clone().requires_grad_()
        aWs = [w.clone().requires_grad_() for w in gWs]

        def through(net):
            def run():
                ax.grad = axa.grad = None
                for w in aWs:
                    w.grad = None
                yi, _ = net(ax, axa)
                yi.backward(gdyi)
            return run

        reps = max(5, min(args.steps, 20))
        surface["autograd_per_stage_nodes_ms_per_step"] = timed_median(
            through(ncn_cuda_amd.NCNNetTestCuda(alpha, "tanh", n, C, L, aWs)), reps)
        surface["autograd_one_node_ms_per_step"] = timed_median(
            through(ncn_cuda_amd.NCNNetTestCuda(alpha, "tanh", n, C, L, aWs, fuse_stages=True,
                                                save_every=save_every)), reps)
        del ax, axa, aWs
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()                       # every kernel's attributes are set before the capture
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                graph_out = step()
            surface["graph_ms_per_step"] = timed_median(graph.replay, reps)
            surface["graph_replay_matches_eager"] = bool(
                torch.equal(graph_out[2], out[2]) and all(torch.equal(a, b) for a, b in zip(graph_out[4], out[4])))
            del graph, graph_out
        except RuntimeError as exc:      # a capture the runtime refuses is reported, not fatal to the headline figure
            surface["graph_error"] = str(exc).splitlines()[0][:200]

    # the invertible-inverse pass over the whole stack (not part of the step; the invertible configuration, cfg5, is quoted with it):
    # from the final outputs back to the inputs, segment by segment as the backward reverses them
    inverse_ms = None
    if args.grouping in ("closed", "radix"):
        fy, fya = gx, gxa          # float32 outputs of the stack (the step above may have stored bf16)
        for a, cnt in segs:
            if args.grouping == "radix":
                fy, fya = M.forward_radix(fy, fya, Wst[a:a + cnt], alpha, 0, n, C, a, cnt)
            else:
                fy, fya = M.forward_stages(fy, fya, Wst[a:a + cnt], alpha, 0, n, C, a, cnt, out_dtype=torch.float32)

        def inverse_all():
            cy, cya = fy, fya
            for a, cnt in reversed(segs):
                if args.grouping == "radix":
                    cy, cya = M.inverse_radix(cy, cya, Wst[a:a + cnt], alpha, 0, n, C, a, cnt)
                else:
                    cy, cya = M.inverse_stages(cy, cya, Wst[a:a + cnt], alpha, 0, n, C, a, cnt)
            return cy, cya

        inverse_all()
        i0, i1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        i0.record()
        for _ in range(5):
            rx, rxa = inverse_all()
        i1.record()
        torch.cuda.synchronize()
        inverse_ms = i0.elapsed_time(i1) / 5
        recon_err = ((rx - gx.float()).abs().max() / gx.float().abs().max()).item()

    # dominant kernel: backward stage launch (its event bracket also holds the microsecond-scale dW reduce)
    # (with multi-stage segments the bracket holds one backward call over a whole segment, and the algorithmic bytes
    # are those of one call: its inputs and outputs once, however many stages it runs)
    # (n_cache >= 8 never uses multi-stage passes: a call over a segment is one launch per stage, so the figures
    # stay per stage launch there)
    lds_passes = save_every > 1 and n in (2, 4)
    bracket_ms = sum(e0.elapsed_time(e1) for e0, e1, _ in events)
    stages_in_brackets = sum(cnt for _, _, cnt in events)
    bwd_ms = bracket_ms / len(events) if lds_passes else bracket_ms / stages_in_brackets
    stages_per_unit = stages_in_brackets / len(events) if lds_passes else 1.0
    # saved outputs of a stage are read as 4 bytes per value in either storage (float32, or two bf16 planes)
    bytes_bwd_launch = 6.0 * P * (sbytes if save_every == 1 else 4)   # read y, ya, dy, dya; write dx, dxa
    hbm_achieved = bytes_bwd_launch / (bwd_ms * 1e-3) / 1e9
    elem_steps_stage = float(P) * n
    flops_bwd_unit = FLOPS_BWD_PER_ELEM_STEP * elem_steps_stage * stages_per_unit
    valu_achieved = flops_bwd_unit / (bwd_ms * 1e-3) / 1e12
    flops_step = (FLOPS_FWD_PER_ELEM_STEP + FLOPS_BWD_PER_ELEM_STEP) * elem_steps_stage * L
    # which roof binds the dominant kernel: at the two peaks, n_cache tanh steps per element cost more time than its
    # bytes from 8 rows per group on (one launch per stage); the multi-stage passes of small groups are built to be
    # limited by their HBM round trips
    valu_bound = n >= 8
    version = lib.ncn_version().decode()
    import ctypes
    on_register_kernels = lib.ncn_kernel_path(ctypes.byref(M._lib.NcnShape(batch, N, E, C, n))) == 2
    wide = next((w for w in (32, 16, 8, 4) if E % w == 0), 0)   # adjacent one-feature heads that a row's lanes hold
    kernel = ((f"headwise_backward_kernel<{n},{wide}> (one feature per head)" if on_register_kernels and C == E else
               f"stage_backward_kernel<{n},{E // C}>" if on_register_kernels else
               f"generic_backward_kernel (n_cache {n}, heads of {E // C}: no register-tile build)") +
              (" (indexed build)" if tables else "") if not lds_passes else
              f"backward call over a segment of up to {save_every} stages (multi-stage passes)")
    roof = {"bound": "fp32_valu" if valu_bound else "hbm",
            "achieved": valu_achieved if valu_bound else hbm_achieved,
            "peak": VALU_PEAK_TFLOPS if valu_bound else HBM_PEAK_GBS,
            "unit": "TFLOP/s" if valu_bound else "GB/s",
            "frac": (valu_achieved / VALU_PEAK_TFLOPS) if valu_bound else (hbm_achieved / HBM_PEAK_GBS),
            "traffic": measured_traffic(args.config, args.grouping, version, args.scalar_heads),
            "kernel": kernel, "avg_launch_ms": bwd_ms,
            "algorithmic_flops_per_launch": flops_bwd_unit,
            "algorithmic_bytes_per_launch": bytes_bwd_launch,
            "valu_achieved_TFLOPs": valu_achieved, "valu_frac_of_peak": valu_achieved / VALU_PEAK_TFLOPS,
            "attainable_valu_TFLOPs": attainable_valu, "valu_frac_of_attainable": valu_achieved / attainable_valu,
            "hbm_achieved_GBps": hbm_achieved, "hbm_frac": hbm_achieved / HBM_PEAK_GBS,
            "attainable_copy_GBps": copy_gbps, "hbm_frac_of_attainable_copy": hbm_achieved / copy_gbps,
            "ncn_version": version, "build_id": lib.ncn_build_id().decode()}
    result = {
        "metric": f"NCN fwd+bwd tokens/sec and achieved HBM GB/s (% roofline), B={tokens} D={N} g={n}",
        "value": value,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",  # arithmetic type; storage is named in config.workload
        "data": "synthetic",
        "config": {"workload": f"{args.config}: B={tokens} D={N} g={n} -> x[batch={batch},N={N},E={E}], "
                               f"{C} heads of {E // C}, n_cache={n}, {L} stages, alpha=0.9, m=0.9, tanh, "
                               f"{cfg['dtype']} storage, outputs saved every {save_every} stage(s), "
                               f"grouping {args.grouping}", "positions_per_s": batch * N / (ms_per_step * 1e-3),
                   "backward_calls_per_step": len(segs)},
        "roofline": roof,
        "stack": {"median_ms_per_step": median_step_ms,
                  "min_ms_per_step": per_step_ms[0], "max_ms_per_step": per_step_ms[-1],
                  "algorithmic_bytes_fused": 10.0 * P * sbytes,
                  "achieved_GBps_fused_bytes": 10.0 * P * sbytes / (ms_per_step * 1e-3) / 1e9,
                  "algorithmic_bytes_per_stage_launches": 10.0 * P * sbytes * L,
                  "achieved_GBps_per_stage_bytes": 10.0 * P * sbytes * L / (ms_per_step * 1e-3) / 1e9,
                  "fp32_flops_per_step": flops_step,
                  "achieved_TFLOPs": flops_step / (ms_per_step * 1e-3) / 1e12,
                  "frac_of_fp32_vector_peak": flops_step / (ms_per_step * 1e-3) / 1e12 / VALU_PEAK_TFLOPS,
                  "frac_of_attainable_valu": flops_step / (ms_per_step * 1e-3) / 1e12 / attainable_valu,
                  **surface,
                  "inverse_ms_per_stack": inverse_ms,
                  "inverse_reconstruction_rel_err": recon_err if inverse_ms is not None else None},
    }

    if not args.no_cpu:
        from oracle import ncn_oracle as O   # the checker, timed here as the CPU baseline and nowhere else in this file
        ncores = os.cpu_count() or 1
        threads = min(ncores, 16)
        torch.set_num_threads(threads)
        f = torch.float32

        def cpu_run(b):
            xs, xas, dys = x[:b].to(f), xa[:b].to(f), dyi[:b].to(f)
            w32 = [w.to(f) for w in Ws]
            t = time.perf_counter()
            O.net_backward_checkpointed(xs, xas, dys, torch.zeros_like(dys), w32, alpha, n, C, save_every=1)
            return time.perf_counter() - t

        probe_b = min(batch, 2)
        cpu_run(1)
        tp = cpu_run(probe_b)
        sample_b = int(max(probe_b, min(batch, round(6.0 / max(tp / probe_b, 1e-6)))))
        ts = cpu_run(sample_b)
        cpu_tokens_s = sample_b * E / ts
        # the literal restatement of torch_ref's Python loops, on the one configuration where it is feasible
        # (configuration 1: x[1,256,32], n_cache 2, 8 stages, one head, forward only)
        lx, lxa, lWs, _, _ = O.make_inputs(1, 256, 32, 8, 2, seed=0, xa_zero=True)
        tl = time.perf_counter()
        O.literal_net_forward(lx, lxa, lWs, alpha, 2, 1)
        literal_s = time.perf_counter() - tl
        # the plain C restatement (oracle/ncn_oracle.c: scalar loops per group, OpenMP over groups), same step:
        # forward keeping every stage's outputs, then the reversible backward stage by stage
        from oracle import c_oracle as CO

        def c_run(b):
            xs, xas, dys = x[:b].to(f), xa[:b].to(f), dyi[:b].to(f)
            w32 = [w.to(f) for w in Ws]
            t = time.perf_counter()
            CO.net_forward_backward(xs, xas, w32, dys, None, alpha, n, C)
            return time.perf_counter() - t

        c_run(1)
        tcp = c_run(probe_b)
        c_sample_b = int(max(probe_b, min(batch, round(12.0 / max(tcp / probe_b, 1e-6)))))
        tcs = c_run(c_sample_b)
        result["cpu_baseline"] = {"value": c_sample_b * E / tcs, "unit": "tokens/s", "cores": CO.threads(),
                                  "kind": "port",
                                  "sample": f"first {c_sample_b} of {batch} batch entries of the same workload "
                                            f"({c_sample_b * E} of {tokens} tokens), float32, plain C restatement of "
                                            f"torch_ref with OpenMP over the groups (forward + reversible backward), "
                                            f"{tcs:.1f} s wall",
                                  "host_cpus_visible": ncores,
                                  "pytorch_restatement": {
                                      "value": cpu_tokens_s, "unit": "tokens/s", "cores": threads,
                                      "sample": f"first {sample_b} of {batch} batch entries, float32, vectorised "
                                                f"PyTorch restatement (forward + reversible backward), {ts:.1f} s wall"},
                                  "literal_loops_cfg1": {"value": 32 / literal_s, "unit": "tokens/s", "cores": 1,
                                                         "sample": "configuration 1 (B=32 D=256 g=2, 8 stages), forward "
                                                                   "only, per-row Python loops as in torch_ref"}}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
