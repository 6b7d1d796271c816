"""Per-layer summary of a rocprofv3 kernel trace of replayed passes.

    python -m ogle_amd.profile_layers KERNEL_TRACE.csv PLAN.json [-o SUMMARY.txt]
    python -m ogle_amd.profile_layers --fetch FETCH.csv --write WRITE.csv PLAN.json [-o SUMMARY.txt]

The second form reads the counter_collection CSVs of two `rocprofv3 --pmc` runs of the same
command (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch) instead of a kernel trace and gives HBM
bytes per launch next to the algorithmic bytes.  Each counter is scaled by what it reads for the
plain copy of known size that `bench.py --profile-layers` launches before the replays.

PLAN.json is what `bench.py --profile-layers PLAN.json` writes: the dispatch sequence of one
pass (Session.launch_plan: which node(s) every call into the kernel library was made for and
how many device operations it became), the number of replays R that ended the run, and the
algorithmic FLOPs / bytes of every convolution layer.  A replayed hipGraph issues exactly that
sequence, so the last R * N dispatches of the trace (N per pass) are R copies of it and every
position belongs to a known node.  Durations are averaged over the replays per position.

Roofline per row: FLOPs = 2 x multiply-adds, bytes = input + weights + bias + output once each;
bound "mfma" rows are divided by 157.3 TFLOP/s (fp32 MFMA), "hbm" rows by 8 TB/s.
"""
import argparse
import csv
import json
import re
import sys

MFMA_F32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0


def short_kernel(name):
    name = name.replace("ogle::(anonymous namespace)::", "").replace("void ", "")
    return name.split("(")[0]


def family_of(nodes, layers):
    kinds = set()
    for n in nodes:
        n = n[len("reduce:"):] if n.startswith("reduce:") else n
        l = layers.get(n)
        if l is None:
            kinds.add("tail")
        elif n.startswith("head") or n.startswith("extra"):
            kinds.add("heads+extras")
        elif l["kind"] == "pw":
            kinds.add("pointwise")
        elif l["kind"] == "dw":
            kinds.add("depthwise")
        else:
            kinds.add("stem")
    return "+".join(sorted(kinds))


def summarize(trace_path, plan):
    csv.field_size_limit(1 << 30)
    rows = [r for r in csv.DictReader(open(trace_path)) if r.get("Kind", "KERNEL_DISPATCH") == "KERNEL_DISPATCH"]
    rows.sort(key=lambda r: int(r["Dispatch_Id"]))
    n, reps = plan["dispatches_per_pass"], plan["replays"]
    if len(rows) < n * reps:
        raise SystemExit("trace holds %d dispatches, fewer than %d replays x %d" % (len(rows), reps, n))
    tail = rows[-n * reps:]
    pos = []
    for j in range(n):
        names = {short_kernel(tail[r * n + j]["Kernel_Name"]) for r in range(reps)}
        if len(names) != 1:
            raise SystemExit("position %d of the pass is not the same kernel in every replay: %s" % (j, names))
        durs = [(int(tail[r * n + j]["End_Timestamp"]) - int(tail[r * n + j]["Start_Timestamp"])) / 1e3
                for r in range(reps)]
        pos.append((names.pop(), sum(durs) / reps))
    spans = []
    for r in range(reps):
        seg = tail[r * n:(r + 1) * n]
        spans.append((max(int(x["End_Timestamp"]) for x in seg) - min(int(x["Start_Timestamp"]) for x in seg)) / 1e3)
    layers = plan["layers"]
    batch = plan["batch"]
    out, fam, at = [], {}, 0
    for label, k in plan["plan"]:
        # "reduce:a#Conv#+b#Conv#": the reductions of a and b; "a#Conv#[0+2/7]": shares of a
        is_reduce = label.startswith("reduce:")
        nodes, share = [], {}
        for name, _typ, f, c, n_parts in re.findall(r"([^#+\[\]:]+)#([A-Za-z0-9_]+)#(?:\[(\d+)\+(\d+)/(\d+)\])?",
                                                   label):
            nodes.append(name)
            if n_parts:
                share[name] = share.get(name, 0.0) + int(c) / int(n_parts)
        kernels = pos[at:at + k]
        at += k
        us = sum(d for _, d in kernels)
        flops = 0 if is_reduce else sum(layers[x]["flops_per_image"] * batch * share.get(x, 1.0)
                                        for x in nodes if x in layers)
        nbytes = 0 if is_reduce else sum((layers[x]["act_bytes_per_image"] * batch + layers[x]["weight_bytes"])
                                         * share.get(x, 1.0) for x in nodes if x in layers)
        nbytes += sum(plan.get("tail_bytes", {}).get(x, 0) for x in nodes)   # the detector's launches
        f = family_of(nodes, layers)
        bound = "hbm" if f in ("depthwise", "stem", "tail") else "mfma"
        if is_reduce:
            nodes = ["reduce:" + nodes[0]] + nodes[1:]
        out.append(dict(nodes=nodes, kernels=kernels, us=us, flops=flops, bytes=nbytes, family=f, bound=bound))
        a = fam.setdefault(f, dict(us=0.0, flops=0.0, bytes=0.0, launches=0, bound=bound))
        a["us"] += us
        a["flops"] += flops
        a["bytes"] += nbytes
        a["launches"] += k
    assert at == n
    return out, fam, pos, sum(spans) / reps


def _dispatch_rows(path, counter):
    csv.field_size_limit(1 << 30)
    rows = [r for r in csv.DictReader(open(path)) if r["Counter_Name"] == counter]
    rows.sort(key=lambda r: int(r["Dispatch_Id"]))
    return rows


def _scaled_tail(path, counter, plan):
    """Per position of the pass: (kernel, bytes per launch) from one counter run, averaged over the
    replays and scaled by the calibration copy's reading."""
    rows = _dispatch_rows(path, counter)
    cal = plan["calibration"]
    seen = [float(r["Counter_Value"]) for r in rows if cal["kernel"] in r["Kernel_Name"]]
    if not seen:
        raise SystemExit("%s: no dispatch of the calibration kernel %s" % (path, cal["kernel"]))
    scale = cal["kib_per_launch"] / (sum(seen) / len(seen))
    n, reps = plan["dispatches_per_pass"], plan["replays"]
    if len(rows) < n * reps:
        raise SystemExit("%s holds %d dispatches, fewer than %d replays x %d" % (path, len(rows), reps, n))
    tail = rows[-n * reps:]
    pos = []
    for j in range(n):
        names = {short_kernel(tail[r * n + j]["Kernel_Name"]) for r in range(reps)}
        if len(names) != 1:
            raise SystemExit("position %d of the pass is not the same kernel in every replay: %s" % (j, names))
        kib = sum(float(tail[r * n + j]["Counter_Value"]) for r in range(reps)) / reps
        pos.append((names.pop(), kib * scale * 1024.0))
    return pos, scale, sum(seen) / len(seen)


def render_traffic(fetch_path, write_path, plan):
    fetch, fscale, fraw = _scaled_tail(fetch_path, "FETCH_SIZE", plan)
    write, wscale, wraw = _scaled_tail(write_path, "WRITE_SIZE", plan)
    layers, batch = plan["layers"], plan["batch"]
    lines = []
    w = lines.append
    w("# HBM traffic per launch of the pass (rocprofv3 counters): %s" % plan["workload"])
    w("")
    w("commands (run from the repository root on one MI355X, one counter per run):")
    for c in plan["commands"]:
        w("    " + c)
    w("")
    cal = plan["calibration"]
    w("Counters are KiB per dispatch.  Before the passes the script launches a plain copy of %d KiB"
      % cal["kib_per_launch"])
    w("(%s: reads and writes that much), which calibrates them:" % cal["kernel"])
    w("    FETCH_SIZE read %.1f KiB for the copy -> scale %.4f" % (fraw, fscale))
    w("    WRITE_SIZE read %.1f KiB for the copy -> scale %.4f" % (wraw, wscale))
    w("Values below are scaled and averaged over %d passes; algorithmic = input + weights + bias + output"
      % plan["replays"])
    w("once each (0 for reductions and concat, whose bytes are all overhead here; the detector's two launches: their lists).")
    w("")
    w("%-44s %-46s %10s %10s %10s %7s" % ("node(s)", "kernel", "fetch MB", "write MB", "algo MB", "ratio"))
    fam, at = {}, 0
    for label, k in plan["plan"]:
        is_reduce = label.startswith("reduce:")
        nodes = [m[0] for m in re.findall(r"([^#+\[\]:]+)#([A-Za-z0-9_]+)#", label)]
        algo = 0 if is_reduce else sum(layers[x]["act_bytes_per_image"] * batch + layers[x]["weight_bytes"]
                                       for x in nodes if x in layers)
        algo += sum(plan.get("tail_bytes", {}).get(x, 0) for x in nodes)
        f = family_of(nodes, layers)
        name = ("reduce:" if is_reduce else "") + "+".join(nodes)
        if len(name) > 43:
            name = name[:40] + "..."
        fb = sum(b for _, b in fetch[at:at + k])
        wb = sum(b for _, b in write[at:at + k])
        for i in range(k):
            w("%-44s %-46s %10.2f %10.2f %10s %7s" % (
                name if i == 0 else "  (same call)", fetch[at + i][0][:46], fetch[at + i][1] / 1e6,
                write[at + i][1] / 1e6, ("%.2f" % (algo / 1e6)) if i == 0 else "",
                ("%.2f" % ((fb + wb) / algo)) if i == 0 and algo else ""))
        at += k
        a = fam.setdefault(f, dict(traffic=0.0, algo=0.0, launches=0))
        a["traffic"] += fb + wb
        a["algo"] += algo
        a["launches"] += k
    w("")
    w("per family (traffic of the family's launches incl. its split-K reductions; per launch = / launches):")
    w("%-28s %9s %12s %12s %7s" % ("family", "launches", "traffic MB", "algo MB", "ratio"))
    for f, a in sorted(fam.items(), key=lambda kv: -kv[1]["traffic"]):
        w("%-28s %9d %12.2f %12.2f %7s" % (f, a["launches"], a["traffic"] / 1e6, a["algo"] / 1e6,
                                            ("%.2f" % (a["traffic"] / a["algo"])) if a["algo"] else ""))
    w("")
    for f, a in sorted(fam.items()):
        w("traffic_bytes_per_launch[%s]=%d" % (f, round(a["traffic"] / a["launches"])))
    return "\n".join(lines) + "\n"


def render(out, fam, pos, span, plan):
    lines = []
    w = lines.append
    w("# per-layer summary of the replayed pass: %s" % plan["workload"])
    w("")
    w("commands (run from the repository root on one MI355X):")
    for c in plan["commands"]:
        w("    " + c)
    w("")
    w("%d replays of the pass, %d dispatches each; pass span (first start to last end) %.1f us; "
      "sum of kernel durations %.1f us" % (plan["replays"], plan["dispatches_per_pass"], span,
                                            sum(d for _, d in pos)))
    w("")
    w("%-44s %-46s %8s %9s %8s %7s %7s %5s %6s" % ("node(s)", "kernel", "avg_us", "GFLOP", "MB", "TF/s", "TB/s", "bound", "frac"))
    for e in out:
        label = "+".join(e["nodes"])
        if len(label) > 43:
            label = label[:40] + "..."
        for i, (kname, d) in enumerate(e["kernels"]):
            if i == 0:
                tf = e["flops"] / e["us"] / 1e6 if e["us"] else 0.0
                tb = e["bytes"] / e["us"] / 1e6 if e["us"] else 0.0
                frac = tb * 1e3 / HBM_PEAK_GBS if e["bound"] == "hbm" else tf / MFMA_F32_PEAK_TFLOPS
                w("%-44s %-46s %8.2f %9.3f %8.2f %7.1f %7.2f %5s %6.3f" % (
                    label, kname[:46], d, e["flops"] / 1e9, e["bytes"] / 1e6, tf, tb, e["bound"], frac))
            else:
                w("%-44s %-46s %8.2f" % ("  (same call)", kname[:46], d))
    w("")
    w("per family (durations add up to the sum of kernel durations):")
    w("%-28s %9s %9s %9s %9s %7s %7s %5s %6s" % ("family", "launches", "us", "GFLOP", "MB", "TF/s", "TB/s", "bound", "frac"))
    for f, a in sorted(fam.items(), key=lambda kv: -kv[1]["us"]):
        tf = a["flops"] / a["us"] / 1e6
        tb = a["bytes"] / a["us"] / 1e6
        frac = tb * 1e3 / HBM_PEAK_GBS if a["bound"] == "hbm" else tf / MFMA_F32_PEAK_TFLOPS
        w("%-28s %9d %9.1f %9.3f %9.2f %7.1f %7.2f %5s %6.3f" % (f, a["launches"], a["us"], a["flops"] / 1e9,
                                                                   a["bytes"] / 1e6, tf, tb, a["bound"], frac))
    w("")
    w("per kernel (calls per pass, average duration):")
    agg = {}
    for kname, d in pos:
        c = agg.setdefault(kname, [0, 0.0])
        c[0] += 1
        c[1] += d
    for kname, (c, t) in sorted(agg.items(), key=lambda kv: -kv[1][1]):
        w("%-90s %4d %9.2f %9.2f" % (kname[:90], c, t, t / c))
    return "\n".join(lines) + "\n"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("trace", nargs="?")
    ap.add_argument("plan")
    ap.add_argument("--fetch", help="counter_collection CSV of a --pmc FETCH_SIZE run")
    ap.add_argument("--write", help="counter_collection CSV of a --pmc WRITE_SIZE run")
    ap.add_argument("-o", "--out")
    args = ap.parse_args()
    plan = json.load(open(args.plan))
    if args.fetch or args.write:
        if not (args.fetch and args.write) or args.trace:
            ap.error("give --fetch and --write together, without a kernel trace")
        text = render_traffic(args.fetch, args.write, plan)
    else:
        if not args.trace:
            ap.error("a kernel trace or --fetch/--write is needed")
        out, fam, pos, span = summarize(args.trace, plan)
        text = render(out, fam, pos, span, plan)
    if args.out:
        with open(args.out, "w") as f:
            f.write(text)
    else:
        sys.stdout.write(text)


if __name__ == "__main__":
    main()
