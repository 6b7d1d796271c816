"""ogle_amd.profile_layers: attribution of a rocprofv3 kernel trace (or of two counter runs) to
the layers of a replayed pass, on made-up CSVs."""
import csv
import json

import pytest

from ogle_amd import profile_layers as PL

LAYERS = {
    "conv0": dict(kind="conv", flops_per_image=1000.0, act_bytes_per_image=400.0, weight_bytes=40.0),
    "b1.dw": dict(kind="dw", flops_per_image=200.0, act_bytes_per_image=800.0, weight_bytes=8.0),
    "b1.pw": dict(kind="pw", flops_per_image=4000.0, act_bytes_per_image=600.0, weight_bytes=64.0),
    "head0.loc": dict(kind="conv", flops_per_image=900.0, act_bytes_per_image=100.0, weight_bytes=36.0),
    "head0.conf": dict(kind="conv", flops_per_image=1800.0, act_bytes_per_image=120.0, weight_bytes=72.0),
}
PLAN = [["conv0#Conv#", 1], ["b1.dw#Conv#", 1], ["b1.pw#Conv#", 1], ["head0.loc#Conv#+head0.conf#Conv#", 1],
        ["reduce:head0.loc#Conv#+head0.conf#Conv#", 1], ["detector.topk_nms#Detector#", 1]]
KERNELS = ["stem_k(float*)", "void ogle::(anonymous namespace)::dw_k<float, 1>(Args)", "gemm_k<float, 64>(P)",
           "mixed_k<float>(G)", "reduce_k<float>(R)", "nms_k<true>(N)"]
DUR_NS = [2000, 1000, 4000, 3000, 500, 1500]


def plan_doc(replays, **extra):
    doc = dict(workload="synthetic", batch=2, replays=replays, dispatches_per_pass=len(PLAN), plan=PLAN,
               layers=LAYERS, commands=["rocprofv3 ... -- python3 bench.py --profile-layers plan.json"])
    doc.update(extra)
    return doc


def write_trace(path, replays, warmup_rows=3):
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Kind", "Dispatch_Id", "Kernel_Name", "Start_Timestamp", "End_Timestamp"])
        t, d = 1000, 1
        for _ in range(warmup_rows):                     # launches before the replays are ignored
            w.writerow(["KERNEL_DISPATCH", d, "warmup_k()", t, t + 100])
            t += 150
            d += 1
        for r in range(replays):
            for name, ns in zip(KERNELS, DUR_NS):
                ns = ns + 100 * r                        # replays differ a little: the mean is reported
                w.writerow(["KERNEL_DISPATCH", d, name, t, t + ns])
                t += ns
                d += 1


def test_kernel_trace_is_attributed_position_by_position(tmp_path):
    trace, replays = tmp_path / "t.csv", 3
    write_trace(trace, replays)
    out, fam, pos, span = PL.summarize(str(trace), plan_doc(replays))
    assert [e["nodes"] for e in out] == [["conv0"], ["b1.dw"], ["b1.pw"], ["head0.loc", "head0.conf"],
                                         ["reduce:head0.loc", "head0.conf"], ["detector.topk_nms"]]
    means = [(ns + 100) / 1e3 for ns in DUR_NS]          # mean over replays 0, 1, 2
    assert [round(e["us"], 6) for e in out] == [round(m, 6) for m in means]
    assert pos[1][0] == "dw_k<float, 1>"                 # namespace and arguments stripped
    assert span == pytest.approx(sum(means))             # back-to-back kernels: span = sum
    # work: batch x per-image figures (+ weights once); a reduction carries none
    assert out[2]["flops"] == 2 * 4000.0 and out[2]["bytes"] == 2 * 600.0 + 64.0
    assert out[3]["flops"] == 2 * (900.0 + 1800.0)
    assert out[4]["flops"] == 0 and out[4]["family"] == "heads+extras"
    assert {f: a["launches"] for f, a in fam.items()} == {"stem": 1, "depthwise": 1, "pointwise": 1,
                                                           "heads+extras": 2, "tail": 1}
    assert fam["heads+extras"]["us"] == pytest.approx(means[3] + means[4])
    text = PL.render(out, fam, pos, span, plan_doc(replays))
    assert "per family" in text and "gemm_k<float, 64>" in text and "rocprofv3 ..." in text


def test_trace_that_does_not_match_the_plan_is_refused(tmp_path):
    trace = tmp_path / "t.csv"
    write_trace(trace, 2)
    with pytest.raises(SystemExit, match="fewer than"):
        PL.summarize(str(trace), plan_doc(5))
    # one replay off by a kernel: the same position holds different kernels
    rows = list(csv.reader(open(trace)))
    rows[-1][2] = "other_k()"
    with open(trace, "w", newline="") as f:
        csv.writer(f).writerows(rows)
    with pytest.raises(SystemExit, match="not the same kernel"):
        PL.summarize(str(trace), plan_doc(2))


def test_counter_runs_give_scaled_traffic_per_family(tmp_path):
    replays = 2
    kib = [64.0, 128.0, 96.0, 40.0, 16.0, 4.0]

    def write_counters(path, counter, factor, copy_reading):
        with open(path, "w", newline="") as f:
            w = csv.writer(f)
            w.writerow(["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"])
            d = 1
            for _ in range(3):
                w.writerow([d, "void convert_kernel<float, float>(A)", counter, copy_reading])
                d += 1
            for _ in range(replays):
                for name, v in zip(KERNELS, kib):
                    w.writerow([d, name, counter, v * factor])
                    w.writerow([d, name, "OTHER", 1.0])      # rows of other counters are skipped
                    d += 1

    fetch, write = tmp_path / "f.csv", tmp_path / "w.csv"
    write_counters(fetch, "FETCH_SIZE", 0.5, 512.0)      # the counter reads half of the 1024 KiB copy
    write_counters(write, "WRITE_SIZE", 1.0, 1024.0)
    doc = plan_doc(replays, calibration=dict(kernel="convert_kernel<float, float>", kib_per_launch=1024))
    text = PL.render_traffic(str(fetch), str(write), doc)
    assert "scale 2.0000" in text and "scale 1.0000" in text
    got = {line.split("[")[1].split("]")[0]: int(line.split("=")[1])
           for line in text.splitlines() if line.startswith("traffic_bytes_per_launch[")}
    # fetch (scaled back to true KiB) + write, per launch of the family
    assert got["pointwise"] == int((96.0 + 96.0) * 1024)
    assert got["heads+extras"] == int((40.0 + 16.0) * 2 * 1024 / 2)
    assert got["depthwise"] == int(2 * 128.0 * 1024)
    bad = dict(doc, calibration=dict(kernel="no_such_kernel", kib_per_launch=1024))
    with pytest.raises(SystemExit, match="calibration kernel"):
        PL.render_traffic(str(fetch), str(write), bad)
