"""Per-stage performance report of a final specification: which node of the monolithic kernel costs what.

    python -m mononn_amd.perf_report --model bert_base [--spec-dir DIR] [--csv out.csv] [--launches 50]
    python -m mononn_amd.perf_report --hlo module.hlo --spec-dir DIR

Reference counterpart: the perf dumper (mononn_engine/tuning/perf_dumper_main.cc) and performance_report.csv, the
hotspot tool the README points users to (README.md:177).  The kernel is rebuilt from the same specification with
`mononn_hip.profile_stages`; every workgroup stamps the wall clock on entering and leaving each stage, the report
lists for every stage the time from the first workgroup in to the last workgroup done (`busy_us`), the mean
per-workgroup work time and the barrier time that follows.  Elided constants are filled with seeded N(0, 0.02)
values (the timing does not depend on them); entry parameters are zeros unless the model fixture makes its own.
"""
from __future__ import annotations

import argparse
import csv
import json
import sys

import numpy as np

from . import MonoNNModule
from .hlo import models


def stage_report(hlo_text: str, constants, inputs, outputs, spec_dir=None, launches=50, device=0, details=None):
    """Rows of the report, one per stage.  `details`, when given, is filled with what the profiled build computed
    (`outputs`, the live-outs of the last launch) and with its event-timed duration (`kernel_us`, the average over
    `launches` back-to-back launches): the report's steps must add up to the kernel they describe."""
    base = MonoNNModule.from_spec_dir(hlo_text, spec_dir) if spec_dir else MonoNNModule.compile(hlo_text, build=False)
    spec = json.loads(base.get_tuning_spec())
    spec["mononn_hip"]["profile_stages"] = True
    m = MonoNNModule.compile(hlo_text, json.dumps(spec))
    m.set_constants(constants)
    m.load(device)
    for _ in range(3):
        m.run(inputs, outputs)
    acc = None
    for _ in range(launches):
        m.run(inputs, outputs)
        p = m.stage_profile()
        if acc is None:
            acc = p
        else:
            for a, b in zip(acc, p):
                for k in ("busy_us", "barrier_us", "mean_wg_us", "step_us"):
                    a[k] += b[k]
    for a in acc:
        for k in ("busy_us", "barrier_us", "mean_wg_us", "step_us"):
            a[k] /= launches
    if details is not None:
        details["outputs"] = m.run(inputs, outputs)
        avg_ms, _ = m.time_raw(m.buffer_pointers(), warmup=5, iters=max(launches, 20))
        m.synchronize()
        details["kernel_us"] = avg_ms * 1e3
    m.close()
    return acc


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", choices=["bert_layer", "bert_base", "bert_large", "gpt2", "vit"])
    ap.add_argument("--hlo", help="HLO text file (parameters are fed zeros)")
    ap.add_argument("--spec-dir")
    ap.add_argument("--csv")
    ap.add_argument("--launches", type=int, default=50)
    args = ap.parse_args(argv)
    if args.model:
        fx = getattr(models, args.model)()
        text, consts, inputs, outputs = fx.hlo_text, fx.make_constants(1, "baseline"), fx.make_inputs(1), fx.outputs
    elif args.hlo:
        text = open(args.hlo).read()
        probe = MonoNNModule.compile(text, build=False)
        rng = np.random.default_rng(1)
        consts = {c["name"]: rng.normal(0, 0.02, c["bytes"] // 2).astype(np.float16) for c in probe.constants() if c["needs_payload"]}
        info = probe.buffer_info()
        inputs = [np.zeros(n, np.uint8) for n in info["parameters"]]
        outputs = [{"dtype": "u8", "dims": [n]} for n in info["liveouts"]]
    else:
        ap.error("one of --model / --hlo is required")
    rows = stage_report(text, consts, inputs, outputs, args.spec_dir, args.launches)
    out = open(args.csv, "w", newline="") if args.csv else sys.stdout
    w = csv.writer(out)
    w.writerow(["stage", "busy_us", "mean_workgroup_us", "barrier_us", "step_us", "nodes"])
    for r in rows:
        w.writerow([r["stage"], f"{r['busy_us']:.3f}", f"{r['mean_wg_us']:.3f}", f"{r['barrier_us']:.3f}", f"{r['step_us']:.3f}", r["nodes"]])
    busy, bar = sum(r["busy_us"] for r in rows), sum(r["barrier_us"] for r in rows)
    print(f"# total: {busy:.1f} us busy in {len(rows)} stages, {bar:.1f} us in {len(rows) - 1} barriers", file=sys.stderr)


if __name__ == "__main__":
    main()
