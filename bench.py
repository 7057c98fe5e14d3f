"""Headline benchmark: full BERT-base encoder (12 layers + embeddings, batch 1, seq 128, fp16) as ONE
launch of the monolithic persistent kernel on one MI355X (an ordinary launch; the grid is checked against the
co-resident capacity when the module is loaded).

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one forward pass = one launch of the generated kernel, inputs and weights resident in
HBM.  Prints one JSON line: throughput (seq/s) as `value`, latency in `ms_per_step` / `latency_us`,
the HBM roofline of the kernel (algorithmic bytes = weights + gathered rows + ids + output, read or
written once) with the launch duration measured by HIP events on the launch stream, and the NumPy
oracle timed on the host cores as `cpu_baseline`.  `other_configs` carries the three batched configurations
(BERT-large b16 s384, GPT-2 b4 s512 with the LM head, ViT-B/16 b8) with their shipped specifications, and the
benchmark's own model in bf16: kernel latency, fraction of the dense fp16 MFMA peak, and a property check of the
output (a few seconds each).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16 MFMA
SPEC_DIR = os.path.join(ROOT, "mononn_amd", "specs", "bert_base_b1_s128")
# HBM-side bytes of one launch of the kernel built from SPEC_DIR: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE of
# this script, each scaled by what the same counter reads for the 256 MiB --calibration-copy (summary under
# profiles/).  Counters cannot be read inside a timed run, so the figure is carried here.
MEASURED_TRAFFIC_BYTES = 451_033_377   # 372,229,281 fetched + 78,804,096 written


def algorithmic_bytes(fx) -> int:
    """Bytes a perfect fusion must move: every weight / bias / LayerNorm constant once, except the
    embedding tables of which only the gathered rows are read; ids in; hidden states out."""
    cfg = fx.config
    total = 0
    for meta in fx.constants.values():
        n = int(np.prod(meta["dims"])) * 2
        if meta["role"].endswith("word_embeddings") or meta["role"].endswith("token_type_embeddings"):
            n = cfg["B"] * cfg["S"] * cfg["H"] * 2          # gathered rows
        elif meta["role"].endswith("position_embeddings"):
            n = cfg["S"] * cfg["H"] * 2                      # first S rows
        total += n
    total += 3 * cfg["B"] * cfg["S"] * 4                     # three int32 id tensors
    total += cfg["B"] * cfg["S"] * cfg["H"] * 2              # output
    return total


def gemm_flops(cfg) -> int:
    B, S, H, NH, F, L = cfg["B"], cfg["S"], cfg["H"], cfg["NH"], cfg["F"], cfg["L"]
    M, d = B * S, H // NH
    per_layer = 2 * M * H * 3 * H + 2 * M * H * H + 4 * M * H * F + 4 * B * NH * S * S * d
    return per_layer * L


def torch_baseline(fx, consts, inputs, got):
    """The same encoder as plain PyTorch-ROCm fp16 (rocBLAS / MIOpen kernels), for scale: eager launches and the same
    launches replayed from a captured HIP graph.  Not part of the measured path."""
    import math
    import torch
    import torch.nn.functional as F
    cfg = fx.config
    dev = torch.device("cuda", 0)
    R = {m["role"]: torch.from_numpy(consts[n]).to(dev) for n, m in fx.constants.items()}
    B, S, H, NH, L = cfg["B"], cfg["S"], cfg["H"], cfg["NH"], cfg["L"]
    D = H // NH
    ids, mask, tt = (torch.from_numpy(a.astype(np.int64)).to(dev) for a in inputs)
    Wt = {k: v.t().contiguous() for k, v in R.items() if k.endswith("/kernel")}   # F.linear takes [out, in]

    def forward():
        emb = R["bert/embeddings/word_embeddings"][ids] + R["bert/embeddings/position_embeddings"][:S][None] + \
            R["bert/embeddings/token_type_embeddings"][tt]
        h = F.layer_norm(emb, (H,), R["bert/embeddings/LayerNorm/gamma"], R["bert/embeddings/LayerNorm/beta"], 1e-12)
        add = ((1.0 - mask.to(torch.float16)) * -10000.0)[:, None, None, :]
        for l in range(L):
            P = f"bert/encoder/layer_{l}/"

            def lin(x, p):
                return F.linear(x, Wt[P + p + "/kernel"], R[P + p + "/bias"])
            q, k, v = (lin(h, "attention/" + n).view(B, S, NH, D).transpose(1, 2) for n in ("query", "key", "value"))
            p = torch.softmax(q @ k.transpose(2, 3) / math.sqrt(D) + add, -1)
            ctx = (p @ v).transpose(1, 2).reshape(B, S, H)
            x1 = F.layer_norm(lin(ctx, "attention/output") + h, (H,), R[P + "attention/LayerNorm/gamma"], R[P + "attention/LayerNorm/beta"], 1e-12)
            a = F.gelu(lin(x1, "intermediate"), approximate="tanh")
            h = F.layer_norm(lin(a, "output") + x1, (H,), R[P + "output/LayerNorm/gamma"], R[P + "output/LayerNorm/beta"], 1e-12)
        return h

    def time_it(fn, n):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    with torch.no_grad():
        out = forward()
        eager_us = time_it(forward, 100)
        graph_us = None
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    forward()
            torch.cuda.current_stream().wait_stream(side)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                forward()
            graph_us = time_it(g.replay, 200)
        except Exception as e:   # graph capture is a convenience here, not a requirement
            print(f"bench.py: HIP graph capture of the torch model failed: {e}", file=sys.stderr)
    diff = float(np.abs(out.float().cpu().numpy() - got).max())
    return {"eager_us_per_forward": round(eager_us, 1), "hip_graph_us_per_forward": None if graph_us is None else round(graph_us, 1),
            "max_abs_diff_vs_kernel": diff, "note": "torch.nn.functional fp16 on the same GPU; scale only"}


def barrier_time(module, fx, consts, inputs, launches=10):
    """Stage count and total time spent in grid barriers (last workgroup done -> first workgroup in the next stage),
    from the in-kernel clocks of the same specification rebuilt with per-stage stamps."""
    from mononn_amd import MonoNNModule
    spec = json.loads(module.get_tuning_spec())
    spec["mononn_hip"]["profile_stages"] = True
    prof_mod = MonoNNModule.compile(fx.hlo_text, json.dumps(spec))
    prof_mod.set_constants(consts)
    prof_mod.load(0)
    for _ in range(3):
        prof_mod.run(inputs, fx.outputs)
    total = 0.0
    for _ in range(launches):
        prof_mod.run(inputs, fx.outputs)
        p = prof_mod.stage_profile()
        total += sum(a["barrier_us"] for a in p)
    n = len(p)
    prof_mod.close()
    return n, total / launches


def other_configs():
    """The batched configurations (parity cases of the path, not the headline): shipped specification, kernel latency
    by HIP events, GEMM FLOPs / latency against the dense fp16 MFMA peak, and a property of the output that needs no
    oracle (the parity tests hold the oracle comparisons)."""
    import torch
    from mononn_amd import MonoNNModule
    from mononn_amd.hlo import models
    out = {}
    for key, make, spec_name, seed in (("bert_large_b16_s384", models.bert_large, "bert_large_b16_s384", 1236),
                                       ("gpt2_b4_s512", models.gpt2, "gpt2_b4_s512", 1237),
                                       ("vit_b16_b8", models.vit, "vit_b16_b8", 1238),
                                       # the benchmark's model stored and multiplied in bf16, on the specification tuned for f16
                                       ("bert_base_b1_s128_bf16", lambda: models.bert_base(ftype="bf16"), "bert_base_b1_s128", 1235)):
        fx = make()
        cfg = fx.config
        spec_dir = os.path.join(ROOT, "mononn_amd", "specs", spec_name)
        used = "default"
        m = None
        if os.path.isdir(spec_dir):
            try:
                m = MonoNNModule.from_spec_dir(fx.hlo_text, spec_dir)
                used = os.path.relpath(spec_dir, ROOT)
            except Exception as e:
                print(f"bench.py: {spec_dir} unusable ({e}); default specification", file=sys.stderr)
        if m is None:
            m = MonoNNModule.compile(fx.hlo_text)
        m.set_constants(fx.make_constants(seed, "baseline"))
        m.load(0)
        inputs = fx.make_inputs(seed)
        y = m.run(inputs, fx.outputs)[0]
        avg_ms, _ = m.time_raw(m.buffer_pointers(), torch.cuda.current_stream().cuda_stream, warmup=3, iters=15)
        flops = gemm_flops(cfg)
        if fx.name.startswith("gpt2"):
            flops += 2 * cfg["B"] * cfg["S"] * cfg["H"] * cfg["vocab"]
        if fx.name.startswith("vit"):
            flops += 2 * cfg["B"] * (cfg["S"] - 1) * cfg["H"] * (3 * cfg["patch"] ** 2)      # patch embedding as a GEMM
        bf = fx.outputs[0]["dtype"] == "bf16"
        if bf:
            from mononn_amd import bf16
            x = bf16.from_bits(y).astype(np.float64)
        else:
            x = y.astype(np.float64)
        if fx.name.startswith("gpt2"):
            again = m.run(inputs, fx.outputs)[0]
            prop = {"check": "finite logits, bit-identical on a second launch", "ok": bool(np.isfinite(x).all() and np.array_equal(again, y))}
        else:   # the output is a LayerNorm with gamma 1 / beta 0 ("baseline" constants): rows of mean 0, variance 1
            tol_mean, tol_var = (2e-2, 5e-2) if bf else (5e-3, 2e-2)      # bf16 keeps 8 bits of every output
            prop = {"check": f"rows of the final LayerNorm: |mean| < {tol_mean:g}, |var - 1| < {tol_var:g}",
                    "ok": bool(np.isfinite(x).all() and np.abs(x.mean(-1)).max() < tol_mean and np.abs(x.var(-1) - 1.0).max() < tol_var)}
        tflops = flops / (avg_ms * 1e-3) / 1e12
        out[key] = {"latency_us": round(avg_ms * 1e3, 1), "tuning_spec": used, "grid_barriers": m.launch_dims()["barriers"],
                    "dtype": "bf16" if bf else "f16",
                    "mfma": {"achieved_tflops": round(tflops, 1), "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4), "gemm_flops": flops},
                    "property": prop}
        m.close()
        del m
        torch.cuda.empty_cache()
    return out


# configurations bench.py can run: name -> (fixture in mononn_amd.hlo.models, seed)
WORKLOADS = {"bert_base_b1_s128": ("bert_base", 1235), "bert_large_b16_s384": ("bert_large", 1236), "gpt2_b4_s512": ("gpt2", 1237),
             "vit_b16_b8": ("vit", 1238), "gemm_stage_6144x4096x1024": ("gemm_stage", 1239)}


def single_workload(args):
    """One configuration other than the benchmark's: its launches and one line with its latency (not the metric)."""
    import torch
    from mononn_amd import MonoNNModule
    from mononn_amd.hlo import models
    make, seed = WORKLOADS[args.workload]
    fx = getattr(models, make)()
    spec_dir = os.path.join(ROOT, "mononn_amd", "specs", args.workload)
    used = "default"
    if os.path.isdir(spec_dir):
        module = MonoNNModule.from_spec_dir(fx.hlo_text, spec_dir)
        used = os.path.relpath(spec_dir, ROOT)
    else:
        module = MonoNNModule.compile(fx.hlo_text)
    consts, inputs = fx.make_constants(seed, "baseline"), fx.make_inputs(seed)
    module.set_constants(consts)
    module.load(0)
    if args.stage_profile:
        stage_profile(module, fx, consts, inputs, args)
        return
    module.run(inputs, fx.outputs)
    avg_ms, _ = module.time_raw(module.buffer_pointers(), torch.cuda.current_stream().cuda_stream, warmup=args.warmup, iters=args.steps)
    line = {"workload": args.workload, "not_the_benchmark_metric": True, "kernel": module.kernel_name, "kernel_avg_us": round(avg_ms * 1e3, 2),
            "steps": args.steps, "warmup": args.warmup, "tuning_spec": used, **module.launch_dims()}
    if make == "gemm_stage" and not args.launches_only:
        # the GEMM stage alone, by the in-kernel clocks of the same specification
        spec = json.loads(module.get_tuning_spec())
        spec["mononn_hip"]["profile_stages"] = True
        prof = MonoNNModule.compile(fx.hlo_text, json.dumps(spec))
        prof.set_constants(consts)
        prof.load(0)
        us = []
        for i in range(8):
            prof.run(inputs, fx.outputs)
            if i >= 3:
                us.append(prof.stage_profile()[1]["busy_us"])
        c = fx.config
        flops = 2 * c["M"] * c["N"] * c["K"]
        line["gemm_stage"] = {"busy_us": round(float(np.mean(us)), 2), "tflops": round(flops / np.mean(us) / 1e6, 1),
                              "frac_of_dense_f16_mfma_peak": round(flops / np.mean(us) / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)}
        prof.close()
    print(json.dumps(line))
    module.close()


def stage_profile(module, fx, consts, inputs, args):
    """Per-stage clocks of the benchmark's own specification (stamped by every workgroup at stage entry / exit)."""
    from mononn_amd import MonoNNModule
    spec = json.loads(module.get_tuning_spec())
    spec["mononn_hip"]["profile_stages"] = True
    prof_mod = MonoNNModule.compile(fx.hlo_text, json.dumps(spec))
    prof_mod.set_constants(consts)
    prof_mod.load(0)
    for _ in range(max(args.warmup, 3)):
        prof_mod.run(inputs, fx.outputs)
    acc = None
    n = max(1, min(args.steps, 50))
    for _ in range(n):
        prof_mod.run(inputs, fx.outputs)
        p = prof_mod.stage_profile()
        if acc is None:
            acc = p
        else:
            for a, b in zip(acc, p):
                for k in ("busy_us", "barrier_us", "mean_wg_us", "step_us"):
                    a[k] += b[k]
    for a in acc:
        for k in ("busy_us", "barrier_us", "mean_wg_us", "step_us"):
            a[k] /= n
    print(f"stage clocks, mean of {n} launches; busy = first workgroup in -> last workgroup done, "
          f"barrier = last workgroup done -> first workgroup in the next stage, "
          f"step = last workgroup done in the previous stage -> last workgroup done in this one")
    print(f"{'stage':>5} {'busy_us':>8} {'mean_wg_us':>10} {'barrier_us':>10} {'step_us':>8}  nodes")
    for a in acc:
        print(f"{a['stage']:5d} {a['busy_us']:8.2f} {a['mean_wg_us']:10.2f} {a['barrier_us']:10.2f} {a['step_us']:8.2f}  {a['nodes'][:90]}")
    busy, bar = sum(a["busy_us"] for a in acc), sum(a["barrier_us"] for a in acc)
    print(f"total: busy {busy:.1f} us in {len(acc)} stages, barriers {bar:.1f} us ({len(acc) - 1} barriers)")
    prof_mod.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the three batched configurations")
    ap.add_argument("--spec-dir", default=SPEC_DIR)
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known traffic for scaling rocprof counters)")
    ap.add_argument("--torch-baseline", action="store_true",
                    help="also time the same model written with torch.nn.functional in fp16 on this GPU (eager and "
                         "captured in a HIP graph), reported under \"torch_baseline\"")
    ap.add_argument("--workload", default="bert_base_b1_s128", choices=sorted(WORKLOADS),
                    help="bert_base_b1_s128 is the benchmark; any other name runs that configuration alone (shipped "
                         "specification where there is one) for --warmup + --steps launches and prints its latency: "
                         "the command profilers are pointed at.  With --stage-profile: its stage clocks")
    ap.add_argument("--launches-only", action="store_true",
                    help="with --workload: nothing but the configuration's own launches (for counter collection, where "
                         "every kernel of the process is profiled)")
    ap.add_argument("--stage-profile", action="store_true",
                    help="instead of the benchmark: rebuild the same specification with per-stage clocks and print, "
                         "per stage, busy time / barrier time averaged over --steps launches")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the monolithic kernel's grid barrier cannot span "
              "devices); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from mononn_amd import MonoNNModule, device_info
    from mononn_amd.hlo import models

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.workload != "bert_base_b1_s128":
        single_workload(args)
        return
    fx = models.bert_base(B=1, S=128)
    consts = fx.make_constants(1235, "baseline")
    inputs = fx.make_inputs(1235)

    used_spec = "default"
    module = None
    if os.path.isdir(args.spec_dir):
        try:
            module = MonoNNModule.from_spec_dir(fx.hlo_text, args.spec_dir)
            used_spec = os.path.relpath(args.spec_dir, ROOT)
        except Exception as e:  # a stale spec must not silently change what is measured
            print(f"bench.py: spec dir unusable ({e}); compiling with the default specification", file=sys.stderr)
            module = None
    if module is None:
        module = MonoNNModule.compile(fx.hlo_text)
    module.set_constants(consts)
    module.load(0)
    dims = module.launch_dims()

    if args.stage_profile:
        stage_profile(module, fx, consts, inputs, args)
        return

    # parity of this very configuration against the oracle (also the CPU baseline's subject)
    got = module.run(inputs, fx.outputs)[0].astype(np.float32)

    if args.calibration_copy:
        a = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        b.copy_(a)
        torch.cuda.synchronize()
        del a, b

    ptrs = module.buffer_pointers()
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(args.warmup):
        module.launch_raw(ptrs, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        module.launch_raw(ptrs, stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # kernel duration by HIP events on the same stream (what rocprof's kernel trace reports)
    avg_ms, each = module.time_raw(ptrs, stream, warmup=10, iters=max(50, min(args.steps, 500)))
    each_us = np.sort(each.astype(np.float64) * 1e3)
    kern_us = float(avg_ms * 1e3)

    # cold caches: a 1 GiB fill between launches evicts L2 and the 256 MiB memory-side cache, so every weight
    # byte of the timed launch comes from HBM
    flush = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    cold = []
    for i in range(12):
        flush.fill_(i)
        torch.cuda.synchronize()
        _, one = module.time_raw(ptrs, stream, warmup=0, iters=1)
        cold.append(float(one[0]) * 1e3)
    del flush
    cold_us = float(np.median(cold[2:]))

    abytes = algorithmic_bytes(fx)
    flops = gemm_flops(fx.config)
    achieved_gbs = abytes / (kern_us * 1e-6) / 1e9
    achieved_tflops = flops / (kern_us * 1e-6) / 1e12

    result = {
        "metric": "per-forward latency (us) & seq/s, BERT-base b1 s128 fp16, 1 MI355X",
        "value": round(fx.config["B"] * 1e3 / ms_per_step, 2),
        "unit": "seq/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "BERT-base encoder, 12 layers + embedding gather, batch 1, seq 128, fp16 weights "
                               "N(0,0.02), one launch of the monolithic persistent kernel per forward",
                   "tuning_spec": used_spec, "grid": dims["grid"], "block": dims["block"], "lds_bytes": dims["smem"],
                   "grid_barriers": dims["barriers"],
                   "barrier_tiers": {"memory_side": dims["barriers"] - dims["regional_barriers"], "one_xcd": dims["regional_barriers"]}},
        "latency_us": {"kernel_avg": round(kern_us, 2), "kernel_p10": round(float(each_us[len(each_us) // 10]), 2),
                       "kernel_median": round(float(each_us[len(each_us) // 2]), 2),
                       "kernel_p90": round(float(each_us[(len(each_us) * 9) // 10]), 2),
                       "kernel_cold_caches_median": round(cold_us, 2),
                       "end_to_end_per_step": round(ms_per_step * 1e3, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved_gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved_gbs / HBM_PEAK_GBS, 5),
                     "traffic": MEASURED_TRAFFIC_BYTES if used_spec != "default" else None,
                     "algorithmic_bytes": abytes, "kernel": module.kernel_name},
        "mfma": {"achieved_tflops": round(achieved_tflops, 2), "peak_tflops": MFMA_F16_PEAK_TFLOPS,
                 "frac": round(achieved_tflops / MFMA_F16_PEAK_TFLOPS, 5), "gemm_flops": flops},
    }

    n_stages, barrier_us = barrier_time(module, fx, consts, inputs)
    result["config"]["stages"] = n_stages
    result["config"]["barrier_us_total"] = round(barrier_us, 1)

    if args.torch_baseline:
        result["torch_baseline"] = torch_baseline(fx, consts, inputs, got)
    if not args.no_other_configs:
        module.close()
        result["other_configs"] = other_configs()

    if not args.no_cpu_baseline:
        from oracle import hlo_interp
        ev = hlo_interp.Evaluator(fx.hlo_text, consts, "fp32")
        want = ev.run(inputs)[0].astype(np.float32)   # also warms the BLAS threads
        n, t0 = 0, time.perf_counter()
        while n < 3 or (time.perf_counter() - t0 < 12.0 and n < 50):
            ev.run(inputs)
            n += 1
        cpu_s = (time.perf_counter() - t0) / n
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            cores = os.cpu_count() or 1
        g, w = got.ravel().astype(np.float64), want.ravel().astype(np.float64)
        result["cpu_baseline"] = {"value": round(fx.config["B"] / cpu_s, 3), "unit": "seq/s", "cores": cores,
                                  "kind": "port",
                                  "sample": f"{n} fp32 forwards of the same HLO and inputs by the NumPy oracle "
                                            f"(multi-threaded BLAS), {cpu_s * 1e3:.1f} ms each"}
        result["parity"] = {"max_abs_err": float(np.abs(g - w).max()),
                            "cosine": float(g @ w / (np.linalg.norm(g) * np.linalg.norm(w)))}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
