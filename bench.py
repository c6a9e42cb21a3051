"""Benchmark of the evaluation hot path: binarize + evaluate trees on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2] [--docs N]

A step is one pass of the two kernels (binarize, evaluate) over one batch of synthetic documents
that already sits in HBM. The default workload is C2: 1000 oblivious trees of depth 8, 200 fp32
features with 5 % NaN, 4M documents. Prints one JSON line. The default run (C2, no --docs) then gives the other
four workloads of the baseline (C1, C3, C4, C5 at their full sizes) five steps each, outside the timed region of the
C2 figure, and reports them under "other_workloads" (kernel times from HIP events, parity of 2000 sampled
documents against the oracle).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
# HBM-side bytes of one step (fetched + written) come from rocprofv3 FETCH_SIZE / WRITE_SIZE runs scaled by a copy
# kernel of known size. They are not measured in this run: the line carries the figure that a profile summary
# holds for exactly this workload and these kernels (a line "TRAFFIC <config> <docs> <trees> <kernels> <bytes>"
# in the file below), and null otherwise.
TRAFFIC_PROFILE = os.path.join("profiles", "c2_hbm_traffic_pmc.txt")


def measured_traffic(config, docs, trees, kernels):
    """(bytes per step, source) from the profile summary, or (None, None) when it holds no matching line."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    if not os.path.exists(path):
        return None, None
    wanted = "+".join(kernels[k] for k in sorted(kernels))
    with open(path) as f:
        for line in f:
            parts = line.split()
            if len(parts) == 6 and parts[0] == "TRAFFIC" and parts[1] == config and int(parts[2]) == docs and \
                    int(parts[3]) == trees and parts[4] == wanted:
                return float(parts[5]), TRAFFIC_PROFILE
    return None, None


def end_to_end_c_abi(model, info, docs):
    """CalcModelPredictionFlat (the reference API: one pointer per row, host memory in and out) on a bounded
    sample: rows gathered into pinned memory, copied over PCIe, evaluated, results copied back."""
    import numpy as np

    from catboost_amd import synthetic as syn

    docs = int(min(docs, 1_000_000))
    x = syn.host_features(info, docs, seed=9)
    model.calc_flat(x[:1000])
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        model.calc_flat(x)
        elapsed = time.perf_counter() - t0
        best = elapsed if best is None else min(best, elapsed)
    return {"docs_per_sec": docs / best, "sample": "%d docs of the same workload, best of 3 calls, %.1f ms" % (docs, best * 1e3),
            "host_to_device_GBps": docs * x.shape[1] * 4 / best / 1e9}


def host_threads():
    """Worker threads for the CPU legs: every host core, unless the machine's environment caps worker pools
    (OMP_NUM_THREADS: a GPU box gives one GPU's job a share of its cores)."""
    cap = os.environ.get("OMP_NUM_THREADS", "")
    cores = os.cpu_count() or 1
    return max(1, min(cores, int(cap))) if cap.isdigit() else cores


def cpu_baseline(model_bytes, info, target_seconds=12.0):
    """Times the CPU oracle (a port of the reference CPU evaluator) on a bounded sample."""
    import numpy as np

    from catboost_amd import synthetic as syn
    from oracle.cbm_reader import read_cbm
    from oracle.oracle import OracleModel

    oracle = OracleModel(read_cbm(model_bytes))
    threads = host_threads()
    docs = int(min(info["docs"], 400_000))
    x = syn.host_features(info, docs, seed=6)
    t0 = time.perf_counter()
    oracle.calc(x, threads=threads)
    probe = time.perf_counter() - t0
    repeats = int(max(1, min(200, round(target_seconds / max(probe, 1e-6)))))
    t0 = time.perf_counter()
    for _ in range(repeats):
        oracle.calc(x, threads=threads)
    elapsed = time.perf_counter() - t0
    total = docs * repeats
    # one thread, on a smaller sample (about 3 s)
    single_docs = min(docs, 20_000)
    t0 = time.perf_counter()
    oracle.calc(x[:single_docs], threads=1)
    single_probe = time.perf_counter() - t0
    single_repeats = int(max(1, min(50, round(3.0 / max(single_probe, 1e-6)))))
    t0 = time.perf_counter()
    for _ in range(single_repeats):
        oracle.calc(x[:single_docs], threads=1)
    single_elapsed = time.perf_counter() - t0
    return {
        "value": total / elapsed,
        "unit": "docs/sec",
        "cores": threads,
        "host_cpu_count": os.cpu_count(),
        "kind": "port",
        "sample": "%d docs of the same workload evaluated %d times, %d threads over 128-doc blocks, %.1f s" % (
            docs, repeats, threads, elapsed),
        "tree_evals_per_sec": total * oracle.tree_count / elapsed,
        "single_thread_docs_per_sec": single_docs * single_repeats / single_elapsed,
    }


def reference_standalone(model_bytes, rows, gpu_values):
    """Times the reference's own standalone evaluator (catboost/libs/standalone_evaluator, built from the
    reference's sources into oracle/_ref/standalone_eval by oracle/build_ref.sh; one scalar thread, float-only
    oblivious one-dimensional models) on `rows` and compares what it prints with the GPU's values.
    Returns None where the binary is not there."""
    import subprocess
    import tempfile

    import numpy as np

    exe = os.path.join(ROOT, "oracle", "_ref", "standalone_eval")
    if not os.path.exists(exe):
        return None
    with tempfile.TemporaryDirectory() as tmp:
        model_path = os.path.join(tmp, "model.cbm")
        with open(model_path, "wb") as f:
            f.write(model_bytes)
        seconds, printed = [], None
        # two sizes: their difference takes the process start and the model load out of the rate
        for count in (rows.shape[0] // 10, rows.shape[0]):
            docs_path = os.path.join(tmp, "docs_%d.f32" % count)
            np.ascontiguousarray(rows[:count], np.float32).tofile(docs_path)
            t0 = time.perf_counter()
            printed = subprocess.run([exe, "apply", model_path, docs_path, str(count)], check=True,
                                     stdout=subprocess.PIPE).stdout
            seconds.append(time.perf_counter() - t0)
    values = np.array(printed.split(), dtype=np.float64)
    rate = (rows.shape[0] - rows.shape[0] // 10) / max(seconds[1] - seconds[0], 1e-9)
    return {"docs_per_sec": rate, "cores": 1, "sample": "%d docs of the same workload, %.1f s" % (rows.shape[0], seconds[1]),
            "max_abs_diff_gpu_vs_reference": float(np.abs(values - gpu_values).max())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="C2")
    ap.add_argument("--docs", type=int, default=0, help="override the document count of the workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-end-to-end", action="store_true", help="skip the CalcModelPredictionFlat figure")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short runs of C1, C3, C4 and C5 that follow the default C2 run")
    ap.add_argument("--check-docs", type=int, default=20000)
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run one device-to-device copy of this many MiB (a kernel of known traffic, used to "
                         "scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (documents would be sharded "
              "across GPUs without any exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import catboost_amd as cb
    from catboost_amd import synthetic as syn

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    result, ok, context = measure_workload(args.config, args.docs, args.steps, args.warmup, args.check_docs, args.copy_probe_mib)
    model, info, docs, model_bytes, sample, got = context
    if not args.no_other_workloads and args.config == "C2" and not args.docs:
        # the other four workloads of the baseline, outside the timed region of the headline figure: a few steps
        # each at their full sizes, the same measurement (HIP events around a step's kernels, a sample of the
        # output against the oracle)
        del context
        others = {}
        for name in ("C1", "C3", "C4", "C5"):
            r, other_ok, other_context = measure_workload(name, 0, 5, 2, 2000, 0)
            del other_context
            torch.cuda.empty_cache()
            others[name] = {"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "docs_per_sec": r["value"],
                            "kernel_ms": r["roofline"]["kernel_ms"], "frac": r["roofline"]["frac"],
                            "kernels": {k: {"name": v["name"], "avg_ms": v["avg_ms"]} for k, v in r["kernels"].items()},
                            "parity": r["parity"]}
            ok = ok and other_ok
        result["other_workloads"] = others
    if not args.no_end_to_end:
        result["end_to_end_c_abi"] = end_to_end_c_abi(model, info, docs)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(model_bytes, info)
        if info["kind"] == "oblivious" and info["dim"] == 1 and not info["cat_hashes"]:
            # the sampled documents of the parity check, through the reference's own scalar evaluator
            ref = reference_standalone(model_bytes, sample, got)
            if ref is not None:
                result["cpu_baseline"]["reference_standalone_evaluator"] = ref
    print(json.dumps(result))
    if not ok:
        sys.exit(1)


def measure_workload(config, docs_override, steps, warmup, check_docs, copy_probe_mib):
    """One workload: `warmup` untimed and `steps` timed steps on documents that sit in HBM, and the parity of a
    sample of the output against the oracle. Returns (the JSON fields, parity ok, what the callers' other legs need)."""
    import numpy as np
    import torch

    import catboost_amd as cb
    from catboost_amd import synthetic as syn

    class args:  # the names the body below uses
        pass
    args.config, args.docs, args.steps, args.warmup, args.check_docs, args.copy_probe_mib = (
        config, docs_override, steps, warmup, check_docs, copy_probe_mib)
    model, info = syn.build_model(args.config)
    model.enable_gpu_evaluation(0)
    docs = args.docs or info["docs"]
    dim = info["dim"]
    ev = model.evaluator()
    x = syn.device_features(info, docs)
    out = torch.zeros(docs * dim, dtype=torch.float64, device="cuda:0")
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    torch.cuda.synchronize()

    if args.copy_probe_mib:
        probe_src = torch.ones(args.copy_probe_mib << 18, dtype=torch.float32, device="cuda:0")
        probe_dst = torch.empty_like(probe_src)
        torch.cuda.synchronize()
        probe_dst.copy_(probe_src)
        torch.cuda.synchronize()
        del probe_src, probe_dst

    for _ in range(args.warmup):
        ev.eval_data(feats, docs, out.data_ptr())
    torch.cuda.synchronize()
    bin_ms, eval_ms = [], []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ev.eval_data(feats, docs, out.data_ptr())  # returns after the step's kernels finished
        b, e = ev.last_kernel_times()
        bin_ms.append(b)
        eval_ms.append(e)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    # parity of a sample of the timed output against the CPU oracle
    model_bytes = model.save_to_buffer()
    from oracle.cbm_reader import read_cbm
    from oracle.oracle import OracleModel

    oracle = OracleModel(read_cbm(model_bytes))
    n_check = min(args.check_docs, docs)
    idx = torch.randperm(docs, device="cuda:0")[:n_check].sort().values
    sample = x[idx].cpu().numpy()
    got = out.view(docs, dim)[idx].cpu().numpy().ravel()
    expected = oracle.calc(sample, threads=host_threads())
    max_abs = float(np.abs(got - expected).max()) if n_check else 0.0
    ok = bool(np.allclose(got, expected, rtol=1e-9, atol=1e-12))

    model_dict = read_cbm(model_bytes)
    used_borders = sorted(len(f["borders"]) for f in model_dict["float_features"] if len(f["borders"]))
    used_floats = len(used_borders)
    used_cats = sum(1 for c in model_dict["cat_features"] if c["used"])
    bytes_per_doc = 4 * used_floats + 4 * used_cats + 8 * dim
    step_bytes = bytes_per_doc * docs
    avg_bin, avg_eval = float(np.mean(bin_ms)), float(np.mean(eval_ms))
    # the kernels of a step run back to back on one stream: the two intervals share their middle event, so
    # their sum is the time from the step's first event to its last (a fused kernel reports one interval)
    kernels_ms = avg_bin + avg_eval
    achieved = step_bytes / (kernels_ms * 1e-3) / 1e9
    buckets = ev.bucket_count
    kernel_names = ev.describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    traffic, traffic_source = measured_traffic(args.config, docs, model.tree_count, kernel_names)
    if "fused" in kernel_names:
        kernels = {"fused": {"name": kernel_names["fused"], "avg_ms": kernels_ms,
                             "tree_evals_per_sec": docs * model.tree_count / (kernels_ms * 1e-3)}}
    else:
        kernels = {
            "binarize": {"name": kernel_names["binarize"], "avg_ms": avg_bin,
                         "GBps": (4 * (used_floats + used_cats) + buckets) * docs / (avg_bin * 1e-3) / 1e9 if avg_bin > 0 else None},
            "evaluate": {"name": kernel_names["evaluate"], "avg_ms": avg_eval,
                         "GBps": (buckets + 8 * dim) * docs / (avg_eval * 1e-3) / 1e9,
                         "tree_evals_per_sec": docs * model.tree_count / (avg_eval * 1e-3)},
        }
    result = {
        "metric": "docs/sec (binarize + evaluate, %d trees, %d docs)" % (model.tree_count, docs),
        "value": docs * args.steps / elapsed,
        "unit": "docs/sec",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8 bins / f64 sums",
        "data": "synthetic",
        "config": {"workload": "%s: %s, %d trees, depth %d, %d float + %d cat features, dim %d, %d docs" % (
            args.config, info["kind"], model.tree_count, info["depth"], info["floats"], len(info["cat_hashes"]), dim,
            docs)},
        "tree_evals_per_sec": docs * model.tree_count * args.steps / elapsed,
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "algorithmic_bytes_per_doc": bytes_per_doc,
            "kernel": " + ".join(kernel_names[k] for k in sorted(kernel_names)),
            "kernel_ms": kernels_ms,
        },
        "kernels": kernels,
        "model": {"buckets": buckets,
                  "used_borders_per_feature": {"min": used_borders[0], "median": used_borders[len(used_borders) // 2],
                                               "max": used_borders[-1]} if used_borders else None},
        "parity": {"checked_docs": int(n_check), "max_abs_err": max_abs, "within_1e-9_rel_1e-12_abs": ok},
    }
    del x, out
    return result, ok, (model, info, docs, model_bytes, sample, got)


if __name__ == "__main__":
    main()
