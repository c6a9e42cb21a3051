"""Benchmark of the evaluation hot path: binarize + evaluate trees on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2] [--docs N]

A step is one pass of the two kernels (binarize, evaluate) over one batch of synthetic documents
that already sits in HBM. The default workload is C2: 1000 oblivious trees of depth 8, 200 fp32
features with 5 % NaN, 4M documents. Prints one JSON line.
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
# HBM bytes of one step (both launches, fetched + written), from rocprofv3 FETCH_SIZE / WRITE_SIZE
# runs scaled by a copy kernel of known size; only known for workloads that were profiled
MEASURED_TRAFFIC_BYTES = {("C2", 4000000, 1000): 6.12e9}


def cpu_baseline(model_bytes, info, target_seconds=12.0):
    """Times the CPU oracle (a port of the reference CPU evaluator) on a bounded sample."""
    import numpy as np

    from catboost_amd import synthetic as syn
    from oracle.cbm_reader import read_cbm
    from oracle.oracle import OracleModel

    oracle = OracleModel(read_cbm(model_bytes))
    threads = min(16, os.cpu_count() or 1)
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
    expected = oracle.calc(sample, threads=min(16, os.cpu_count() or 1))
    max_abs = float(np.abs(got - expected).max()) if n_check else 0.0
    ok = bool(np.allclose(got, expected, rtol=1e-9, atol=1e-12))

    used_floats = sum(1 for f in read_cbm(model_bytes)["float_features"] if len(f["borders"]))
    used_cats = sum(1 for c in read_cbm(model_bytes)["cat_features"] if c["used"])
    bytes_per_doc = 4 * used_floats + 4 * used_cats + 8 * dim
    step_bytes = bytes_per_doc * docs
    avg_bin, avg_eval = float(np.mean(bin_ms)), float(np.mean(eval_ms))
    kernels_ms = avg_bin + avg_eval
    achieved = step_bytes / (kernels_ms * 1e-3) / 1e9
    buckets = ev.bucket_count
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
            "traffic": MEASURED_TRAFFIC_BYTES.get((args.config, docs, model.tree_count)),
            "algorithmic_bytes_per_doc": bytes_per_doc,
            "kernel": "binarize + evaluate (the two launches of one step)",
        },
        "kernels": {
            "binarize": {"avg_ms": avg_bin, "GBps": (4 * (used_floats + used_cats) + buckets) * docs / (avg_bin * 1e-3) / 1e9
                         if avg_bin > 0 else None},
            "evaluate": {"avg_ms": avg_eval, "GBps": (buckets + 8 * dim) * docs / (avg_eval * 1e-3) / 1e9,
                         "tree_evals_per_sec": docs * model.tree_count / (avg_eval * 1e-3)},
        },
        "parity": {"checked_docs": int(n_check), "max_abs_err": max_abs, "within_1e-9_rel_1e-12_abs": ok},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(model_bytes, info)
        if info["kind"] == "oblivious" and dim == 1 and not info["cat_hashes"]:
            # the sampled documents of the parity check, through the reference's own scalar evaluator
            ref = reference_standalone(model_bytes, sample, got)
            if ref is not None:
                result["cpu_baseline"]["reference_standalone_evaluator"] = ref
    print(json.dumps(result))
    if not ok:
        sys.exit(1)


if __name__ == "__main__":
    main()
