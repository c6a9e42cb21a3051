"""Throughput of a model on this machine's GPU, in the spirit of the reference's model_perftest tool
(catboost/tools/model_perftest/lib/main.cpp:165-330: --model-path, --block-size, --threads, --repetitions;
it times the evaluator's entry points block by block over a pool).

    python -m catboost_amd.perftest -m model.cbm [--pool-path pool.tsv] [--docs N] [--block-size B]
                                    [--repetitions R] [--threads T] [--model-format cbm|json] [--device-id D]
                                    [--graph]

Without a pool the documents are random: floats around the model's borders, categorical hashes at random.
A pool is a tab-separated file of flat feature rows (categorical columns as strings). Reports documents
per second of the host entry points (rows by pointer, columns by pointer, leaf indexes; PCIe both ways) and of the device entry points
on features that already sit in HBM; with --graph also of a block's quantize + evaluate launches captured
once into a HIP graph and replayed per block (what a serving loop with small blocks does). With
--threads T above 1 the host entry points are also timed from T caller threads at once, each going through
all blocks (one model handle: calls from several threads are allowed and run on staging contexts of their own).
"""
import argparse
import json
import sys
import time

import numpy as np

import catboost_amd as cb


def _feature_positions(model):
    """Flat indexes of the model's float and categorical features."""
    return model.get_float_feature_indices(), model.get_cat_feature_indices()


def _random_rows(model, docs, seed):
    floats, cats = _feature_positions(model)
    width = max(floats + cats, default=-1) + 1
    rng = np.random.default_rng(seed)
    rows = rng.normal(size=(docs, width)).astype(np.float32)
    for c in cats:
        rows[:, c] = rng.integers(-2 ** 31, 2 ** 31, size=docs, dtype=np.int64).astype(np.int32).view(np.float32)
    return rows


def _pool_rows(model, path):
    floats, cats = _feature_positions(model)
    width = max(floats + cats, default=-1) + 1
    rows = []
    with open(path) as f:
        for line in f:
            parts = line.rstrip("\n").split("\t")
            if len(parts) < width:
                raise cb.CatBoostError("pool row has %d columns, the model needs %d" % (len(parts), width))
            row = np.zeros(width, np.float32)
            for i in floats:
                row[i] = np.float32(parts[i]) if parts[i] != "" else np.float32("nan")
            for i in cats:
                row[i:i + 1] = np.array([cb.string_cat_feature_hash(parts[i])], np.int32).view(np.float32)
            rows.append(row)
    return np.array(rows, np.float32).reshape(len(rows), width)


def run(args):
    import torch

    model = cb.ModelCalcer(args.model_path, model_format=args.model_format)
    model.enable_gpu_evaluation(args.device_id)
    rows = _pool_rows(model, args.pool_path) if args.pool_path else _random_rows(model, args.docs, args.seed)
    docs = rows.shape[0]
    block = min(args.block_size or docs, docs)
    if block <= 0:
        raise cb.CatBoostError("Empty pool")
    blocks = [rows[b:b + block] for b in range(0, docs - block + 1, block)]
    report = {"model": args.model_path, "trees": model.tree_count, "dimensions": model.dimensions_count, "docs": docs,
              "block_size": block, "repetitions": args.repetitions}

    model.calc_flat(blocks[0])  # binds the model to the device, uploads its tables
    # the host entry point families: rows by pointer, columns by pointer, leaf indexes of rows by pointer
    transposed = [np.ascontiguousarray(b.T) for b in blocks]
    leaf_docs = max(1, min(block, (64 << 20) // max(1, 4 * model.tree_count)))  # bounds the index matrix of a call
    entry_points = {
        "host_flat": (lambda i: model.calc_flat(blocks[i]), block),
        "host_transposed": (lambda i: model.calc_flat_transposed(transposed[i]), block),
        "host_leaf_indexes": (lambda i: model.calc_leaf_indexes_flat(blocks[i][:leaf_docs]), leaf_docs),
    }
    for name, (call, docs_per_call) in entry_points.items():
        call(0)
        start = time.perf_counter()
        for _ in range(args.repetitions):
            for i in range(len(blocks)):
                call(i)
        seconds = time.perf_counter() - start
        report[name + "_docs_per_sec"] = args.repetitions * len(blocks) * docs_per_call / seconds

    if args.threads > 1:
        import threading

        report["threads"] = args.threads
        for name, (call, docs_per_call) in entry_points.items():
            # every caller thread goes through all blocks: the calls of one handle run side by side on
            # staging contexts of their own
            failures = []

            def caller():
                try:
                    for _ in range(args.repetitions):
                        for i in range(len(blocks)):
                            call(i)
                except Exception as e:  # reported by the main thread
                    failures.append(e)

            callers = [threading.Thread(target=caller) for _ in range(args.threads)]
            start = time.perf_counter()
            for t in callers:
                t.start()
            for t in callers:
                t.join()
            seconds = time.perf_counter() - start
            if failures:
                raise failures[0]
            report[name + "_threads_docs_per_sec"] = args.threads * args.repetitions * len(blocks) * docs_per_call / seconds

    ev = model.evaluator()
    device = "cuda:%d" % args.device_id
    resident = [torch.from_numpy(np.ascontiguousarray(b)).to(device) for b in blocks]
    out = torch.zeros(block * ev.dim, dtype=torch.float64, device=device)
    torch.cuda.synchronize()
    feats = [ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]) for x in resident]
    ev.eval_data(feats[0], block, out.data_ptr())
    ev.synchronize()
    start = time.perf_counter()
    for _ in range(args.repetitions):
        for f in feats:
            ev.eval_data(f, block, out.data_ptr())
    ev.synchronize()
    seconds = time.perf_counter() - start
    report["device_docs_per_sec"] = args.repetitions * len(blocks) * block / seconds
    binarize_ms, evaluate_ms = ev.last_kernel_times()
    report["last_block_kernel_ms"] = {"binarize": binarize_ms, "evaluate": evaluate_ms}

    if args.graph:
        # quantize + evaluate of one block captured once into a HIP graph (the quantized-data entry points
        # only launch kernels); a call is then a copy into the captured input buffer and a replay
        captured_in = resident[0].clone()
        bins = torch.zeros(ev.quantized_bytes(block), dtype=torch.uint8, device=device)
        captured = ev.features(cb.LAYOUT_FLAT_ROWS, captured_in.data_ptr(), captured_in.shape[1])

        def launch(stream):
            ev.quantize(captured, block, bins.data_ptr(), stream=stream)
            ev.eval_quantized(bins.data_ptr(), block, out.data_ptr(), stream=stream)

        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            launch(side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            launch(torch.cuda.current_stream().cuda_stream)
        stream = torch.cuda.current_stream()
        start = time.perf_counter()
        for _ in range(args.repetitions):
            for x in resident:
                captured_in.copy_(x, non_blocking=True)
                graph.replay()
                stream.synchronize()  # like eval_data, a call ends when its results are there
        seconds = time.perf_counter() - start
        report["graph_replay_docs_per_sec"] = args.repetitions * len(blocks) * block / seconds
    return report


def main(argv=None):
    parser = argparse.ArgumentParser(prog="python -m catboost_amd.perftest", description=__doc__.split("\n\n")[0])
    parser.add_argument("-m", "--model-path", required=True)
    parser.add_argument("--model-format", default="cbm", choices=["cbm", "json"])
    parser.add_argument("-f", "--pool-path")
    parser.add_argument("--docs", type=int, default=1_000_000, help="random documents when no pool is given")
    parser.add_argument("--block-size", type=int, default=0, help="documents per call (default: all)")
    parser.add_argument("--repetitions", type=int, default=10)
    parser.add_argument("-T", "--threads", type=int, default=1, help="caller threads for the host entry point")
    parser.add_argument("--graph", action="store_true", help="also time the block as a replayed HIP graph")
    parser.add_argument("--device-id", type=int, default=0)
    parser.add_argument("--seed", type=int, default=0)
    args = parser.parse_args(argv)
    print(json.dumps(run(args)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
