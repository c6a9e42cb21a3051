"""Seeded synthetic models with CTR features of every kind, for the oracle and the HIP evaluator.

The reference's binding tests only hold models with Borders and Counter CTRs over categorical
features. The models made here also carry Buckets, BinarizedTargetMeanValue, FloatTargetMeanValue and
FeatureFreq CTRs, tables with more than two target classes, and projections that mix categorical
features with float splits and one-hot splits (TFeatureCombination, catboost/libs/model/online_ctr.h:108-170).
A model is the dict that oracle/cbm_reader.read_cbm returns; tests/cbm_writer.py turns it into a .cbm.
"""
import struct

import numpy as np

MAGIC = 0x4906ba494954cb65  # catboost/libs/model/hash.h:9
MASK64 = (1 << 64) - 1


def calc_hash(a, b):
    """CalcHash, catboost/libs/model/hash.h:11-14."""
    return (MAGIC * ((a + MAGIC * b) & MASK64)) & MASK64


def projection_hash(cat_values, float_bits, one_hot_bits):
    """Hash of a projection's values: hashed categorical values as (ui64)(int), then one bit per float
    split and per one-hot split (ctr_provider.h:94-123)."""
    h = 0
    for v in cat_values:
        h = calc_hash(h, int(v) & MASK64)
    for bit in list(float_bits) + list(one_hot_bits):
        h = calc_hash(h, int(bit))
    return h


def build_index_hash(keys):
    """Buckets of a TDenseIndexHashView (catboost/libs/helpers/dense_hash_view.h:12-66): a power of two
    of {ui64 hash, ui32 row} buckets, linear probing from hash & (size - 1), empty hash = all ones."""
    size = 2
    while size < 2 * max(len(keys), 1):
        size *= 2
    hashes = [MASK64] * size
    rows = [0xFFFFFFFF] * size
    for row, key in enumerate(keys):
        z = key & (size - 1)
        while hashes[z] != MASK64:
            z = (z + 1) & (size - 1)
        hashes[z], rows[z] = key, row
    return np.frombuffer(b"".join(struct.pack("<QI", h, r) for h, r in zip(hashes, rows)), np.uint8).copy()


def random_ctr_model(seed, n_float=4, n_cat=4, n_bases=8, n_trees=40, max_depth=6, wide_float=False, dim=1):
    """Returns (model dict, known values per categorical feature index)."""
    rng = np.random.default_rng(seed)
    floats = []
    for i in range(n_float):
        count = 300 if (wide_float and i == 0) else int(rng.integers(1, 12))
        borders = np.unique(rng.normal(size=count).astype(np.float32))
        if i == n_float - 1 and n_float > 2:
            borders = np.zeros(0, np.float32)  # a feature the model does not use
        floats.append({"has_nans": False, "index": i, "flat_index": i, "borders": borders,
                       "feature_id": "f%d" % i, "nan_treatment": 0})
    cats = [{"index": j, "flat_index": n_float + j, "feature_id": "c%d" % j, "used": True} for j in range(n_cat)]
    known = {j: np.unique(rng.integers(-2 ** 31, 2 ** 31, size=int(rng.integers(3, 12)), dtype=np.int64))
             for j in range(n_cat)}
    one_hots = []
    for j in range(n_cat):
        if j % 2 == 0:
            take = max(1, len(known[j]) // 2)
            one_hots.append({"cat_index": j, "values": rng.permutation(known[j])[:take].astype(np.int32),
                             "string_values": []})
    used_floats = [f for f in floats if f["borders"].size]

    # ---- tables: one per (projection, type, classifier)
    tables, ctrs = [], []
    projections = []
    for b in range(n_bases):
        if b % 3 == 1 and projections:
            proj = projections[-1]  # same projection, another type: shares the hash with the previous one
        else:
            k = int(rng.integers(1, min(3, n_cat) + 1))
            proj = {"cat_features": np.sort(rng.choice(n_cat, size=k, replace=False)).astype(np.int32),
                    "float_splits": [], "one_hot_splits": []}
            if b % 2 == 0:
                for _ in range(int(rng.integers(1, 3))):
                    f = used_floats[int(rng.integers(0, len(used_floats)))]
                    pick = int(rng.integers(0, f["borders"].size))
                    if wide_float and f["index"] == 0:
                        pick = [254, 260, f["borders"].size - 1, 253, 3][b // 2 % 5]  # both sides of bin 254
                    proj["float_splits"].append((f["index"], np.float32(f["borders"][pick])))
                proj["float_splits"] = sorted(set(proj["float_splits"]))
            if b % 4 >= 2 and one_hots:
                o = one_hots[int(rng.integers(0, len(one_hots)))]
                proj["one_hot_splits"].append((o["cat_index"], int(o["values"][int(rng.integers(0, o["values"].size))])))
        projections.append(proj)
        ctr_type = int(b % 6) if b < 6 else int(rng.integers(0, 6))
        base = dict(proj, ctr_type=ctr_type, target_border_classifier_idx=int(rng.integers(0, 2)))
        while any(_same_base(base, t["base"]) for t in tables):
            base["target_border_classifier_idx"] += 2
        keys = set()
        for _ in range(int(rng.integers(20, 200))):
            values = [known[int(c)][int(rng.integers(0, len(known[int(c)])))] for c in proj["cat_features"]]
            keys.add(projection_hash(values, rng.integers(0, 2, size=len(proj["float_splits"])),
                                     rng.integers(0, 2, size=len(proj["one_hot_splits"]))))
        keys = sorted(keys)
        rng.shuffle(keys)
        rows = len(keys)
        classes, denominator = 0, 0
        if ctr_type in (0, 1):
            classes = int(rng.choice([2, 2, 3, 5])) if ctr_type == 0 else int(rng.choice([1, 2, 3, 5]))
            blob = rng.integers(0, 60, size=(rows, classes), dtype=np.int64).astype(np.int32)
        elif ctr_type in (2, 3):
            blob = np.zeros(rows, np.dtype([("sum", "<f4"), ("count", "<i4")]))
            blob["count"] = rng.integers(0, 80, size=rows)
            blob["sum"] = (rng.random(rows) * blob["count"]).astype(np.float32)
        else:
            denominator = int(rng.integers(50, 1000))
            blob = rng.integers(0, denominator + 1, size=rows, dtype=np.int64).astype(np.int32)
        tables.append({"base": base, "index_hash_raw": build_index_hash(keys),
                       "ctr_blob": np.frombuffer(blob.tobytes(), np.uint8).copy(),
                       "counter_denominator": denominator, "target_classes_count": classes})
        for _ in range(int(rng.integers(1, 3))):
            if ctr_type == 0:
                target = int(rng.integers(0, max(classes - 1, 1)))
            elif ctr_type == 1:
                target = int(rng.integers(0, classes))
            else:
                target = 0
            shift, scale = np.float32(rng.choice([0.0, -0.25, -0.5])), np.float32(rng.choice([1.0, 15.0, 3.5]))
            lo, hi = float(shift * scale), float((1 + shift) * scale)
            ctrs.append({"base": base, "target_border_idx": target,
                         "prior_num": np.float32(rng.choice([0.0, 0.5, 1.0])),
                         "prior_denom": np.float32(rng.choice([1.0, 2.0])), "shift": shift, "scale": scale,
                         "borders": np.unique(rng.uniform(lo, hi, size=int(rng.integers(1, 7))).astype(np.float32))})

    # ---- trees over all binary features: float borders, one-hot values, CTR borders in this order
    n_bin = (sum(f["borders"].size for f in floats) + sum(o["values"].size for o in one_hots) +
             sum(c["borders"].size for c in ctrs))
    first_ctr_bin = n_bin - sum(c["borders"].size for c in ctrs)
    tree_splits, tree_sizes, tree_starts, leaves = [], [], [], []
    for _ in range(n_trees):
        depth = int(rng.integers(1, max_depth + 1))
        tree_starts.append(len(tree_splits))
        for _ in range(depth):
            if rng.random() < 0.6:
                tree_splits.append(int(rng.integers(first_ctr_bin, n_bin)))
            else:
                tree_splits.append(int(rng.integers(0, n_bin)))
        tree_sizes.append(depth)
        leaves.append(rng.normal(size=(1 << depth) * dim))
    model = {
        "info": {"generator": "tests/ctr_models.py seed %d" % seed}, "model_part_ids": ["static_provider_v1"],
        "approx_dimension": dim,
        "tree_splits": np.asarray(tree_splits, np.int32), "tree_sizes": np.asarray(tree_sizes, np.int32),
        "tree_start_offsets": np.asarray(tree_starts, np.int32),
        "cat_features": cats, "float_features": floats, "one_hot_features": one_hots,
        "ctr_feature_count": len(ctrs), "ctr_features": ctrs,
        "leaf_values": np.concatenate(leaves), "leaf_weights": np.zeros(0),
        "step_nodes": np.zeros((0, 2), np.uint16), "node_id_to_leaf_id": np.zeros(0, np.uint32),
        "text_feature_count": 0, "estimated_feature_count": 0, "embedding_feature_count": 0,
        "scale": 1.0, "bias": np.zeros(dim), "ctr_tables": tables,
    }
    return model, {j: v.astype(np.int32) for j, v in known.items()}


def _same_base(a, b):
    return (list(a["cat_features"]) == list(b["cat_features"]) and
            [(f, np.float32(x).tobytes()) for f, x in a["float_splits"]] ==
            [(f, np.float32(x).tobytes()) for f, x in b["float_splits"]] and
            list(a["one_hot_splits"]) == list(b["one_hot_splits"]) and a["ctr_type"] == b["ctr_type"] and
            a["target_border_classifier_idx"] == b["target_border_classifier_idx"])


def random_documents(model, known, docs, seed):
    """(floats [doc][float index], hashed cats [doc][cat index]): floats on and around the borders, hashed
    values mostly from the known ones."""
    rng = np.random.default_rng(seed)
    n_float = len(model["float_features"])
    n_cat = len(model["cat_features"])
    floats = rng.normal(size=(docs, n_float)).astype(np.float32)
    for f in model["float_features"]:
        b = f["borders"]
        if b.size:
            on = rng.random(docs) < 0.3
            floats[on, f["index"]] = b[rng.integers(0, b.size, size=int(on.sum()))]
    cats = rng.integers(-2 ** 31, 2 ** 31, size=(docs, n_cat), dtype=np.int64).astype(np.int32)
    for j in range(n_cat):
        use = rng.random(docs) < 0.85
        cats[use, j] = known[j][rng.integers(0, len(known[j]), size=int(use.sum()))]
    return floats, cats


# (seed, keyword arguments of random_ctr_model): the cases of tests/golden/ctr_ref_vectors.npz
CASES = [
    (1, {}),
    (2, {"n_bases": 12, "n_trees": 60}),
    (3, {"wide_float": True, "n_float": 3, "n_bases": 10}),
    (4, {"n_cat": 2, "n_float": 2, "n_bases": 6, "max_depth": 8}),
    (5, {"n_cat": 6, "n_bases": 18, "dim": 3}),
]
