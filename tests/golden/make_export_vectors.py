"""Writes tests/golden/cpp_export_{cat,nocat}.cbm and tests/golden/cpp_export_vectors.npz from the two
models that the reference holds as exported C++ code (the canonical outputs of its export tests,
catboost/python-package/ut/medium/canondata/test.test_cpp_export_{with,no}_cat_features_CPU_/model.cpp:
the tables of a trained model as static data plus the applier of
catboost/libs/model/model_export/resources/apply_catboost_model*.cpp). oracle/build_ref.sh compiles them
where they lie, with oracle/ref_export_main.cpp, into oracle/_ref/export_{cat,nocat}.

Run in the build container only (needs /root/reference for the build):
    bash oracle/build_ref.sh && python tests/golden/make_export_vectors.py

`export_* dump` prints the model's tables; they are put together into a .cbm here (tests/cbm_writer.py),
which is what the library and the oracle then read. `export_* apply` runs the reference's applier on
seeded documents; the .npz stores the documents, those predictions and, for the model with categorical
features, the arrays (bucket, split index, xor mask) per tree split that the reference's exporter wrote
into the code (what TModelTrees' RepackedBins hold, catboost/libs/model/model.cpp:543-576).

What the exported code does not carry: the flat positions of the features (floats are placed first
here), the classifier index of a CTR base (numbered here per projection and type, in order of appearance)
and NaN treatment (no document has a NaN). A hashed categorical value outside the code's own
string -> hash table is an unknown category for that applier. It answers an unknown category with
Calc(0, 0) for Counter CTRs where the evaluator answers Calc(0, denominator)
(static_ctr_provider.cpp:63-75); the stored mask `comparable` is false for documents with such a lookup.
"""
import json
import os
import struct
import subprocess
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import cbm_writer  # noqa: E402
import ctr_models  # noqa: E402

GOLDEN = os.path.join(ROOT, "tests", "golden")
DOCS = 3000
MASK64 = (1 << 64) - 1


def index_hash(pairs):
    """TDenseIndexHashView buckets (dense_hash_view.h:12-66) for (hash, row) pairs."""
    size = 2
    while size < 2 * max(len(pairs), 1):
        size *= 2
    hashes, rows = [MASK64] * size, [0xFFFFFFFF] * size
    for key, row in pairs:
        z = key & (size - 1)
        while hashes[z] != MASK64:
            z = (z + 1) & (size - 1)
        hashes[z], rows[z] = key, row
    return np.frombuffer(b"".join(struct.pack("<QI", h, r) for h, r in zip(hashes, rows)), np.uint8).copy()


def model_from_dump(d, name):
    n_float, n_cat = d["float_feature_count"], d["cat_feature_count"]
    floats = [{"has_nans": False, "index": i, "flat_index": i, "borders": np.asarray(b, np.float32),
               "feature_id": "", "nan_treatment": 0} for i, b in enumerate(d["float_feature_borders"])]
    assert len(floats) == n_float
    cat_index = d.get("cat_features_index", [])
    cats = [{"index": int(c), "flat_index": n_float + j, "feature_id": "", "used": True}
            for j, c in enumerate(cat_index)]
    one_hots = [{"cat_index": int(c), "values": np.asarray(v, np.int32), "string_values": []}
                for c, v in zip(d.get("one_hot_cat_feature_index", []), d.get("one_hot_hash_values", []))]
    ctrs, tables, classifier_of = [], [], {}
    for p in d.get("projections", []):
        assert not p["binarized_indexes"], "projection with float or one-hot splits: not handled here"
        cat_features = np.asarray([cat_index[t] for t in p["transposed_cat_feature_indexes"]], np.int32)
        for c in p["ctrs"]:
            key = (tuple(cat_features), c["type"])
            seen = classifier_of.setdefault(key, {})
            classifier = seen.setdefault(c["base_hash"], len(seen))
            base = {"cat_features": cat_features, "float_splits": [], "one_hot_splits": [],
                    "ctr_type": c["type"], "target_border_classifier_idx": classifier}
            ctrs.append({"base": base, "target_border_idx": c["target_border_idx"],
                         "prior_num": np.float32(c["prior_num"]), "prior_denom": np.float32(c["prior_denom"]),
                         "shift": np.float32(c["shift"]), "scale": np.float32(c["scale"]),
                         "borders": np.asarray(d["ctr_feature_borders"][len(ctrs)], np.float32),
                         "_base_hash": c["base_hash"]})
    done = set()
    for c in ctrs:
        h = c.pop("_base_hash")
        if h in done:
            continue
        done.add(h)
        t = d["tables"][h]
        tables.append({"base": c["base"], "index_hash_raw": index_hash([(int(k), int(r)) for k, r in t["index"]]),
                       "ctr_blob": np.frombuffer(np.asarray(t["total"], np.int32).tobytes(), np.uint8).copy(),
                       "counter_denominator": t["counter_denominator"],
                       "target_classes_count": t["target_classes_count"]})
    sizes = np.asarray(d["tree_depth"], np.int32)
    return {
        "info": {"source": "reference canondata %s" % name}, "model_part_ids": ["static_provider_v1"] if tables else [],
        "approx_dimension": d["dimension"], "tree_splits": np.asarray(d["tree_splits"], np.int32),
        "tree_sizes": sizes, "tree_start_offsets": (np.cumsum(sizes) - sizes).astype(np.int32),
        "cat_features": cats, "float_features": floats, "one_hot_features": one_hots,
        "ctr_feature_count": len(ctrs), "ctr_features": ctrs,
        "leaf_values": np.asarray(d["leaf_values"], np.float64), "leaf_weights": np.zeros(0),
        "step_nodes": np.zeros((0, 2), np.uint16), "node_id_to_leaf_id": np.zeros(0, np.uint32),
        "text_feature_count": 0, "estimated_feature_count": 0, "embedding_feature_count": 0,
        "scale": d["scale"], "bias": np.asarray(d["biases"], np.float64), "ctr_tables": tables,
    }


def documents(d, seed):
    """Floats around and on the borders; categorical values that the feature's own tables know (a feature
    without a table of its own takes any of the model's values), one in 25 unknown."""
    rng = np.random.default_rng(seed)
    floats = np.zeros((DOCS, d["float_feature_count"]), np.float32)
    for i, borders in enumerate(d["float_feature_borders"]):
        b = np.asarray(borders, np.float32)
        if not b.size:
            floats[:, i] = rng.normal(size=DOCS)
            continue
        lo, hi = float(b.min()), float(b.max())
        span = max(hi - lo, 1.0)
        floats[:, i] = rng.uniform(lo - 0.2 * span, hi + 0.2 * span, size=DOCS)
        on = rng.random(DOCS) < 0.3  # exactly on a border: the compare is strict
        floats[on, i] = b[rng.integers(0, b.size, size=int(on.sum()))]
    known = np.asarray(sorted(d.get("cat_feature_hashes", {}).values()), np.int32)
    cats = np.zeros((DOCS, d["cat_feature_count"]), np.int32)
    if known.size:
        for j in range(cats.shape[1]):
            # the values of this feature: those that a table over the feature alone holds
            keys = set()
            for p in d["projections"]:
                if p["transposed_cat_feature_indexes"] == [j]:
                    for c in p["ctrs"]:
                        keys |= set(int(k) for k, _ in d["tables"][c["base_hash"]]["index"])
            own = np.asarray([h for h in known if ctr_models.projection_hash([h], [], []) in keys], np.int32)
            values = own if own.size else known
            cats[:, j] = values[rng.integers(0, values.size, size=DOCS)]
        unknown = rng.random(cats.shape) < 0.04
        cats[unknown] = rng.integers(-2 ** 31, 2 ** 31, size=int(unknown.sum()), dtype=np.int64).astype(np.int32)
        cats[np.isin(cats, known) & unknown] = 0x7FFFFFFF
    return floats, cats


def apply_reference(exe, floats, cats):
    with tempfile.TemporaryDirectory() as tmp:
        src, dst = os.path.join(tmp, "in.bin"), os.path.join(tmp, "out.f64")
        with open(src, "wb") as f:
            f.write(struct.pack("<I", floats.shape[0]))
            for row_f, row_c in zip(floats, cats):
                f.write(row_f.tobytes() + row_c.tobytes())
        subprocess.check_call([exe, "apply", src, dst])
        return np.fromfile(dst, np.float64)


def counter_lookups_found(model, d, cats):
    """Per document: every Counter / FeatureFreq CTR of the model finds its row."""
    position = {int(c): j for j, c in enumerate(d.get("cat_features_index", []))}
    ok = np.ones(cats.shape[0], bool)
    for t in model["ctr_tables"]:
        if t["base"]["ctr_type"] not in (4, 5):
            continue
        raw = t["index_hash_raw"].reshape(-1, 12)
        keys = set(int(k) for k in raw[:, :8].copy().view(np.uint64).ravel() if int(k) != MASK64)
        for doc in range(cats.shape[0]):
            h = ctr_models.projection_hash([cats[doc, position[int(c)]] for c in t["base"]["cat_features"]], [], [])
            ok[doc] &= h in keys
    return ok


def main():
    out = {}
    for name, with_cats in (("cat", True), ("nocat", False)):
        exe = os.path.join(ROOT, "oracle", "_ref", "export_" + name)
        if not os.path.exists(exe):
            raise SystemExit("%s is missing: run oracle/build_ref.sh where /root/reference is mounted" % exe)
        d = json.loads(subprocess.check_output([exe, "dump"]))
        model = model_from_dump(d, "test_cpp_export_%s_cat_features" % ("with" if with_cats else "no"))
        with open(os.path.join(GOLDEN, "cpp_export_%s.cbm" % name), "wb") as f:
            f.write(cbm_writer.write_cbm(model))
        floats, cats = documents(d, 7 if with_cats else 8)
        out["floats_" + name] = floats
        out["cats_" + name] = cats
        out["predictions_" + name] = apply_reference(exe, floats, cats)
        out["comparable_" + name] = counter_lookups_found(model, d, cats)
        if with_cats:
            out["split_bucket_cat"] = np.asarray(d["tree_split_feature_index"], np.uint16)
            out["split_idx_cat"] = np.asarray(d["tree_split_idxs"], np.uint8)
            out["split_xor_mask_cat"] = np.asarray(d["tree_split_xor_mask"], np.uint8)
            strings = sorted(d["cat_feature_hashes"])
            out["hash_strings_cat"] = np.asarray(strings)
            out["hash_values_cat"] = np.asarray([d["cat_feature_hashes"][s] for s in strings], np.int32)
        print("%s: %d trees, %d ctrs, %d documents, %d comparable" % (
            name, len(model["tree_sizes"]), len(model["ctr_features"]), DOCS, int(out["comparable_" + name].sum())))
    np.savez_compressed(os.path.join(GOLDEN, "cpp_export_vectors.npz"), **out)


if __name__ == "__main__":
    main()
