"""Writes tests/golden/synthetic_ctr_<seed>.cbm and tests/golden/ctr_ref_vectors.npz: CTR values that the
reference's own CTR calculator for exported models (catboost/libs/model/model_export/resources/
ctr_structs.cpp + ctr_calcer.cpp, built where they lie by oracle/build_ref.sh into oracle/_ref/ctr_calc)
computes on the seeded synthetic models of tests/ctr_models.py.

Run in the build container only (needs /root/reference for the build):
    bash oracle/build_ref.sh && python tests/golden/make_ctr_vectors.py

What goes into the reference code: the projections (positions of the hashed categorical values, the
(bin, compare kind, value) of every float and one-hot split as TStaticCtrProvider::SetupBinFeatureIndexes
derives them, static_ctr_provider.cpp:139-170, restated here), the CTRs, the value tables (hash -> row
pairs and rows), and per document the bins of the float and one-hot features plus the hashed categorical
values. What comes out: one float per document and CTR. Stored per case: the documents and those floats.

That calculator answers a hash that a table does not hold with Calc(0, 0) for every CTR type, while
the evaluator's TStaticCtrProvider::CalcCtrs (static_ctr_provider.cpp:63-75) answers Calc(0, denominator)
for Counter and FeatureFreq; the stored mask `comparable` is false for exactly those (document, CTR) pairs.
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import cbm_writer  # noqa: E402
import ctr_models  # noqa: E402
from oracle.cbm_reader import ctr_base_key  # noqa: E402
from oracle.oracle import OracleModel  # noqa: E402

EXE = os.path.join(ROOT, "oracle", "_ref", "ctr_calc")
GOLDEN = os.path.join(ROOT, "tests", "golden")
MAX_VALUES_PER_BIN = 254
DOCS = 600


def f32_word(x):
    return int(np.array([x], np.float32).view(np.uint32)[0])


def i32_word(x):
    return int(x) & 0xFFFFFFFF


def bin_feature_indexes(model):
    """SetupBinFeatureIndexes: {(float index, border bits): (bin, 0, value)}, {(cat index, value): (bin, 1, value)}."""
    current = 0
    float_indexes, one_hot_indexes = {}, {}
    for f in model["float_features"]:
        borders = np.asarray(f["borders"], np.float32)
        if not borders.size:
            continue
        for b in range(borders.size):
            float_indexes[(f["index"], borders[b].tobytes())] = (current + b // MAX_VALUES_PER_BIN, 0,
                                                                 b % MAX_VALUES_PER_BIN + 1)
        current += (borders.size + MAX_VALUES_PER_BIN - 1) // MAX_VALUES_PER_BIN
    for o in model["one_hot_features"]:
        for v, value in enumerate(o["values"]):
            one_hot_indexes[(o["cat_index"], int(value))] = (current + v // MAX_VALUES_PER_BIN, 1,
                                                             v % MAX_VALUES_PER_BIN + 1)
        current += (len(o["values"]) + MAX_VALUES_PER_BIN - 1) // MAX_VALUES_PER_BIN
    return float_indexes, one_hot_indexes


def reference_ctrs(model, bins, cats):
    """Runs oracle/_ref/ctr_calc; returns ([ctr][doc] values, [ctr][doc] table row found)."""
    float_indexes, one_hot_indexes = bin_feature_indexes(model)
    cat_position = {}
    for c in model["cat_features"]:
        if c.get("used", True):
            cat_position[c["index"]] = len(cat_position)
    table_of = {ctr_base_key(t["base"]): i for i, t in enumerate(model["ctr_tables"])}
    ctrs = model["ctr_features"]
    words = [len(ctrs)]  # one projection per CTR: sharing a projection changes no value
    for c in ctrs:
        base = c["base"]
        words.append(len(base["cat_features"]))
        words += [cat_position[int(x)] for x in base["cat_features"]]
        splits = [float_indexes[(f, np.float32(b).tobytes())] for f, b in base["float_splits"]]
        splits += [one_hot_indexes[(f, int(v))] for f, v in base["one_hot_splits"]]
        words.append(len(splits))
        for s in splits:
            words += list(s)
        words += [1, table_of[ctr_base_key(base)], int(base["ctr_type"]), i32_word(c["target_border_idx"]),
                  f32_word(c["prior_num"]), f32_word(c["prior_denom"]), f32_word(c["shift"]), f32_word(c["scale"])]
    words.append(len(model["ctr_tables"]))
    key_sets = []
    for i, t in enumerate(model["ctr_tables"]):
        raw = np.asarray(t["index_hash_raw"], np.uint8).reshape(-1, 12)
        keys = raw[:, :8].copy().view(np.uint64).ravel()
        rows = raw[:, 8:].copy().view(np.uint32).ravel()
        held = keys != np.uint64(0xFFFFFFFFFFFFFFFF)
        key_sets.append(set(int(k) for k in keys[held]))
        words += [i, i32_word(t["target_classes_count"]), i32_word(t["counter_denominator"]), int(held.sum())]
        for k, r in zip(keys[held], rows[held]):
            words += [int(k) & 0xFFFFFFFF, int(k) >> 32, int(r)]
        blob = np.asarray(t["ctr_blob"], np.uint8)
        if t["base"]["ctr_type"] in (2, 3):
            words.append(blob.size // 8)
            words += [int(w) for w in blob.view(np.uint32)]
            words.append(0)
        else:
            words.append(0)
            words.append(blob.size // 4)
            words += [int(w) for w in blob.view(np.uint32)]
    docs = bins.shape[0]
    words += [docs, bins.shape[1], len(cat_position)]
    used_cats = [c["index"] for c in model["cat_features"] if c.get("used", True)]
    per_doc = np.concatenate([bins.astype(np.uint32), cats[:, used_cats].astype(np.int32).view(np.uint32)], axis=1)
    with tempfile.TemporaryDirectory() as tmp:
        src, dst = os.path.join(tmp, "in.words"), os.path.join(tmp, "out.f32")
        with open(src, "wb") as f:
            f.write(np.asarray(words, np.uint32).tobytes())
            f.write(np.ascontiguousarray(per_doc).tobytes())
        subprocess.check_call([EXE, src, dst])
        values = np.fromfile(dst, np.float32).reshape(docs, len(ctrs)).T.copy()
    # which (ctr, doc) pairs found a row: recomputed from the hashes, only to build the mask
    found = np.zeros((len(ctrs), docs), bool)
    for ci, c in enumerate(ctrs):
        base = c["base"]
        splits = [float_indexes[(f, np.float32(b).tobytes())] for f, b in base["float_splits"]]
        splits += [one_hot_indexes[(f, int(v))] for f, v in base["one_hot_splits"]]
        keys = key_sets[table_of[ctr_base_key(base)]]
        for d in range(docs):
            bits = [(bins[d, s[0]] == s[2]) if s[1] else (bins[d, s[0]] >= s[2]) for s in splits]
            h = ctr_models.projection_hash([cats[d, int(x)] for x in base["cat_features"]], bits, [])
            found[ci, d] = h in keys
    return values, found


def main():
    if not os.path.exists(EXE):
        raise SystemExit("oracle/_ref/ctr_calc is missing: run oracle/build_ref.sh where /root/reference is mounted")
    out = {}
    for seed, kwargs in ctr_models.CASES:
        model, known = ctr_models.random_ctr_model(seed, **kwargs)
        with open(os.path.join(GOLDEN, "synthetic_ctr_%d.cbm" % seed), "wb") as f:
            f.write(cbm_writer.write_cbm(model))
        floats, cats = ctr_models.random_documents(model, known, DOCS, 1000 + seed)
        oracle = OracleModel(model)
        # bins of the float and one-hot features as the evaluator quantizes them; the CTR buckets that
        # follow them in a row are not looked at by any projection
        bins = oracle.binarize_doc_major(floats, cats, layout="split")
        values, found = reference_ctrs(model, bins, cats)
        counter = np.array([c["base"]["ctr_type"] in (4, 5) for c in model["ctr_features"]])
        out["floats_%d" % seed] = floats
        out["cats_%d" % seed] = cats
        out["ctrs_%d" % seed] = values
        out["comparable_%d" % seed] = found | ~counter[:, None]
        print("seed %d: %d ctrs, %d tables, %.0f%% of lookups found a row" %
              (seed, values.shape[0], len(model["ctr_tables"]), 100 * found.mean()))
    np.savez_compressed(os.path.join(GOLDEN, "ctr_ref_vectors.npz"), **out)


if __name__ == "__main__":
    main()
