"""Hand-built models and expected outputs of the reference's own unit tests, as plain data.

Each model dict has the keys of oracle.cbm_reader.read_cbm. Sources:
  catboost/libs/model/ut/lib/model_test_helpers.cpp:186-224 (SimpleFloatModel), :305-319
  (SimpleDeepTreeModel), :321-388 (SimpleAsymmetricModel), :458-490 (MultiValueFloatModel);
  expected values catboost/libs/model/ut/formula_evaluator_ut.cpp:16-25, 76-146, 284-307.
"""
import numpy as np

from oracle import model_builder as mb

# formula_evaluator_ut.cpp:16-25
DATA = np.array([
    [0, 0, 0], [3, 0, 0], [0, 1, 0], [3, 1, 0],
    [0, 0, 1], [3, 0, 1], [0, 1, 1], [3, 1, 1]], dtype=np.float32)


def _raw(float_features, tree_splits, tree_sizes, leaf_values, dim=1, scale=1.0, bias=None):
    starts = np.concatenate([[0], np.cumsum(tree_sizes)[:-1]]).astype(np.int32) if len(tree_sizes) else np.zeros(0, np.int32)
    return {
        "approx_dimension": dim,
        "tree_splits": np.asarray(tree_splits, np.int32),
        "tree_sizes": np.asarray(tree_sizes, np.int32),
        "tree_start_offsets": starts,
        "float_features": float_features, "cat_features": [], "one_hot_features": [],
        "leaf_values": np.asarray(leaf_values, np.float64), "leaf_weights": np.zeros(0),
        "step_nodes": np.zeros((0, 2), np.uint16), "node_id_to_leaf_id": np.zeros(0, np.uint32),
        "scale": scale, "bias": np.zeros(dim) if bias is None else np.asarray(bias, np.float64),
        "info": {}, "model_part_ids": [], "ctr_feature_count": 0, "text_feature_count": 0,
        "estimated_feature_count": 0, "embedding_feature_count": 0,
    }


def _ff(index, borders):
    f = mb.float_feature(index)
    f["borders"] = np.asarray(borders, np.float32)
    return f


def simple_float_model(tree_count=1, scale=1.0, bias=None):
    """Feature 0 has 301 borders -298..2 (two buckets), features 1 and 2 one border 0.5; every
    tree splits on bin features {300, 301, 302}; leaf values leaf * 10^tree."""
    ffs = [_ff(0, [-298.0 + i for i in range(301)]), _ff(1, [0.5]), _ff(2, [0.5])]
    splits, sizes, leaves = [], [], []
    ten = 1.0
    for _ in range(tree_count):
        splits += [300, 301, 302]
        sizes.append(3)
        leaves += [leaf * ten for leaf in range(8)]
        ten *= 10.0
    return _raw(ffs, splits, sizes, leaves, scale=scale, bias=bias)


def simple_deep_tree_model(depth=9):
    ffs = [_ff(i, [0.5]) for i in range(depth)]
    return _raw(ffs, list(range(depth)), [depth], [float(v) for v in range(1 << depth)])


def deep_tree_data(depth=9):
    n = 1 << depth
    data = np.zeros((n, depth), np.float32)
    for s in range(n):
        for f in range(depth):
            data[s, f] = (s >> f) & 1
    return data


def multi_value_float_model():
    ffs = [_ff(0, [0.5]), _ff(1, [0.5])]
    leaves = [0., 10., 20., 1., 11., 21., 2., 12., 22., 3., 13., 23.]
    return _raw(ffs, [0, 1], [2], leaves, dim=3)


def simple_asymmetric_trees():
    """The three trees of SimpleAsymmetricModel as builder input."""
    t0 = mb.split_node(("float", 0, 0.5),
                       mb.split_node(("float", 1, 0.5), mb.leaf_node(1.0), mb.leaf_node(2.0)),
                       mb.leaf_node(3.0))
    t1 = mb.split_node(("float", 2, 0.5), mb.leaf_node(0.0), mb.leaf_node(10.0))
    t2 = mb.split_node(("float", 0, 0.5),
                       mb.leaf_node(100.0),
                       mb.split_node(("float", 1, 0.5), mb.leaf_node(200.0), mb.leaf_node(300.0)))
    return [mb.float_feature(i) for i in range(3)], [t0, t1, t2]


def simple_asymmetric_model():
    ffs, heads = simple_asymmetric_trees()
    return mb.build_non_symmetric(ffs, [], 1, heads)


# formula_evaluator_ut.cpp:286-299
ASYMMETRIC_PREDICTIONS = np.array([101., 203., 102., 303., 111., 213., 112., 313.])
ASYMMETRIC_LEAF_INDEXES = np.array([
    [1, 0, 0], [0, 0, 1], [2, 0, 0], [0, 0, 2],
    [1, 1, 0], [0, 1, 1], [2, 1, 0], [0, 1, 2]], dtype=np.uint32)

# golden predictions held by the binding tests of the reference
NUMERIC_ONLY_ROWS = np.array([[0.1, 0.3, 0.2], [0.5, 1.5, -2.5], [0.7, 6.4, 2.4], [-2.0, -1.0, 6.0]], np.float32)
# CatBoostModelTest.java:290, 344-347
NUMERIC_ONLY_EXPECTED = np.array([0.029172098906116373, 0.03547209874741901, 0.008157865240661602,
                                  0.009992472030400074])

# rust-package/src/model.rs:325-350 (exact equality asserted there)
RUST_FLOATS = np.array([[-10.0, 5.0, 753.0], [30.0, 1.0, 760.0], [40.0, 0.1, 705.0]], np.float32)
RUST_CATS = [["north"], ["south"], ["south"]]
RUST_EXPECTED = np.array([0.9980003729960197, 0.00249414628534181, -0.0013677527881450977])

# rust-package/src/model.rs:422-456 (tolerance 1e-6 there), node-package/bindings/tests/model.ts:51-56
QUERYWISE_ROWS_TEXT = [
    "0.257727	0.0215909	0.171299	1	1	1	1	1	0	0	0	0	0	0	0.431373	0.935065	0.0208333	0.070824	1	0	0.313726	1	1	0	0.937724	0	1	0	0	0	0	0.0566038	0	0	1	0.73929	1	0.000505391	0.885819	0.000172727	0	0	0	0	0	0	0.153262	0.578118	0.222098	1",
    "0.424438	0.164384	0.572649	1	1	0	1	0	0	1	0	0	0	0	0.360784	0.512195	0.0447049	0.0717587	1	1	0.321569	1	1	0	0.941214	0	1	0	0	0	0	0.275362	1	0.209302	1	0.391239	1	0.0143194	0.885819	0.00140996	0	0	0	0	0	0	0.357143	0.883721	0.820312	1",
    "0.345548	0.248034	0.0853067	1	1	0	1	0	0	1	0	0	0	0	0.6	0.5	0.114292	0.071371	1	0	0.396078	1	1	0	0.939218	0	1	0	0	0	0	0.0384615	0	0	1	0	0	0	0.885819	0.00224069	0	0	0	0	0	0	0.588235	0.444444	0.608696	1",
    "0.946305	0.139752	0.429885	1	1	1	1	1	0	1	0	0	0	0	0.811765	0.75	0.119755	0.071636	0	1	0.541176	1	1	0	0.993828	0	1	0	0	0	0	0.509804	1	0.000398	1	1.5	1	0.417659	0.885819	0.00117792	0	0	0	0	0	0	0.52962	0.958103	0.885843	1",
]
QUERYWISE_EXPECTED = np.array([0.08819508860736715, 0.043193651033534904, -0.0019333444540111586,
                               0.0836685835428004])


def querywise_rows():
    return np.array([[float(x) for x in row.split("\t")] for row in QUERYWISE_ROWS_TEXT], dtype=np.float32)


# CatBoostModelTest.java:122-134
HASH_KNOWN_ANSWERS = {"foo": -553946371, "bar": 50123586, "baz": 825262476, "\U0001F621": 11426516}


def load_iris(golden_dir):
    """iris.data rows -> (features float32 [150, 4], label index)."""
    import os
    names = ["Iris-setosa", "Iris-versicolor", "Iris-virginica"]
    feats, labels = [], []
    with open(os.path.join(golden_dir, "iris.data")) as f:
        for line in f:
            parts = line.strip().split(",")
            if len(parts) < 5:
                continue
            if parts[-1] not in names:
                continue  # header row
            feats.append([float(x) for x in parts[:4]])
            labels.append(names.index(parts[-1]))
    return np.asarray(feats, np.float32), np.asarray(labels)


def load_boston(golden_dir):
    import os
    feats, target = [], []
    with open(os.path.join(golden_dir, "boston_housing.data")) as f:
        for line in f:
            tok = line.split()
            if not tok:
                continue
            feats.append([float(x) for x in tok[:-1]])
            target.append(float(tok[-1]))
    return np.asarray(feats, np.float32), np.asarray(target)


# ---- models with CTR (target statistics) features ------------------------------------------
# categoric_only_model.cbm, CatBoostModelTest.java:528-547 (three categorical features, strings)
JVM_CATEGORIC_ONLY_CATS = [["a", "d", "g"], ["b", "e", "h"], ["c", "f", "k"]]
JVM_CATEGORIC_ONLY_EXPECTED = np.array([0.04146251510837989, 0.015486266021159064, 0.04146251510837989])
# model.cbm of the JVM tests (here jvm_model_with_ctr.cbm), CatBoostModelTest.java:720-743
JVM_CTR_FLOATS = np.array([[0.5, 1.5], [0.7, 6.4], [-2.0, -1.0]], np.float32)
JVM_CTR_CATS = JVM_CATEGORIC_ONLY_CATS
JVM_CTR_EXPECTED = np.array([0.04666924366060905, 0.026244613740247648, 0.03094452158737013])
# features_num_cat__dataset_adult.cbm, rust-package/src/model.rs:459-499 (tolerance there: 1e-6)
RUST_ADULT_FLOATS = np.array([[44.0, 403782.0, 11.0, 0.0, 0.0, 45.0], [19.0, 208874.0, 10.0, 0.0, 0.0, 40.0],
                              [27.0, 158647.0, 10.0, 0.0, 0.0, 40.0], [18.0, 115258.0, 6.0, 0.0, 0.0, 40.0]], np.float32)
RUST_ADULT_CATS = [["0", "n", "1", "Private", "Assoc-voc", "Divorced", "Sales", "Not-in-family", "White", "Male",
                    "United-States"]] * 4
RUST_ADULT_EXPECTED = np.array([0.9876043724015489, 0.9869589576174197, 0.997648058191363, 1.0147797830459155])
# node-package/test_data/adult.cbm (here node_adult.cbm), node-package/bindings/tests/model.ts:67-96:
# predictions printed with two decimals
NODE_ADULT_FLOATS = np.array([[40., 85019., 16., 0., 0., 45.], [28., 85019., 13., 0., 0., 13.]], np.float32)
NODE_ADULT_CATS = [["Private", "Doctorate", "Married-civ-spouce", "Prof-specialty", "Husband", "Asian-Pac-Islander",
                    "Male", "nan"],
                   ["Self-emp-not-inc", "Bachelors", "Married-civ-spouce", "Exec-managerial", "Husband", "White", "Male",
                    "United-States"]]
NODE_ADULT_EXPECTED_2DP = ["1.54", "-1.17"]


def mushrooms(golden_dir):
    """mushrooms.csv of the .NET tests (CatBoostModelEvaluatorTest.cs:101-127): label, then 22 categorical
    features; the model's raw prediction is positive exactly for label "p"."""
    import os
    labels, rows = [], []
    with open(os.path.join(golden_dir, "mushrooms.csv")) as f:
        for line in f:
            parts = line.strip().split(",")
            if len(parts) == 23:
                labels.append(parts[0])
                rows.append(parts[1:])
    return labels, rows


CTR_FIXTURES = ["categoric_only_model.cbm", "jvm_model_with_ctr.cbm", "features_num_cat__dataset_adult.cbm",
                "node_adult.cbm", "mushroom_model.cbm", "cloudness_small.cbm"]


def random_ctr_inputs(model, docs, seed, known_cats=None):
    """Random documents for a model dict with CTR features: floats around the model's borders and
    categorical hashes drawn from the hashes the CTR tables know (plus unknown ones)."""
    rng = np.random.default_rng(seed)
    ffs, cfs = model["float_features"], model["cat_features"]
    n_float = max([f["index"] for f in ffs], default=-1) + 1
    n_cat = max([c["index"] for c in cfs], default=-1) + 1
    floats = rng.normal(size=(docs, n_float)).astype(np.float32)
    for f in ffs:
        b = np.asarray(f["borders"], np.float32)
        if b.size:
            pick = b[rng.integers(0, b.size, size=docs)]
            jitter = rng.choice(np.array([-1.0, 0.0, 1.0], np.float32), size=docs) * np.abs(pick) * 1e-3
            floats[:, f["index"]] = pick + jitter.astype(np.float32)
    cats = rng.integers(-2 ** 31, 2 ** 31, size=(docs, n_cat), dtype=np.int64).astype(np.int32)
    if known_cats is not None:
        for c in cfs:
            pool = known_cats.get(c["index"])
            if pool is not None and len(pool):
                use = rng.random(docs) < 0.9
                cats[use, c["index"]] = np.asarray(pool, np.int32)[rng.integers(0, len(pool), size=int(use.sum()))]
    return floats, cats


def known_cat_hashes(model):
    """Per categorical feature index: hashed values its single-feature CTR tables have rows for. A table
    key of such a projection is MAGIC * (0 + MAGIC * (u64)(i32)hash) (catboost/libs/model/hash.h:11-14);
    MAGIC is odd, so the key is inverted modulo 2^64."""
    magic = 0x4906ba494954cb65
    inv = pow(magic, -1, 1 << 64)
    inv2 = (inv * inv) % (1 << 64)
    out = {}
    for table in model.get("ctr_tables", []):
        base = table["base"]
        if len(base["cat_features"]) != 1 or base["float_splits"] or base["one_hot_splits"]:
            continue
        raw = np.asarray(table["index_hash_raw"], np.uint8).reshape(-1, 12)
        keys = raw[:, :8].copy().view(np.uint64).ravel()
        values = []
        for key in keys:
            if int(key) == 0xFFFFFFFFFFFFFFFF:
                continue
            v = (int(key) * inv2) % (1 << 64)
            if v >= 1 << 63:
                v -= 1 << 64
            if -2 ** 31 <= v < 2 ** 31:
                values.append(v)
        out.setdefault(int(base["cat_features"][0]), set()).update(values)
    return {k: sorted(v) for k, v in out.items()}


def flat_rows(model, floats, cats):
    """[doc][flat feature index] rows from split float / hashed categorical matrices (hashes bit-cast)."""
    ffs, cfs = model["float_features"], model["cat_features"]
    width = max([f["flat_index"] for f in ffs] + [c["flat_index"] for c in cfs], default=-1) + 1
    flat = np.zeros((floats.shape[0] if floats.size or not len(cats) else cats.shape[0], width), np.float32)
    for f in ffs:
        flat[:, f["flat_index"]] = floats[:, f["index"]]
    for c in cfs:
        flat[:, c["flat_index"]] = np.ascontiguousarray(cats[:, c["index"]]).view(np.float32)
    return flat


def model_to_json(model):
    """A model dict in CatBoost's "json" model format, as ConvertModelToJson writes it
    (catboost/libs/model/model_export/json_model_helpers.cpp:293-364, 469-498): the keys the importer
    reads."""
    import json

    dim = int(model["approx_dimension"])
    leaves = np.asarray(model["leaf_values"], np.float64)
    doc = {"model_info": dict(model.get("info", {})), "features_info": {}}
    if model["float_features"]:
        doc["features_info"]["float_features"] = [
            {"has_nans": bool(f["has_nans"]), "feature_index": int(f["index"]), "flat_feature_index": int(f["flat_index"]),
             "borders": [float(b) for b in np.asarray(f["borders"], np.float32)], "feature_id": f.get("feature_id", ""),
             "nan_value_treatment": ["AsIs", "AsFalse", "AsTrue"][int(f["nan_treatment"])]}
            for f in model["float_features"]]
    if model["cat_features"]:
        one_hot = {int(o["cat_index"]): o for o in model["one_hot_features"]}
        cats = []
        for c in model["cat_features"]:
            item = {"feature_index": int(c["index"]), "flat_feature_index": int(c["flat_index"]),
                    "feature_id": c.get("feature_id", "")}
            if int(c["index"]) in one_hot:
                item["values"] = [int(v) for v in one_hot[int(c["index"])]["values"]]
            cats.append(item)
        doc["features_info"]["categorical_features"] = cats
    steps = np.asarray(model["step_nodes"]).reshape(-1, 2)
    if len(steps) == 0:
        trees, first = [], 0
        for t, depth in enumerate(model["tree_sizes"]):
            begin = int(model["tree_start_offsets"][t])
            count = (1 << int(depth)) * dim
            trees.append({"leaf_values": [float(v) for v in leaves[first:first + count]],
                          "splits": [{"split_index": int(s)} for s in model["tree_splits"][begin:begin + int(depth)]]})
            first += count
        doc["oblivious_trees"] = trees
    else:
        leaf_of = np.asarray(model["node_id_to_leaf_id"])

        def leaf(node):
            values = leaves[int(leaf_of[node]):int(leaf_of[node]) + dim]
            return {"value": float(values[0]) if dim == 1 else [float(v) for v in values]}

        def node_json(node):
            left, right = int(steps[node][0]), int(steps[node][1])
            if left == 0 and right == 0:
                return leaf(node)
            return {"split": {"split_index": int(model["tree_splits"][node])},
                    "left": node_json(node + left) if left else leaf(node),
                    "right": node_json(node + right) if right else leaf(node)}

        doc["trees"] = [node_json(int(start)) for start in model["tree_start_offsets"]]
    doc["scale_and_bias"] = [float(model["scale"]), [float(b) for b in np.asarray(model["bias"], np.float64)]]
    if model.get("ctr_features"):
        # ToJson(TCtrFeature) and ConvertCtrsToJson, json_model_helpers.cpp:105-117, 433-485
        type_names = ["Borders", "Buckets", "BinarizedTargetMeanValue", "FloatTargetMeanValue", "Counter", "FeatureFreq"]

        def elements(base):
            items = [{"cat_feature_index": int(c), "combination_element": "cat_feature_value"} for c in base["cat_features"]]
            items += [{"float_feature_index": int(f), "border": float(np.float32(b)), "combination_element": "float_feature"}
                      for f, b in base["float_splits"]]
            items += [{"cat_feature_index": int(f), "value": int(v), "combination_element": "cat_feature_exact_value"}
                      for f, v in base["one_hot_splits"]]
            return items

        def identifier(base):
            return json.dumps({"type": type_names[int(base["ctr_type"])], "identifier": elements(base)})

        doc["features_info"]["ctrs"] = [
            {"identifier": identifier(c["base"]), "elements": elements(c["base"]),
             "ctr_type": type_names[int(c["base"]["ctr_type"])], "prior_numerator": float(c["prior_num"]),
             "prior_denomerator": float(c["prior_denom"]), "shift": float(c["shift"]), "scale": float(c["scale"]),
             "target_border_idx": int(c["target_border_idx"]), "borders": [float(b) for b in np.asarray(c["borders"], np.float32)]}
            for c in model["ctr_features"]]
        data = {}
        for t in model.get("ctr_tables", []):
            kind = int(t["base"]["ctr_type"])
            raw = np.asarray(t["index_hash_raw"], np.uint8).reshape(-1, 12)
            keys = raw[:, :8].copy().view(np.uint64).ravel()
            rows = raw[:, 8:].copy().view(np.uint32).ravel()
            blob = np.asarray(t["ctr_blob"], np.uint8)
            flat = []
            for k, r in zip(keys, rows):
                if int(k) == 0xFFFFFFFFFFFFFFFF:
                    continue
                flat.append(str(int(k)))
                if kind in (2, 3):
                    flat.append(float(blob[8 * r:8 * r + 4].view(np.float32)[0]))
                    flat.append(int(blob[8 * r + 4:8 * r + 8].view(np.int32)[0]))
                elif kind in (4, 5):
                    flat.append(int(blob[4 * r:4 * r + 4].view(np.int32)[0]))
                else:
                    n = int(t["target_classes_count"])
                    flat += [int(v) for v in blob[4 * n * r:4 * n * (r + 1)].view(np.int32)]
            stride = 3 if kind in (2, 3) else 2 if kind in (4, 5) else int(t["target_classes_count"]) + 1
            data[identifier(t["base"])] = {"hash_map": flat, "hash_stride": stride,
                                           "counter_denominator": int(t["counter_denominator"])}
        doc["ctr_data"] = data
    return json.dumps(doc)
