"""Restatement of the reference model builders for the CPU oracle. TEST INFRASTRUCTURE ONLY.

Follows catboost/libs/model/model_build_helper.cpp:100-126 (ProcessSplitsSet), :144-204
(TObliviousTreeBuilder), :206-304 (TNonSymmetricTreeModelBuilder), catboost/libs/model/model.cpp:181-236
(TModelTrees::ProcessSplitsSet) and :634-674 (ConvertObliviousToAsymmetric). Split ordering is
that of TModelSplit::operator< (catboost/libs/model/split.h:69-87): float splits before one-hot
splits, float splits by (feature index, border), one-hot splits by (cat feature index, value).

A split is ("float", float_feature_index, border) or ("onehot", cat_feature_index, value).
The result is a model dict with the same keys as oracle.cbm_reader.read_cbm.
"""
import numpy as np


def float_feature(index, flat_index=None, has_nans=False, nan_treatment=0, feature_id=""):
    return {"index": index, "flat_index": index if flat_index is None else flat_index,
            "has_nans": has_nans, "nan_treatment": nan_treatment, "feature_id": feature_id,
            "borders": np.zeros(0, np.float32)}


def cat_feature(index, flat_index, feature_id=""):
    return {"index": index, "flat_index": flat_index, "feature_id": feature_id, "used": False}


def _split_key(s):
    if s[0] == "float":
        return (0, int(s[1]), float(np.float32(s[2])))
    return (2, int(s[1]), int(s[2]))


def _process_splits_set(split_keys, float_features, cat_features):
    """Returns (float_features, cat_features, one_hot_features, {split key: bin feature index})."""
    ffs = [dict(f, borders=[]) for f in float_features]
    cfs = [dict(c, used=False) for c in cat_features]
    ff_by_index = {f["index"]: i for i, f in enumerate(ffs)}
    cf_by_index = {c["index"]: i for i, c in enumerate(cfs)}
    one_hot = []
    ordered = sorted(split_keys)
    for key in ordered:
        if key[0] == 0:
            ffs[ff_by_index[key[1]]]["borders"].append(np.float32(key[2]))
        else:
            cfs[cf_by_index[key[1]]]["used"] = True
            if not one_hot or one_hot[-1]["cat_index"] != key[1]:
                one_hot.append({"cat_index": key[1], "values": [], "string_values": []})
            one_hot[-1]["values"].append(key[2])
    for f in ffs:
        f["borders"] = np.asarray(f["borders"], dtype=np.float32)
    for o in one_hot:
        o["values"] = np.asarray(o["values"], dtype=np.int32)
    return ffs, cfs, one_hot, {k: i for i, k in enumerate(ordered)}


def _finish(model, approx_dim, scale, bias):
    model["approx_dimension"] = approx_dim
    model["scale"] = float(scale)
    model["bias"] = np.zeros(approx_dim) if bias is None else np.asarray(bias, dtype=np.float64)
    model["leaf_weights"] = np.zeros(0)
    model["info"] = {}
    model["model_part_ids"] = []
    model["ctr_feature_count"] = 0
    model["text_feature_count"] = 0
    model["estimated_feature_count"] = 0
    model["embedding_feature_count"] = 0
    return model


def build_oblivious(float_features, cat_features, approx_dim, trees, scale=1.0, bias=None):
    """trees: list of (splits, leaf_values) with leaf_values laid out [leaf * approx_dim + k]."""
    keys = set()
    for splits, _ in trees:
        for s in splits:
            keys.add(_split_key(s))
    ffs, cfs, one_hot, ids = _process_splits_set(keys, float_features, cat_features)
    tree_splits, tree_sizes, tree_starts, leaves = [], [], [], []
    for splits, leaf_values in trees:
        assert len(leaf_values) == (1 << len(splits)) * approx_dim
        tree_starts.append(len(tree_splits))
        tree_splits.extend(ids[_split_key(s)] for s in splits)
        tree_sizes.append(len(splits))
        leaves.append(np.asarray(leaf_values, dtype=np.float64))
    model = {
        "tree_splits": np.asarray(tree_splits, dtype=np.int32),
        "tree_sizes": np.asarray(tree_sizes, dtype=np.int32),
        "tree_start_offsets": np.asarray(tree_starts, dtype=np.int32),
        "float_features": ffs, "cat_features": cfs, "one_hot_features": one_hot,
        "leaf_values": np.concatenate(leaves) if leaves else np.zeros(0),
        "step_nodes": np.zeros((0, 2), np.uint16),
        "node_id_to_leaf_id": np.zeros(0, np.uint32),
    }
    return _finish(model, approx_dim, scale, bias)


def split_node(split, left, right):
    return ("split", split, left, right)


def leaf_node(value):
    return ("leaf", value)


def build_non_symmetric(float_features, cat_features, approx_dim, tree_heads, scale=1.0, bias=None):
    """tree_heads: nested split_node(...) / leaf_node(value or vector) structures."""
    flat_splits, flat_value_idx, flat_steps, values = [], [], [], []
    tree_sizes, tree_starts = [], []
    keys = set()

    def insert_value(node):
        flat_value_idx.append(len(values))
        v = node[1]
        if np.isscalar(v):
            assert approx_dim == 1
            values.append(float(v))
        else:
            assert len(v) == approx_dim
            values.extend(float(x) for x in v)

    def add_node(node):
        node_id = len(flat_steps)
        if node[0] == "split":
            _, split, left, right = node
            keys.add(_split_key(split))
            flat_splits.append(_split_key(split))
            flat_steps.append(None)
            if (left[0] == "split") == (right[0] == "split"):
                flat_value_idx.append(0xFFFFFFFF)
                lid = add_node(left)
                rid = add_node(right)
                flat_steps[node_id] = (lid - node_id, rid - node_id)
            elif right[0] == "split":
                insert_value(left)
                flat_steps[node_id] = (0, add_node(right) - node_id)
            else:
                insert_value(right)
                flat_steps[node_id] = (add_node(left) - node_id, 0)
        else:
            flat_splits.append(None)
            flat_steps.append((0, 0))
            insert_value(node)
        return node_id

    for head in tree_heads:
        prev = len(flat_splits)
        tree_starts.append(prev)
        add_node(head)
        tree_sizes.append(len(flat_splits) - prev)
    ffs, cfs, one_hot, ids = _process_splits_set(keys, float_features, cat_features)
    model = {
        "tree_splits": np.asarray([0 if s is None else ids[s] for s in flat_splits], dtype=np.int32),
        "tree_sizes": np.asarray(tree_sizes, dtype=np.int32),
        "tree_start_offsets": np.asarray(tree_starts, dtype=np.int32),
        "float_features": ffs, "cat_features": cfs, "one_hot_features": one_hot,
        "leaf_values": np.asarray(values, dtype=np.float64),
        "step_nodes": np.asarray(flat_steps, dtype=np.uint16).reshape(-1, 2),
        "node_id_to_leaf_id": np.asarray(flat_value_idx, dtype=np.uint32),
    }
    return _finish(model, approx_dim, scale, bias)


def convert_oblivious_to_asymmetric(model):
    """TModelTrees::ConvertObliviousToAsymmetric, model.cpp:634-674."""
    assert len(model["step_nodes"]) == 0
    dim = model["approx_dimension"]
    tree_splits, tree_sizes, tree_starts, steps, node_to_leaf = [], [], [], [], []
    leaf_start = 0
    for t, depth_n in enumerate(model["tree_sizes"]):
        size = 0
        start = model["tree_start_offsets"][t]
        tree_starts.append(len(tree_splits))
        for depth in range(depth_n):
            split = model["tree_splits"][start + depth_n - 1 - depth]
            for _ in range(1 << depth):
                tree_splits.append(split)
                node_to_leaf.append(0xFFFFFFFF)
                steps.append((size + 1, size + 2))
                size += 1
        for clone in range(1 << depth_n):
            tree_splits.append(0)
            node_to_leaf.append((leaf_start + clone) * dim)
            steps.append((0, 0))
            size += 1
        leaf_start += 1 << depth_n
        tree_sizes.append(size)
    out = dict(model)
    out["tree_splits"] = np.asarray(tree_splits, dtype=np.int32)
    out["tree_sizes"] = np.asarray(tree_sizes, dtype=np.int32)
    out["tree_start_offsets"] = np.asarray(tree_starts, dtype=np.int32)
    out["step_nodes"] = np.asarray(steps, dtype=np.uint16).reshape(-1, 2)
    out["node_id_to_leaf_id"] = np.asarray(node_to_leaf, dtype=np.uint32)
    return out
