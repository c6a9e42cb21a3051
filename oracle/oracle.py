"""ctypes front end of the CPU oracle (oracle/cb_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the cpu_baseline leg of
bench.py; never by the shipped package.

A model is a dict with the keys produced by oracle.cbm_reader.read_cbm or
oracle.model_builder.build_*.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcb_oracle.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "all"])
    return _LIB_PATH


class _Desc(ctypes.Structure):
    _fields_ = [
        ("approx_dim", ctypes.c_int32),
        ("n_trees", ctypes.c_int32),
        ("tree_sizes", ctypes.c_void_p),
        ("tree_start_offsets", ctypes.c_void_p),
        ("n_tree_splits", ctypes.c_int32),
        ("tree_splits", ctypes.c_void_p),
        ("n_float", ctypes.c_int32),
        ("ff_index", ctypes.c_void_p),
        ("ff_flat_index", ctypes.c_void_p),
        ("ff_has_nans", ctypes.c_void_p),
        ("ff_nan_treatment", ctypes.c_void_p),
        ("ff_border_offsets", ctypes.c_void_p),
        ("ff_borders", ctypes.c_void_p),
        ("n_cat", ctypes.c_int32),
        ("cf_index", ctypes.c_void_p),
        ("cf_flat_index", ctypes.c_void_p),
        ("cf_used", ctypes.c_void_p),
        ("n_onehot", ctypes.c_int32),
        ("oh_cat_index", ctypes.c_void_p),
        ("oh_value_offsets", ctypes.c_void_p),
        ("oh_values", ctypes.c_void_p),
        ("n_leaf_values", ctypes.c_uint64),
        ("leaf_values", ctypes.c_void_p),
        ("n_step_nodes", ctypes.c_int32),
        ("step_nodes", ctypes.c_void_p),
        ("node_id_to_leaf_id", ctypes.c_void_p),
        ("scale", ctypes.c_double),
        ("bias", ctypes.c_void_p),
        ("n_ctr", ctypes.c_int32),
        ("ctr_border_offsets", ctypes.c_void_p),
        ("ctr_borders", ctypes.c_void_p),
        ("ctr_cat_offsets", ctypes.c_void_p),
        ("ctr_cats", ctypes.c_void_p),
        ("ctr_float_offsets", ctypes.c_void_p),
        ("ctr_float_feature", ctypes.c_void_p),
        ("ctr_float_border", ctypes.c_void_p),
        ("ctr_onehot_offsets", ctypes.c_void_p),
        ("ctr_onehot_cat", ctypes.c_void_p),
        ("ctr_onehot_value", ctypes.c_void_p),
        ("ctr_type", ctypes.c_void_p),
        ("ctr_target_border_idx", ctypes.c_void_p),
        ("ctr_prior_num", ctypes.c_void_p),
        ("ctr_prior_denom", ctypes.c_void_p),
        ("ctr_shift", ctypes.c_void_p),
        ("ctr_scale", ctypes.c_void_p),
        ("ctr_table", ctypes.c_void_p),
        ("n_ctr_tables", ctypes.c_int32),
        ("table_bucket_offsets", ctypes.c_void_p),
        ("table_buckets", ctypes.c_void_p),
        ("table_blob_offsets", ctypes.c_void_p),
        ("table_blobs", ctypes.c_void_p),
        ("table_counter_denominator", ctypes.c_void_p),
        ("table_target_classes_count", ctypes.c_void_p),
    ]


class _Features(ctypes.Structure):
    _fields_ = [
        ("layout", ctypes.c_int32),
        ("floats", ctypes.c_void_p),
        ("stride", ctypes.c_size_t),
        ("cats", ctypes.c_void_p),
        ("cat_stride", ctypes.c_size_t),
    ]


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.cbo_model_create.restype = ctypes.c_void_p
        lib.cbo_model_create.argtypes = [ctypes.POINTER(_Desc), ctypes.c_char_p, ctypes.c_size_t]
        lib.cbo_model_free.argtypes = [ctypes.c_void_p]
        for name in ("cbo_bucket_count", "cbo_is_oblivious", "cbo_tree_count", "cbo_approx_dim"):
            getattr(lib, name).restype = ctypes.c_int32
            getattr(lib, name).argtypes = [ctypes.c_void_p]
        for name in ("cbo_flat_vector_expected_size", "cbo_min_float_vector_size",
                     "cbo_min_cat_vector_size", "cbo_used_cat_count"):
            getattr(lib, name).restype = ctypes.c_size_t
            getattr(lib, name).argtypes = [ctypes.c_void_p]
        lib.cbo_repacked_bins.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        lib.cbo_first_leaf_offsets.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        lib.cbo_binarize.argtypes = [ctypes.c_void_p, ctypes.POINTER(_Features), ctypes.c_size_t, ctypes.c_void_p]
        lib.cbo_calc.argtypes = [ctypes.c_void_p, ctypes.POINTER(_Features), ctypes.c_size_t,
                                 ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p]
        lib.cbo_calc_ctrs.argtypes = [ctypes.c_void_p, ctypes.POINTER(_Features), ctypes.c_size_t, ctypes.c_void_p]
        lib.cbo_calc_mt.argtypes = lib.cbo_calc.argtypes + [ctypes.c_int]
        lib.cbo_calc_leaf_indexes.argtypes = lib.cbo_calc.argtypes
        lib.cbo_calc_bruteforce.argtypes = lib.cbo_calc.argtypes + [ctypes.c_void_p]
        lib.cbo_city_hash64.restype = ctypes.c_uint64
        lib.cbo_city_hash64.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
        lib.cbo_cat_feature_hash.restype = ctypes.c_uint32
        lib.cbo_cat_feature_hash.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
        lib.cbo_integer_cat_feature_hash.restype = ctypes.c_int32
        lib.cbo_integer_cat_feature_hash.argtypes = [ctypes.c_longlong]
        lib.cbo_fast_exp_inplace.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        lib.cbo_apply_prediction_type.restype = ctypes.c_int
        lib.cbo_apply_prediction_type.argtypes = [ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p,
                                                  ctypes.c_void_p]
        _lib = lib
    return _lib


def cat_feature_hash(s):
    if isinstance(s, str):
        s = s.encode("utf-8")
    return int(_load().cbo_cat_feature_hash(s, len(s)))


def cat_feature_hash_signed(s):
    return int(np.uint32(cat_feature_hash(s)).astype(np.int32))


def city_hash64(s):
    if isinstance(s, str):
        s = s.encode("utf-8")
    return int(_load().cbo_city_hash64(s, len(s)))


def integer_cat_feature_hash(v):
    return int(_load().cbo_integer_cat_feature_hash(int(v)))


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


PREDICTION_TYPES = {"RawFormulaVal": 0, "Exponent": 1, "RMSEWithUncertainty": 2, "Probability": 3, "Class": 4,
                    "MultiProbability": 5}


def fast_exp(values, chunk=None):
    """The reference's exponent applied to runs of `chunk` values (default: all at once)."""
    x = np.array(values, dtype=np.float64).ravel()
    chunk = len(x) if chunk is None else chunk
    for begin in range(0, len(x), max(chunk, 1)):
        part = np.ascontiguousarray(x[begin:begin + chunk])
        _load().cbo_fast_exp_inplace(_p(part), len(part))
        x[begin:begin + chunk] = part
    return x


def apply_prediction_type(raw, dim, prediction_type):
    """Raw formula values [doc * dim + k] -> the prediction type, as TEvalResultProcessor does."""
    raw = np.ascontiguousarray(np.asarray(raw, dtype=np.float64).ravel())
    docs = len(raw) // dim
    kind = PREDICTION_TYPES[prediction_type]
    out = np.zeros(docs if prediction_type == "Class" else docs * dim)
    if _load().cbo_apply_prediction_type(kind, dim, docs, _p(raw), _p(out)) != 0:
        raise ValueError("unsupported prediction type %s for dimension %d" % (prediction_type, dim))
    return out


class OracleModel:
    """The reference CPU evaluator restated; built from a model dict."""

    def __init__(self, model):
        lib = _load()
        self._keep = []

        def arr(values, dtype):
            a = np.ascontiguousarray(np.asarray(values, dtype=dtype))
            if a.size == 0:
                a = np.zeros(1, dtype=dtype)
            self._keep.append(a)
            return a

        ff = model["float_features"]
        cf = model["cat_features"]
        oh = model["one_hot_features"]
        border_off = np.zeros(len(ff) + 1, dtype=np.int32)
        for i, f in enumerate(ff):
            border_off[i + 1] = border_off[i] + len(f["borders"])
        borders = np.concatenate([np.asarray(f["borders"], dtype=np.float32) for f in ff]) if ff else np.zeros(0, np.float32)
        value_off = np.zeros(len(oh) + 1, dtype=np.int32)
        for i, o in enumerate(oh):
            value_off[i + 1] = value_off[i] + len(o["values"])
        values = np.concatenate([np.asarray(o["values"], dtype=np.int32) for o in oh]) if oh else np.zeros(0, np.int32)
        d = _Desc()
        d.approx_dim = int(model["approx_dimension"])
        d.n_trees = len(model["tree_sizes"])
        d.tree_sizes = _p(arr(model["tree_sizes"], np.int32))
        d.tree_start_offsets = _p(arr(model["tree_start_offsets"], np.int32))
        d.n_tree_splits = len(model["tree_splits"])
        d.tree_splits = _p(arr(model["tree_splits"], np.int32))
        d.n_float = len(ff)
        d.ff_index = _p(arr([f["index"] for f in ff], np.int32))
        d.ff_flat_index = _p(arr([f["flat_index"] for f in ff], np.int32))
        d.ff_has_nans = _p(arr([int(f["has_nans"]) for f in ff], np.int32))
        d.ff_nan_treatment = _p(arr([int(f["nan_treatment"]) for f in ff], np.int32))
        d.ff_border_offsets = _p(arr(border_off, np.int32))
        d.ff_borders = _p(arr(borders, np.float32))
        d.n_cat = len(cf)
        d.cf_index = _p(arr([c["index"] for c in cf], np.int32))
        d.cf_flat_index = _p(arr([c["flat_index"] for c in cf], np.int32))
        d.cf_used = _p(arr([int(c["used"]) for c in cf], np.int32))
        d.n_onehot = len(oh)
        d.oh_cat_index = _p(arr([o["cat_index"] for o in oh], np.int32))
        d.oh_value_offsets = _p(arr(value_off, np.int32))
        d.oh_values = _p(arr(values, np.int32))
        d.n_leaf_values = len(model["leaf_values"])
        d.leaf_values = _p(arr(model["leaf_values"], np.float64))
        steps = np.asarray(model["step_nodes"], dtype=np.uint16).reshape(-1, 2)
        d.n_step_nodes = steps.shape[0]
        d.step_nodes = _p(arr(steps, np.uint16))
        d.node_id_to_leaf_id = _p(arr(model["node_id_to_leaf_id"], np.uint32))
        d.scale = float(model["scale"])
        d.bias = _p(arr(model["bias"], np.float64))
        ctrs = model.get("ctr_features", [])
        tables = model.get("ctr_tables", [])
        d.n_ctr = len(ctrs)
        d.n_ctr_tables = len(tables)
        if ctrs:
            from .cbm_reader import ctr_base_key
            table_of = {ctr_base_key(t["base"]): i for i, t in enumerate(tables)}

            def offsets(lengths):
                return np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)

            def concat(parts, dtype):
                parts = [np.asarray(p, dtype=dtype).ravel() for p in parts]
                return np.concatenate(parts) if parts else np.zeros(0, dtype)

            d.ctr_border_offsets = _p(arr(offsets([len(c["borders"]) for c in ctrs]), np.int32))
            d.ctr_borders = _p(arr(concat([c["borders"] for c in ctrs], np.float32), np.float32))
            d.ctr_cat_offsets = _p(arr(offsets([len(c["base"]["cat_features"]) for c in ctrs]), np.int32))
            d.ctr_cats = _p(arr(concat([c["base"]["cat_features"] for c in ctrs], np.int32), np.int32))
            d.ctr_float_offsets = _p(arr(offsets([len(c["base"]["float_splits"]) for c in ctrs]), np.int32))
            d.ctr_float_feature = _p(arr(concat([[f for f, _ in c["base"]["float_splits"]] for c in ctrs], np.int32),
                                         np.int32))
            d.ctr_float_border = _p(arr(concat([[b for _, b in c["base"]["float_splits"]] for c in ctrs], np.float32),
                                        np.float32))
            d.ctr_onehot_offsets = _p(arr(offsets([len(c["base"]["one_hot_splits"]) for c in ctrs]), np.int32))
            d.ctr_onehot_cat = _p(arr(concat([[f for f, _ in c["base"]["one_hot_splits"]] for c in ctrs], np.int32),
                                      np.int32))
            d.ctr_onehot_value = _p(arr(concat([[v for _, v in c["base"]["one_hot_splits"]] for c in ctrs], np.int32),
                                        np.int32))
            d.ctr_type = _p(arr([c["base"]["ctr_type"] for c in ctrs], np.int32))
            d.ctr_target_border_idx = _p(arr([c["target_border_idx"] for c in ctrs], np.int32))
            d.ctr_prior_num = _p(arr([c["prior_num"] for c in ctrs], np.float32))
            d.ctr_prior_denom = _p(arr([c["prior_denom"] for c in ctrs], np.float32))
            d.ctr_shift = _p(arr([c["shift"] for c in ctrs], np.float32))
            d.ctr_scale = _p(arr([c["scale"] for c in ctrs], np.float32))
            d.ctr_table = _p(arr([table_of.get(ctr_base_key(c["base"]), -1) for c in ctrs], np.int32))
            bucket_off = np.concatenate([[0], np.cumsum([len(t["index_hash_raw"]) // 12 for t in tables])])
            blob_off = np.concatenate([[0], np.cumsum([len(t["ctr_blob"]) for t in tables])])
            d.table_bucket_offsets = _p(arr(bucket_off, np.uint64))
            d.table_buckets = _p(arr(concat([t["index_hash_raw"] for t in tables], np.uint8), np.uint8))
            d.table_blob_offsets = _p(arr(blob_off, np.uint64))
            d.table_blobs = _p(arr(concat([t["ctr_blob"] for t in tables], np.uint8), np.uint8))
            d.table_counter_denominator = _p(arr([t["counter_denominator"] for t in tables], np.int32))
            d.table_target_classes_count = _p(arr([t["target_classes_count"] for t in tables], np.int32))
        self.ctr_count = len(ctrs)
        err = ctypes.create_string_buffer(512)
        self._h = lib.cbo_model_create(ctypes.byref(d), err, 512)
        if not self._h:
            raise ValueError(err.value.decode())
        self._lib = lib
        self.dim = d.approx_dim
        self.tree_count = d.n_trees
        self.n_tree_splits = d.n_tree_splits
        self.bucket_count = int(lib.cbo_bucket_count(self._h))
        self.is_oblivious = bool(lib.cbo_is_oblivious(self._h))
        self.flat_size = int(lib.cbo_flat_vector_expected_size(self._h))
        self.min_float_size = int(lib.cbo_min_float_vector_size(self._h))
        self.min_cat_size = int(lib.cbo_min_cat_vector_size(self._h))

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.cbo_model_free(self._h)
            self._h = None

    def repacked_bins(self):
        """(feature_index, xor_mask, split_idx) per tree split."""
        out = np.zeros(max(self.n_tree_splits, 1), dtype=np.uint32)
        self._lib.cbo_repacked_bins(self._h, _p(out))
        out = out[:self.n_tree_splits]
        return (out & 0xFFFF).astype(np.uint16), ((out >> 16) & 0xFF).astype(np.uint8), (out >> 24).astype(np.uint8)

    def first_leaf_offsets(self):
        out = np.zeros(max(self.tree_count, 1), dtype=np.uint64)
        self._lib.cbo_first_leaf_offsets(self._h, _p(out))
        return out[:self.tree_count]

    def _features(self, floats, cats, layout):
        f = _Features()
        if floats is None:
            floats = np.zeros((0, 0), dtype=np.float32)
        floats = np.ascontiguousarray(floats, dtype=np.float32)
        self._cur = [floats]
        if layout == "flat":
            f.layout = 0
            n = floats.shape[0]
            f.stride = floats.shape[1]
            assert floats.shape[1] >= self.flat_size
        elif layout == "transposed":
            f.layout = 1
            n = floats.shape[1]
            f.stride = floats.shape[1]
            assert floats.shape[0] >= self.flat_size
        else:
            f.layout = 2
            f.stride = floats.shape[1] if floats.ndim == 2 else 0
            n = floats.shape[0]
            assert f.stride >= self.min_float_size
            if cats is not None:
                cats = np.ascontiguousarray(cats, dtype=np.int32)
                self._cur.append(cats)
                f.cats = _p(cats)
                f.cat_stride = cats.shape[1]
                n = max(n, cats.shape[0])
                assert f.cat_stride >= self.min_cat_size
        f.floats = _p(floats) if floats.size else None
        return f, n

    def calc(self, floats, cats=None, layout="flat", tree_start=0, tree_end=None, threads=1):
        f, n = self._features(floats, cats, layout)
        tree_end = self.tree_count if tree_end is None else tree_end
        out = np.zeros(n * self.dim, dtype=np.float64)
        if threads > 1:
            self._lib.cbo_calc_mt(self._h, ctypes.byref(f), n, tree_start, tree_end, _p(out), threads)
        else:
            self._lib.cbo_calc(self._h, ctypes.byref(f), n, tree_start, tree_end, _p(out))
        return out

    def ctrs(self, floats, cats=None, layout="flat"):
        """CTR values, one row per CTR feature of the model."""
        f, n = self._features(floats, cats, layout)
        out = np.zeros(max(self.ctr_count * n, 1), dtype=np.float32)
        self._lib.cbo_calc_ctrs(self._h, ctypes.byref(f), n, _p(out))
        return out[:self.ctr_count * n].reshape(self.ctr_count, n)

    def binarize(self, floats, cats=None, layout="flat"):
        """Bins in the reference layout: [block of 128][bucket][doc in block], flattened."""
        f, n = self._features(floats, cats, layout)
        out = np.zeros(max(n * self.bucket_count, 1), dtype=np.uint8)
        self._lib.cbo_binarize(self._h, ctypes.byref(f), n, _p(out))
        return out[:n * self.bucket_count]

    def binarize_doc_major(self, floats, cats=None, layout="flat"):
        """Bins as an [n_docs, bucket_count] matrix."""
        raw = self.binarize(floats, cats, layout)
        nb = self.bucket_count
        n = raw.size // nb if nb else 0
        out = np.zeros((n, nb), dtype=np.uint8)
        for start in range(0, n, 128):
            dc = min(128, n - start)
            out[start:start + dc] = raw[start * nb:(start + dc) * nb].reshape(nb, dc).T
        return out

    def leaf_indexes(self, floats, cats=None, layout="flat", tree_start=0, tree_end=None):
        f, n = self._features(floats, cats, layout)
        tree_end = self.tree_count if tree_end is None else tree_end
        out = np.zeros(max(n * (tree_end - tree_start), 1), dtype=np.uint32)
        self._lib.cbo_calc_leaf_indexes(self._h, ctypes.byref(f), n, tree_start, tree_end, _p(out))
        return out[:n * (tree_end - tree_start)].reshape(n, tree_end - tree_start)

    def bruteforce(self, floats, cats=None, layout="flat", tree_start=0, tree_end=None):
        f, n = self._features(floats, cats, layout)
        tree_end = self.tree_count if tree_end is None else tree_end
        out = np.zeros(n * self.dim, dtype=np.float64)
        li = np.zeros(max(n * (tree_end - tree_start), 1), dtype=np.uint32)
        self._lib.cbo_calc_bruteforce(self._h, ctypes.byref(f), n, tree_start, tree_end, _p(out), _p(li))
        return out, li[:n * (tree_end - tree_start)].reshape(n, tree_end - tree_start)
