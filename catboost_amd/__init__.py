"""MI355X-native CatBoost model evaluator: Python front end over the C ABI of libcatboostmodel.so.

`ModelCalcer` mirrors the reference's header-only C++ wrapper ModelCalcerWrapper
(catboost/libs/model_interface/wrapped_calcer.h:17-582): same operations, each one a call of the
exported C function of the same name. Everything is evaluated on the GPU by the HIP kernels of
catboost_amd/csrc; there is no CPU path, and loading fails loudly when the library is not built.
"""
import ctypes
import os
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcatboostmodel.so")

APT_RAW_FORMULA_VAL, APT_EXPONENT, APT_RMSE_WITH_UNCERTAINTY, APT_PROBABILITY, APT_CLASS, APT_MULTI_PROBABILITY = range(6)
LAYOUT_FLAT_ROWS, LAYOUT_FLAT_COLUMNS, LAYOUT_SPLIT_ROWS = range(3)

_lib = None

c_float_pp = ctypes.POINTER(ctypes.POINTER(ctypes.c_float))
c_int_pp = ctypes.POINTER(ctypes.POINTER(ctypes.c_int))
c_char_ppp = ctypes.POINTER(ctypes.POINTER(ctypes.c_char_p))


class CatBoostError(RuntimeError):
    pass


class ModelArrays(ctypes.Structure):
    """CbHipModelArrays of include/cb_hip_evaluator.h."""
    _fields_ = [
        ("ApproxDimension", ctypes.c_int32),
        ("TreeCount", ctypes.c_int32),
        ("TreeSizes", ctypes.c_void_p),
        ("TreeStartOffsets", ctypes.c_void_p),
        ("TreeSplitsCount", ctypes.c_int32),
        ("TreeSplits", ctypes.c_void_p),
        ("FloatFeatureCount", ctypes.c_int32),
        ("FloatFeatureIndex", ctypes.c_void_p),
        ("FloatFeatureFlatIndex", ctypes.c_void_p),
        ("FloatFeatureHasNans", ctypes.c_void_p),
        ("FloatFeatureNanTreatment", ctypes.c_void_p),
        ("FloatFeatureBorderOffsets", ctypes.c_void_p),
        ("FloatFeatureBorders", ctypes.c_void_p),
        ("CatFeatureCount", ctypes.c_int32),
        ("CatFeatureIndex", ctypes.c_void_p),
        ("CatFeatureFlatIndex", ctypes.c_void_p),
        ("CatFeatureUsed", ctypes.c_void_p),
        ("OneHotFeatureCount", ctypes.c_int32),
        ("OneHotCatFeatureIndex", ctypes.c_void_p),
        ("OneHotValueOffsets", ctypes.c_void_p),
        ("OneHotValues", ctypes.c_void_p),
        ("LeafValuesCount", ctypes.c_uint64),
        ("LeafValues", ctypes.c_void_p),
        ("StepNodeCount", ctypes.c_int32),
        ("StepNodes", ctypes.c_void_p),
        ("NodeIdToLeafId", ctypes.c_void_p),
        ("Scale", ctypes.c_double),
        ("Bias", ctypes.c_void_p),
    ]


class DeviceFeatures(ctypes.Structure):
    """CbHipFeatures of include/cb_hip_evaluator.h."""
    _fields_ = [
        ("Layout", ctypes.c_int32),
        ("Floats", ctypes.c_void_p),
        ("Stride", ctypes.c_size_t),
        ("Cats", ctypes.c_void_p),
        ("CatStride", ctypes.c_size_t),
    ]


SPLIT_DTYPE = np.dtype([("Type", np.int32), ("FeatureIndex", np.int32), ("Border", np.float32), ("Value", np.int32)])


def library_path():
    return LIB_PATH


def load_library():
    """Loads libcatboostmodel.so; raises when the HIP extension has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CatBoostError(
            "%s is missing: build it with `python -m catboost_amd.build` (needs hipcc); "
            "this package has no CPU fallback" % LIB_PATH)
    if "torch" not in sys.modules and not os.environ.get("CATBOOST_AMD_NO_TORCH_PRELOAD"):
        # A process must hold one HIP runtime only. PyTorch wheels carry their own libamdhip64
        # (same soname as the system one); loading it first makes this library bind to that copy
        # instead of bringing in a second runtime, which could not see the GPU any more.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
    lib = ctypes.CDLL(LIB_PATH)
    vp, sz, dp = ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_double)
    sig = {
        "ModelCalcerCreate": (vp, []),
        "ModelCalcerDelete": (None, [vp]),
        "GetErrorString": (ctypes.c_char_p, []),
        "LoadFullModelFromFile": (ctypes.c_bool, [vp, ctypes.c_char_p]),
        "LoadFullModelFromBuffer": (ctypes.c_bool, [vp, vp, sz]),
        "LoadFullModelZeroCopy": (ctypes.c_bool, [vp, vp, sz]),
        "EnableGPUEvaluation": (ctypes.c_bool, [vp, ctypes.c_int]),
        "GetSupportedEvaluatorTypes": (ctypes.c_bool, [vp, ctypes.POINTER(ctypes.POINTER(ctypes.c_int)), ctypes.POINTER(sz)]),
        "SetPredictionType": (ctypes.c_bool, [vp, ctypes.c_int]),
        "SetPredictionTypeString": (ctypes.c_bool, [vp, ctypes.c_char_p]),
        "CalcModelPredictionFlat": (ctypes.c_bool, [vp, sz, c_float_pp, sz, dp, sz]),
        "CalcModelPredictionFlatStaged": (ctypes.c_bool, [vp, sz, sz, sz, c_float_pp, sz, dp, sz]),
        "CalcModelPredictionFlatTransposed": (ctypes.c_bool, [vp, sz, c_float_pp, sz, dp, sz]),
        "CalcModelPredictionFlatTransposedStaged": (ctypes.c_bool, [vp, sz, sz, sz, c_float_pp, sz, dp, sz]),
        "CalcModelPrediction": (ctypes.c_bool, [vp, sz, c_float_pp, sz, c_char_ppp, sz, dp, sz]),
        "CalcModelPredictionStaged": (ctypes.c_bool, [vp, sz, sz, sz, c_float_pp, sz, c_char_ppp, sz, dp, sz]),
        "CalcModelPredictionSingle": (ctypes.c_bool, [vp, ctypes.POINTER(ctypes.c_float), sz, ctypes.POINTER(ctypes.c_char_p), sz, dp, sz]),
        "CalcModelPredictionWithHashedCatFeatures": (ctypes.c_bool, [vp, sz, c_float_pp, sz, c_int_pp, sz, dp, sz]),
        "PredictSpecificClassFlat": (ctypes.c_bool, [vp, sz, c_float_pp, sz, ctypes.c_int, dp, sz]),
        "GetStringCatFeatureHash": (ctypes.c_int, [ctypes.c_char_p, sz]),
        "GetIntegerCatFeatureHash": (ctypes.c_int, [ctypes.c_longlong]),
        "GetFloatFeaturesCount": (sz, [vp]),
        "GetCatFeaturesCount": (sz, [vp]),
        "GetTextFeaturesCount": (sz, [vp]),
        "GetEmbeddingFeaturesCount": (sz, [vp]),
        "GetTreeCount": (sz, [vp]),
        "GetDimensionsCount": (sz, [vp]),
        "GetPredictionDimensionsCount": (sz, [vp]),
        "GetFloatFeatureIndices": (ctypes.c_bool, [vp, ctypes.POINTER(ctypes.POINTER(sz)), ctypes.POINTER(sz)]),
        "GetCatFeatureIndices": (ctypes.c_bool, [vp, ctypes.POINTER(ctypes.POINTER(sz)), ctypes.POINTER(sz)]),
        "CheckModelMetadataHasKey": (ctypes.c_bool, [vp, ctypes.c_char_p, sz]),
        "GetModelInfoValueSize": (sz, [vp, ctypes.c_char_p, sz]),
        "GetModelInfoValue": (vp, [vp, ctypes.c_char_p, sz]),
        "GetModelUsedFeaturesNames": (ctypes.c_bool, [vp, ctypes.POINTER(ctypes.POINTER(ctypes.c_char_p)), ctypes.POINTER(sz)]),
        # evaluator-level ABI
        "CbHipEvaluatorCreate": (vp, [ctypes.POINTER(ModelArrays), ctypes.c_int]),
        "CbHipEvaluatorDelete": (None, [vp]),
        "CbHipTreeCount": (sz, [vp]),
        "CbHipApproxDimension": (ctypes.c_int32, [vp]),
        "CbHipBucketCount": (ctypes.c_uint32, [vp]),
        "CbHipQuantizedBytes": (sz, [vp, sz]),
        "CbHipQuantize": (ctypes.c_bool, [vp, ctypes.POINTER(DeviceFeatures), sz, vp, vp]),
        "CbHipEvalQuantized": (ctypes.c_bool, [vp, vp, sz, sz, sz, vp, vp]),
        "CbHipEvalData": (ctypes.c_bool, [vp, ctypes.POINTER(DeviceFeatures), sz, sz, sz, vp, vp]),
        "CbHipEvalDataNoAlloc": (ctypes.c_bool, [vp, ctypes.POINTER(DeviceFeatures), sz, sz, sz, vp, vp]),
        "CbHipLeafIndexesQuantized": (ctypes.c_bool, [vp, vp, sz, sz, sz, vp, vp]),
        "CbHipExportQuantized": (ctypes.c_bool, [vp, vp, sz, vp, vp]),
        "CbHipApplyPredictionTypeDevice": (ctypes.c_bool, [vp, ctypes.c_int, sz, vp, vp, vp]),
        "CbHipSynchronize": (ctypes.c_bool, [vp, vp]),
        "CbHipLastKernelTimes": (ctypes.c_bool, [vp, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]),
        "CbHipDescribeKernels": (ctypes.c_bool, [vp, ctypes.c_int, sz, ctypes.c_char_p, sz]),
        "CbHipGetEvaluator": (vp, [vp]),
        "CbHipEvaluatorSetSmallBatchSlicing": (ctypes.c_bool, [vp, ctypes.c_bool]),
        "CbHipSetSmallBatchSlicing": (ctypes.c_bool, [vp, ctypes.c_bool]),
        "CbHipSetFeatureLayout": (ctypes.c_bool, [vp, vp, sz, vp, sz, vp, sz]),
        "CbHipLoadModelFromArrays": (ctypes.c_bool, [vp, ctypes.POINTER(ModelArrays)]),
        "CbHipBuildObliviousModel": (ctypes.c_bool, [vp, ctypes.POINTER(ModelArrays), ctypes.c_int32, vp, vp, vp]),
        "CbHipBuildNonSymmetricModel": (ctypes.c_bool, [vp, ctypes.POINTER(ModelArrays), ctypes.c_int32, vp, vp, vp, vp, vp, vp, vp]),
        "CbHipLoadFullModelFromJsonFile": (ctypes.c_bool, [vp, ctypes.c_char_p]),
        "CbHipLoadFullModelFromJsonBuffer": (ctypes.c_bool, [vp, ctypes.c_char_p, sz]),
        "CbHipSaveModelToFile": (ctypes.c_bool, [vp, ctypes.c_char_p]),
        "CbHipSaveModelToBuffer": (ctypes.c_bool, [vp, ctypes.POINTER(vp), ctypes.POINTER(sz)]),
        "CbHipConvertObliviousToAsymmetric": (ctypes.c_bool, [vp]),
        "CbHipSetScaleAndBias": (ctypes.c_bool, [vp, ctypes.c_double, dp, sz]),
        "CbHipSetModelInfo": (ctypes.c_bool, [vp, ctypes.c_char_p, ctypes.c_char_p]),
        "CbHipCalcFlatContiguous": (ctypes.c_bool, [vp, vp, sz, sz, sz, sz, dp, sz]),
        "CbHipCalcLeafIndexesFlat": (ctypes.c_bool, [vp, sz, c_float_pp, sz, sz, sz, vp, sz]),
        "CbHipQuantizeFlat": (ctypes.c_bool, [vp, sz, c_float_pp, sz, vp, sz]),
        "CbHipQuantizeWithHashedCatFeatures": (ctypes.c_bool, [vp, sz, c_float_pp, sz, c_int_pp, sz, vp, sz]),
        "CbHipModelBucketCount": (ctypes.c_uint32, [vp]),
        "CbHipFastExpInplace": (None, [vp, sz]),
        "CbHipApplyPredictionType": (ctypes.c_bool, [ctypes.c_int, sz, sz, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    lib._libc_free = ctypes.CDLL(None).free
    lib._libc_free.argtypes = [ctypes.c_void_p]
    _lib = lib
    return lib


def last_error():
    msg = load_library().GetErrorString()
    return msg.decode("utf-8", errors="replace") if msg else ""


def _check(ok):
    if not ok:
        raise CatBoostError(last_error())


def string_cat_feature_hash(s):
    """GetStringCatFeatureHash."""
    if isinstance(s, str):
        s = s.encode("utf-8")
    return int(load_library().GetStringCatFeatureHash(s, len(s)))


def integer_cat_feature_hash(v):
    """GetIntegerCatFeatureHash."""
    return int(load_library().GetIntegerCatFeatureHash(int(v)))


def _row_pointers(matrix, ctype):
    """Array of per-row pointers into a C-contiguous 2-D numpy array."""
    n = matrix.shape[0]
    addresses = matrix.ctypes.data + np.arange(max(n, 1), dtype=np.uint64) * np.uint64(matrix.strides[0])
    # the ctypes array shares (and keeps alive) the numpy buffer of addresses
    return (ctypes.POINTER(ctype) * max(n, 1)).from_buffer(addresses)


def fast_exp(values, chunk=None):
    """The reference's exponent (CbHipFastExpInplace) over runs of `chunk` values (default: all at once)."""
    lib = load_library()
    x = np.array(values, dtype=np.float64).ravel()
    chunk = len(x) if chunk is None else chunk
    for begin in range(0, len(x), max(chunk, 1)):
        part = np.ascontiguousarray(x[begin:begin + chunk])
        lib.CbHipFastExpInplace(part.ctypes.data, len(part))
        x[begin:begin + chunk] = part
    return x


def apply_prediction_type(raw, dim, prediction_type):
    """Raw formula values [doc * dim + k] -> prediction type (an APT_* constant), on the host."""
    lib = load_library()
    raw = np.ascontiguousarray(np.asarray(raw, dtype=np.float64).ravel())
    docs = len(raw) // dim
    out = np.zeros(docs if prediction_type == APT_CLASS else docs * dim)
    _check(lib.CbHipApplyPredictionType(prediction_type, dim, docs, raw.ctypes.data, out.ctypes.data))
    return out


def model_arrays(float_features=(), cat_features=(), one_hot_features=(), approx_dimension=1, tree_sizes=(),
                 tree_start_offsets=(), tree_splits=(), leaf_values=(), step_nodes=(), node_id_to_leaf_id=(),
                 scale=1.0, bias=None):
    """Packs a model description into a ModelArrays struct. Returns (struct, keep_alive)."""
    keep = []

    def arr(values, dtype):
        a = np.ascontiguousarray(np.asarray(values, dtype=dtype))
        if a.size == 0:
            a = np.zeros(1, dtype=dtype)
        keep.append(a)
        return a.ctypes.data

    m = ModelArrays()
    m.ApproxDimension = int(approx_dimension)
    m.TreeCount = len(tree_sizes)
    m.TreeSizes = arr(tree_sizes, np.int32)
    m.TreeStartOffsets = arr(tree_start_offsets, np.int32)
    m.TreeSplitsCount = len(tree_splits)
    m.TreeSplits = arr(tree_splits, np.int32)
    ff = list(float_features)
    m.FloatFeatureCount = len(ff)
    m.FloatFeatureIndex = arr([f["index"] for f in ff], np.int32)
    m.FloatFeatureFlatIndex = arr([f["flat_index"] for f in ff], np.int32)
    m.FloatFeatureHasNans = arr([int(f.get("has_nans", False)) for f in ff], np.int32)
    m.FloatFeatureNanTreatment = arr([int(f.get("nan_treatment", 0)) for f in ff], np.int32)
    offs = np.zeros(len(ff) + 1, np.int32)
    for i, f in enumerate(ff):
        offs[i + 1] = offs[i] + len(f.get("borders", ()))
    m.FloatFeatureBorderOffsets = arr(offs, np.int32)
    borders = [np.asarray(f.get("borders", ()), np.float32) for f in ff]
    m.FloatFeatureBorders = arr(np.concatenate(borders) if borders else [], np.float32)
    cf = list(cat_features)
    m.CatFeatureCount = len(cf)
    m.CatFeatureIndex = arr([c["index"] for c in cf], np.int32)
    m.CatFeatureFlatIndex = arr([c["flat_index"] for c in cf], np.int32)
    m.CatFeatureUsed = arr([int(c.get("used", True)) for c in cf], np.int32)
    oh = list(one_hot_features)
    m.OneHotFeatureCount = len(oh)
    m.OneHotCatFeatureIndex = arr([o["cat_index"] for o in oh], np.int32)
    voffs = np.zeros(len(oh) + 1, np.int32)
    for i, o in enumerate(oh):
        voffs[i + 1] = voffs[i] + len(o["values"])
    m.OneHotValueOffsets = arr(voffs, np.int32)
    vals = [np.asarray(o["values"], np.int32) for o in oh]
    m.OneHotValues = arr(np.concatenate(vals) if vals else [], np.int32)
    m.LeafValuesCount = len(leaf_values)
    m.LeafValues = arr(leaf_values, np.float64)
    steps = np.asarray(step_nodes, dtype=np.uint16).reshape(-1, 2)
    m.StepNodeCount = steps.shape[0]
    m.StepNodes = arr(steps, np.uint16)
    m.NodeIdToLeafId = arr(node_id_to_leaf_id, np.uint32)
    m.Scale = float(scale)
    m.Bias = arr(np.zeros(approx_dimension) if bias is None else bias, np.float64)
    return m, keep


def model_arrays_from_dict(model):
    """ModelArrays from a model dict with the keys used by the .cbm tables."""
    return model_arrays(
        float_features=model["float_features"], cat_features=model["cat_features"],
        one_hot_features=model["one_hot_features"], approx_dimension=model["approx_dimension"],
        tree_sizes=model["tree_sizes"], tree_start_offsets=model["tree_start_offsets"],
        tree_splits=model["tree_splits"], leaf_values=model["leaf_values"], step_nodes=model["step_nodes"],
        node_id_to_leaf_id=model["node_id_to_leaf_id"], scale=model["scale"], bias=model["bias"])


def make_splits(splits):
    """[("float", feature, border) | ("onehot", cat feature, value)] -> CbHipModelSplit array."""
    out = np.zeros(len(splits), dtype=SPLIT_DTYPE)
    for i, s in enumerate(splits):
        if s[0] == "float":
            out[i] = (0, s[1], s[2], 0)
        else:
            out[i] = (2, s[1], 0.0, s[2])
    return out


class DeviceEvaluator:
    """Evaluator-level handle (CbHipEvaluatorHandle): device pointers in, device pointers out."""

    def __init__(self, handle, owner=None, owned=False):
        self._lib = load_library()
        self._h = handle
        self._owner = owner
        self._owned = owned

    @classmethod
    def from_arrays(cls, arrays, device_id=0):
        lib = load_library()
        h = lib.CbHipEvaluatorCreate(ctypes.byref(arrays), device_id)
        if not h:
            raise CatBoostError(last_error())
        return cls(h, owned=True)

    def __del__(self):
        if getattr(self, "_owned", False) and self._h:
            self._lib.CbHipEvaluatorDelete(self._h)
            self._h = None

    @property
    def tree_count(self):
        return int(self._lib.CbHipTreeCount(self._h))

    @property
    def dim(self):
        return int(self._lib.CbHipApproxDimension(self._h))

    @property
    def bucket_count(self):
        return int(self._lib.CbHipBucketCount(self._h))

    def quantized_bytes(self, doc_count):
        return int(self._lib.CbHipQuantizedBytes(self._h, doc_count))

    @staticmethod
    def features(layout, floats_ptr, stride, cats_ptr=0, cat_stride=0):
        f = DeviceFeatures()
        f.Layout = layout
        f.Floats = floats_ptr
        f.Stride = stride
        f.Cats = cats_ptr
        f.CatStride = cat_stride
        return f

    def quantize(self, features, doc_count, bins_ptr, stream=None):
        _check(self._lib.CbHipQuantize(self._h, ctypes.byref(features), doc_count, bins_ptr, stream))

    def eval_quantized(self, bins_ptr, doc_count, results_ptr, tree_start=0, tree_end=None, stream=None):
        tree_end = self.tree_count if tree_end is None else tree_end
        _check(self._lib.CbHipEvalQuantized(self._h, bins_ptr, doc_count, tree_start, tree_end, results_ptr, stream))

    def eval_data(self, features, doc_count, results_ptr, tree_start=0, tree_end=None, stream=None):
        tree_end = self.tree_count if tree_end is None else tree_end
        _check(self._lib.CbHipEvalData(self._h, ctypes.byref(features), doc_count, tree_start, tree_end, results_ptr, stream))

    def eval_data_no_alloc(self, features, doc_count, results_ptr, tree_start=0, tree_end=None, stream=None):
        """eval_data with the bins in the library's fixed device array: allocates nothing, asynchronous."""
        tree_end = self.tree_count if tree_end is None else tree_end
        _check(self._lib.CbHipEvalDataNoAlloc(self._h, ctypes.byref(features), doc_count, tree_start, tree_end, results_ptr, stream))

    def leaf_indexes_quantized(self, bins_ptr, doc_count, indexes_ptr, tree_start=0, tree_end=None, stream=None):
        tree_end = self.tree_count if tree_end is None else tree_end
        _check(self._lib.CbHipLeafIndexesQuantized(self._h, bins_ptr, doc_count, tree_start, tree_end, indexes_ptr, stream))

    def export_quantized(self, bins_ptr, doc_count, out_ptr, stream=None):
        _check(self._lib.CbHipExportQuantized(self._h, bins_ptr, doc_count, out_ptr, stream))

    def apply_prediction_type(self, prediction_type, doc_count, raw_ptr, result_ptr, stream=None):
        """Raw formula values on the device -> a prediction type (an APT_* constant)."""
        kind = int(prediction_type)
        _check(self._lib.CbHipApplyPredictionTypeDevice(self._h, kind, doc_count, raw_ptr, result_ptr, stream))

    def synchronize(self, stream=None):
        _check(self._lib.CbHipSynchronize(self._h, stream))

    def describe_kernels(self, layout=LAYOUT_FLAT_ROWS, doc_count=1 << 24):
        """The kernels of a whole-model eval_data call on doc_count documents as a dict: {"fused": name} or
        {"binarize": name, "evaluate": name}."""
        buf = ctypes.create_string_buffer(512)
        _check(self._lib.CbHipDescribeKernels(self._h, int(layout), doc_count, buf, len(buf)))
        return dict(item.split("=", 1) for item in buf.value.decode().split(";"))

    def last_kernel_times(self):
        a, b = ctypes.c_float(), ctypes.c_float()
        _check(self._lib.CbHipLastKernelTimes(self._h, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def set_small_batch_slicing(self, enabled):
        """False: small batches are evaluated in one pass in tree order like large ones (CbHipEvaluatorSetSmallBatchSlicing)."""
        _check(self._lib.CbHipEvaluatorSetSmallBatchSlicing(self._h, bool(enabled)))


class ModelCalcer:
    """Model handle of the model_calcer C API (ModelCalcerWrapper, wrapped_calcer.h:17-110)."""

    def __init__(self, filename=None, buffer=None, model_format="cbm"):
        self._lib = load_library()
        self._h = self._lib.ModelCalcerCreate()
        if not self._h:
            raise CatBoostError(last_error())
        if model_format not in ("cbm", "json"):
            raise CatBoostError("unknown model format %r" % (model_format,))
        if filename is not None:
            self.init_from_json_file(filename) if model_format == "json" else self.init_from_file(filename)
        elif buffer is not None:
            self.init_from_json(buffer) if model_format == "json" else self.init_from_memory(buffer)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ModelCalcerDelete(self._h)
            self._h = None

    @property
    def handle(self):
        return self._h

    # ---- loading / building
    def init_from_file(self, filename):
        _check(self._lib.LoadFullModelFromFile(self._h, os.fsencode(filename)))

    def init_from_memory(self, data):
        data = bytes(data)
        _check(self._lib.LoadFullModelFromBuffer(self._h, data, len(data)))

    def init_from_json_file(self, filename):
        _check(self._lib.CbHipLoadFullModelFromJsonFile(self._h, os.fsencode(filename)))

    def init_from_json(self, text):
        data = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        _check(self._lib.CbHipLoadFullModelFromJsonBuffer(self._h, data, len(data)))

    def load_from_arrays(self, arrays):
        _check(self._lib.CbHipLoadModelFromArrays(self._h, ctypes.byref(arrays)))

    def load_from_dict(self, model):
        arrays, keep = model_arrays_from_dict(model)
        self.load_from_arrays(arrays)
        del keep

    def build_oblivious(self, float_features, cat_features, approx_dimension, trees, scale=1.0, bias=None):
        """trees: list of (splits, leaf_values[leaf * dim + k]) (TObliviousTreeBuilder)."""
        arrays, keep = model_arrays(float_features=float_features, cat_features=cat_features,
                                    approx_dimension=approx_dimension, scale=scale, bias=bias)
        depths = np.asarray([len(t[0]) for t in trees], dtype=np.int32)
        splits = make_splits([s for t in trees for s in t[0]])
        leaves = np.ascontiguousarray(np.concatenate([np.asarray(t[1], np.float64) for t in trees])
                                      if trees else np.zeros(0))
        _check(self._lib.CbHipBuildObliviousModel(
            self._h, ctypes.byref(arrays), len(trees), depths.ctypes.data if len(trees) else None,
            splits.ctypes.data if len(splits) else None, leaves.ctypes.data if leaves.size else None))
        del keep

    def build_oblivious_packed(self, float_features, cat_features, approx_dimension, depths, splits, leaves,
                               scale=1.0, bias=None):
        """Same with pre-packed numpy arrays (depths int32, splits SPLIT_DTYPE, leaves float64)."""
        arrays, keep = model_arrays(float_features=float_features, cat_features=cat_features,
                                    approx_dimension=approx_dimension, scale=scale, bias=bias)
        depths = np.ascontiguousarray(depths, np.int32)
        splits = np.ascontiguousarray(splits, SPLIT_DTYPE)
        leaves = np.ascontiguousarray(leaves, np.float64)
        _check(self._lib.CbHipBuildObliviousModel(self._h, ctypes.byref(arrays), len(depths), depths.ctypes.data,
                                                  splits.ctypes.data, leaves.ctypes.data))
        del keep

    def build_non_symmetric_packed(self, float_features, cat_features, approx_dimension, tree_node_offsets,
                                   node_is_split, node_splits, node_left, node_right, node_value_offset,
                                   node_values, scale=1.0, bias=None):
        arrays, keep = model_arrays(float_features=float_features, cat_features=cat_features,
                                    approx_dimension=approx_dimension, scale=scale, bias=bias)
        a = [np.ascontiguousarray(tree_node_offsets, np.int32), np.ascontiguousarray(node_is_split, np.int32),
             np.ascontiguousarray(node_splits, SPLIT_DTYPE), np.ascontiguousarray(node_left, np.int32),
             np.ascontiguousarray(node_right, np.int32), np.ascontiguousarray(node_value_offset, np.int64),
             np.ascontiguousarray(node_values, np.float64)]
        _check(self._lib.CbHipBuildNonSymmetricModel(self._h, ctypes.byref(arrays), len(a[0]) - 1,
                                                     *[x.ctypes.data for x in a]))
        del keep

    def build_non_symmetric(self, float_features, cat_features, approx_dimension, tree_heads, scale=1.0, bias=None):
        """tree_heads: nested ("split", split, left, right) / ("leaf", value or vector) nodes."""
        offsets, is_split, splits, left, right, voff, values = [0], [], [], [], [], [], []
        for head in tree_heads:
            base = len(is_split)

            def add(node):  # pre-order numbering, children follow their parent
                i = len(is_split) - base
                if node[0] == "split":
                    is_split.append(1)
                    splits.append(node[1])
                    left.append(0)
                    right.append(0)
                    voff.append(0)
                    pos = len(is_split) - 1
                    left[pos] = add(node[2])
                    right[pos] = add(node[3])
                else:
                    is_split.append(0)
                    splits.append(("float", 0, 0.0))
                    left.append(0)
                    right.append(0)
                    voff.append(len(values))
                    v = node[1]
                    values.extend([float(v)] if np.isscalar(v) else [float(x) for x in v])
                return i

            add(head)
            offsets.append(len(is_split))
        self.build_non_symmetric_packed(float_features, cat_features, approx_dimension, offsets, is_split,
                                        make_splits(splits), left, right, voff, values, scale=scale, bias=bias)

    def save_to_file(self, filename):
        _check(self._lib.CbHipSaveModelToFile(self._h, os.fsencode(filename)))

    def save_to_buffer(self):
        buf, size = ctypes.c_void_p(), ctypes.c_size_t()
        _check(self._lib.CbHipSaveModelToBuffer(self._h, ctypes.byref(buf), ctypes.byref(size)))
        data = ctypes.string_at(buf.value, size.value)
        self._lib._libc_free(buf)
        return data

    def convert_oblivious_to_asymmetric(self):
        _check(self._lib.CbHipConvertObliviousToAsymmetric(self._h))

    def set_scale_and_bias(self, scale, bias):
        b = np.ascontiguousarray(bias, np.float64)
        _check(self._lib.CbHipSetScaleAndBias(self._h, float(scale), b.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), b.size))

    def set_model_info(self, key, value):
        _check(self._lib.CbHipSetModelInfo(self._h, key.encode(), value.encode()))

    def set_feature_layout(self, float_feature_indexes=None, cat_feature_indexes=None, flat_indexes=None):
        """TFeatureLayout (evaluation_interface.h:17-69): a feature at model position p is read at
        list[p] of the caller's data; None leaves a kind of position as the model has it."""
        lists = [None if v is None else np.ascontiguousarray(v, np.uint32)
                 for v in (float_feature_indexes, cat_feature_indexes, flat_indexes)]
        args = []
        placeholder = ctypes.c_uint32()  # a defined but empty list still needs a non-null pointer
        for a in lists:
            args += [None, 0] if a is None else [a.ctypes.data if a.size else ctypes.addressof(placeholder), a.size]
        _check(self._lib.CbHipSetFeatureLayout(self._h, *args))

    # ---- evaluator selection
    def enable_gpu_evaluation(self, device_id=0):
        _check(self._lib.EnableGPUEvaluation(self._h, device_id))

    def get_supported_evaluator_types(self):
        p, n = ctypes.POINTER(ctypes.c_int)(), ctypes.c_size_t()
        _check(self._lib.GetSupportedEvaluatorTypes(self._h, ctypes.byref(p), ctypes.byref(n)))
        out = [p[i] for i in range(n.value)]
        self._lib._libc_free(ctypes.cast(p, ctypes.c_void_p))
        return out

    def set_prediction_type(self, prediction_type):
        if isinstance(prediction_type, str):
            _check(self._lib.SetPredictionTypeString(self._h, prediction_type.encode()))
        else:
            _check(self._lib.SetPredictionType(self._h, int(prediction_type)))

    def set_small_batch_slicing(self, enabled):
        """False: small batches are evaluated in one pass in tree order, the CPU evaluator's order of additions,
        instead of as slices of the trees (CbHipSetSmallBatchSlicing)."""
        _check(self._lib.CbHipSetSmallBatchSlicing(self._h, bool(enabled)))

    def evaluator(self):
        h = self._lib.CbHipGetEvaluator(self._h)
        if not h:
            raise CatBoostError(last_error())
        return DeviceEvaluator(h, owner=self)

    # ---- description
    @property
    def tree_count(self):
        return int(self._lib.GetTreeCount(self._h))

    @property
    def dimensions_count(self):
        return int(self._lib.GetDimensionsCount(self._h))

    @property
    def prediction_dimensions_count(self):
        return int(self._lib.GetPredictionDimensionsCount(self._h))

    @property
    def float_features_count(self):
        return int(self._lib.GetFloatFeaturesCount(self._h))

    @property
    def cat_features_count(self):
        return int(self._lib.GetCatFeaturesCount(self._h))

    @property
    def bucket_count(self):
        return int(self._lib.CbHipModelBucketCount(self._h))

    def _indices(self, fn):
        p, n = ctypes.POINTER(ctypes.c_size_t)(), ctypes.c_size_t()
        _check(fn(self._h, ctypes.byref(p), ctypes.byref(n)))
        out = [int(p[i]) for i in range(n.value)]
        if n.value:
            self._lib._libc_free(ctypes.cast(p, ctypes.c_void_p))
        return out

    def get_float_feature_indices(self):
        return self._indices(self._lib.GetFloatFeatureIndices)

    def get_cat_feature_indices(self):
        return self._indices(self._lib.GetCatFeatureIndices)

    def check_metadata_has_key(self, key):
        k = key.encode()
        return bool(self._lib.CheckModelMetadataHasKey(self._h, k, len(k)))

    def get_metadata_key_value(self, key):
        k = key.encode()
        n = self._lib.GetModelInfoValueSize(self._h, k, len(k))
        p = self._lib.GetModelInfoValue(self._h, k, len(k))
        return ctypes.string_at(p, n).decode() if p else ""

    def get_used_features_names(self):
        p, n = ctypes.POINTER(ctypes.c_char_p)(), ctypes.c_size_t()
        _check(self._lib.GetModelUsedFeaturesNames(self._h, ctypes.byref(p), ctypes.byref(n)))
        out = []
        raw = ctypes.cast(p, ctypes.POINTER(ctypes.c_void_p))
        for i in range(n.value):
            out.append(ctypes.string_at(raw[i]).decode())
            self._lib._libc_free(raw[i])
        self._lib._libc_free(ctypes.cast(p, ctypes.c_void_p))
        return out

    # ---- predictions
    def _result(self, doc_count):
        return np.zeros(doc_count * self.prediction_dimensions_count, dtype=np.float64)

    @staticmethod
    def _dp(a):
        return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))

    def calc_flat(self, features, tree_start=None, tree_end=None, result_size=None):
        """CalcModelPredictionFlat[Staged]: features[doc][flat feature index]."""
        x = np.ascontiguousarray(features, dtype=np.float32)
        if x.ndim == 1:
            x = x.reshape(1, -1)
        n = x.shape[0]
        out = self._result(n) if result_size is None else np.zeros(result_size)
        rows = _row_pointers(x, ctypes.c_float)
        if tree_start is None and tree_end is None:
            _check(self._lib.CalcModelPredictionFlat(self._h, n, rows, x.shape[1], self._dp(out), out.size))
        else:
            ts = 0 if tree_start is None else tree_start
            te = self.tree_count if tree_end is None else tree_end
            _check(self._lib.CalcModelPredictionFlatStaged(self._h, n, ts, te, rows, x.shape[1], self._dp(out), out.size))
        return out

    def calc_flat_contiguous(self, features, tree_start=0, tree_end=None):
        x = np.ascontiguousarray(features, dtype=np.float32)
        n = x.shape[0]
        out = self._result(n)
        te = self.tree_count if tree_end is None else tree_end
        _check(self._lib.CbHipCalcFlatContiguous(self._h, x.ctypes.data, n, x.shape[1], tree_start, te, self._dp(out), out.size))
        return out

    def calc_flat_transposed(self, transposed_features, tree_start=None, tree_end=None):
        """CalcModelPredictionFlatTransposed[Staged]: features[flat feature index][doc]."""
        x = np.ascontiguousarray(transposed_features, dtype=np.float32)
        n = x.shape[1]
        out = self._result(n)
        cols = _row_pointers(x, ctypes.c_float)
        if tree_start is None and tree_end is None:
            _check(self._lib.CalcModelPredictionFlatTransposed(self._h, n, cols, x.shape[0], self._dp(out), out.size))
        else:
            ts = 0 if tree_start is None else tree_start
            te = self.tree_count if tree_end is None else tree_end
            _check(self._lib.CalcModelPredictionFlatTransposedStaged(self._h, n, ts, te, cols, x.shape[0], self._dp(out), out.size))
        return out

    def calc(self, float_features, cat_features, tree_start=None, tree_end=None):
        """CalcModelPrediction[Staged]: float rows + string categorical rows."""
        x = np.ascontiguousarray(float_features, dtype=np.float32)
        if x.ndim == 1:
            x = x.reshape(len(cat_features), -1)
        n = max(x.shape[0], len(cat_features))
        n_cat = len(cat_features[0]) if len(cat_features) else 0
        keep = []
        cat_rows = (ctypes.POINTER(ctypes.c_char_p) * max(n, 1))()
        for i in range(len(cat_features)):
            row = (ctypes.c_char_p * max(n_cat, 1))()
            for j, s in enumerate(cat_features[i]):
                row[j] = s.encode("utf-8") if isinstance(s, str) else s
            keep.append(row)
            cat_rows[i] = ctypes.cast(row, ctypes.POINTER(ctypes.c_char_p))
        out = self._result(n)
        rows = _row_pointers(x, ctypes.c_float)
        if tree_start is None and tree_end is None:
            _check(self._lib.CalcModelPrediction(self._h, n, rows, x.shape[1], cat_rows, n_cat, self._dp(out), out.size))
        else:
            ts = 0 if tree_start is None else tree_start
            te = self.tree_count if tree_end is None else tree_end
            _check(self._lib.CalcModelPredictionStaged(self._h, n, ts, te, rows, x.shape[1], cat_rows, n_cat, self._dp(out), out.size))
        return out

    def calc_single(self, float_features, cat_features):
        x = np.ascontiguousarray(float_features, dtype=np.float32)
        row = (ctypes.c_char_p * max(len(cat_features), 1))()
        for j, s in enumerate(cat_features):
            row[j] = s.encode("utf-8") if isinstance(s, str) else s
        out = self._result(1)
        _check(self._lib.CalcModelPredictionSingle(self._h, x.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), x.size,
                                                   row, len(cat_features), self._dp(out), out.size))
        return out

    def calc_hashed(self, float_features, hashed_cat_features):
        """CalcModelPredictionWithHashedCatFeatures."""
        x = np.ascontiguousarray(float_features, dtype=np.float32)
        c = np.ascontiguousarray(hashed_cat_features, dtype=np.int32)
        n = max(x.shape[0] if x.ndim == 2 else 0, c.shape[0] if c.ndim == 2 else 0)
        out = self._result(n)
        frows = _row_pointers(x, ctypes.c_float) if x.ndim == 2 and x.shape[1] else None
        crows = _row_pointers(c, ctypes.c_int) if c.ndim == 2 and c.shape[1] else None
        _check(self._lib.CalcModelPredictionWithHashedCatFeatures(
            self._h, n, frows, x.shape[1] if x.ndim == 2 else 0, crows, c.shape[1] if c.ndim == 2 else 0,
            self._dp(out), out.size))
        return out

    def predict_specific_class_flat(self, features, class_id):
        x = np.ascontiguousarray(features, dtype=np.float32)
        n = x.shape[0]
        out = np.zeros(n)
        _check(self._lib.PredictSpecificClassFlat(self._h, n, _row_pointers(x, ctypes.c_float), x.shape[1], class_id,
                                                  self._dp(out), n))
        return out

    def calc_leaf_indexes_flat(self, features, tree_start=0, tree_end=None):
        x = np.ascontiguousarray(features, dtype=np.float32)
        n = x.shape[0]
        te = self.tree_count if tree_end is None else tree_end
        out = np.zeros(max(n * (te - tree_start), 1), dtype=np.uint32)
        _check(self._lib.CbHipCalcLeafIndexesFlat(self._h, n, _row_pointers(x, ctypes.c_float), x.shape[1], tree_start,
                                                  te, out.ctypes.data, n * (te - tree_start)))
        return out[:n * (te - tree_start)].reshape(n, te - tree_start)

    def quantize_flat(self, features):
        """Bins in the reference layout (blocks of 128 docs, [block][bucket][doc]), flattened."""
        x = np.ascontiguousarray(features, dtype=np.float32)
        n = x.shape[0]
        size = n * self.bucket_count
        out = np.zeros(max(size, 1), dtype=np.uint8)
        _check(self._lib.CbHipQuantizeFlat(self._h, n, _row_pointers(x, ctypes.c_float), x.shape[1], out.ctypes.data, size))
        return out[:size]

    def quantize_hashed(self, float_features, hashed_cat_features):
        x = np.ascontiguousarray(float_features, dtype=np.float32)
        c = np.ascontiguousarray(hashed_cat_features, dtype=np.int32)
        n = max(x.shape[0], c.shape[0])
        size = n * self.bucket_count
        out = np.zeros(max(size, 1), dtype=np.uint8)
        frows = _row_pointers(x, ctypes.c_float) if x.shape[1] else None
        crows = _row_pointers(c, ctypes.c_int) if c.shape[1] else None
        _check(self._lib.CbHipQuantizeWithHashedCatFeatures(self._h, n, frows, x.shape[1], crows, c.shape[1],
                                                            out.ctypes.data, size))
        return out[:size]
