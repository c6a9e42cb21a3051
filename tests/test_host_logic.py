"""Host-side logic of libcatboostmodel.so that needs no GPU: exported symbols, .cbm reader /
writer, model builders, hashes, error reporting."""
import ctypes
import os
import re
import time

import numpy as np
import pytest

import catboost_amd as cb
from oracle import model_builder as mb
from oracle.cbm_reader import ctr_base_key, read_cbm, read_cbm_file
from oracle.oracle import OracleModel
from tests import refmodels as rm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# export list of the reference library (catboost/libs/model_interface/calcer.exports)
REFERENCE_EXPORTS = """GetErrorString ModelCalcerCreate ModelCalcerDelete DataWrapperCreate DataWrapperDelete
AddFloatFeatures AddCatFeatures AddTextFeatures AddEmbeddingFeatures BuildDataProvider LoadFullModelFromFile
LoadFullModelFromBuffer LoadFullModelZeroCopy EnableGPUEvaluation GetSupportedEvaluatorTypes SetPredictionType
SetPredictionTypeString CalcModelPrediction CalcModelPredictionStaged CalcModelPredictionText
CalcModelPredictionTextStaged CalcModelPredictionTextAndEmbeddings CalcModelPredictionTextAndEmbeddingsStaged
CalcModelPredictionSingle CalcModelPredictionSingleStaged CalcModelPredictionFlat CalcModelPredictionFlatStaged
CalcModelPredictionFlatTransposed CalcModelPredictionFlatTransposedStaged CalcModelPredictionWithHashedCatFeatures
CalcModelPredictionWithHashedCatFeaturesAndTextFeatures
CalcModelPredictionWithHashedCatFeaturesAndTextAndEmbeddingFeatures PredictSpecificClassFlat PredictSpecificClass
PredictSpecificClassText PredictSpecificClassTextAndEmbeddings PredictSpecificClassSingle
PredictSpecificClassWithHashedCatFeatures PredictSpecificClassWithHashedCatFeaturesAndTextFeatures
PredictSpecificClassWithHashedCatFeaturesAndTextAndEmbeddingFeatures GetStringCatFeatureHash GetIntegerCatFeatureHash
GetFloatFeaturesCount GetCatFeaturesCount GetTextFeaturesCount GetEmbeddingFeaturesCount GetTreeCount
GetDimensionsCount GetPredictionDimensionsCount CheckModelMetadataHasKey GetModelInfoValueSize GetModelInfoValue
GetModelUsedFeaturesNames GetCatFeatureIndices GetFloatFeatureIndices GetTextFeatureIndices
GetEmbeddingFeatureIndices""".split()


def _declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:CbHip|[A-Z])[A-Za-z0-9]+)\s*\(", text)) - {"CATBOOST_API"})


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(cb.library_path())
    declared = _declared_functions("c_api.h") + _declared_functions("cb_hip_evaluator.h")
    assert len(declared) > 80
    for name in declared + REFERENCE_EXPORTS:
        assert hasattr(lib, name), name
    assert len(REFERENCE_EXPORTS) == 57
    assert set(REFERENCE_EXPORTS) <= set(_declared_functions("c_api.h"))


def test_hash_known_answers_through_c_api():
    for s, expected in rm.HASH_KNOWN_ANSWERS.items():
        assert cb.string_cat_feature_hash(s) == expected
    for v in (0, 7, -12, 10 ** 15):
        assert cb.integer_cat_feature_hash(v) == cb.string_cat_feature_hash(str(v))
    # every length class of the hash (0, 1-3, 4-8, 9-16, 17-32, 33-64, >64 bytes) against the oracle's copy
    from oracle.oracle import cat_feature_hash_signed
    rng = np.random.default_rng(0)
    for n in list(range(0, 70)) + [127, 128, 129, 200, 1000]:
        s = bytes(rng.integers(1, 256, size=n, dtype=np.uint8))
        assert cb.string_cat_feature_hash(s) == cat_feature_hash_signed(s)


@pytest.mark.parametrize("name", ["numeric_only_model.cbm", "features_num__dataset_querywise.cbm",
                                  "rust_tmp_model.cbm", "iris_model.cbm", "boston_housing_model.cbm"])
def test_cbm_load_save_roundtrip(golden_dir, name):
    path = os.path.join(golden_dir, name)
    ref = read_cbm_file(path)
    m = cb.ModelCalcer(path)
    got = read_cbm(m.save_to_buffer())
    for k in ("approx_dimension", "tree_splits", "tree_sizes", "tree_start_offsets", "leaf_values", "leaf_weights",
              "step_nodes", "node_id_to_leaf_id", "scale", "bias", "info"):
        np.testing.assert_array_equal(np.asarray(got[k]), np.asarray(ref[k]), err_msg=k)
    assert len(got["float_features"]) == len(ref["float_features"])
    for a, b in zip(got["float_features"], ref["float_features"]):
        np.testing.assert_array_equal(a["borders"], b["borders"])
        assert {k: a[k] for k in a if k != "borders"} == {k: b[k] for k in b if k != "borders"}
    assert got["cat_features"] == ref["cat_features"]
    for a, b in zip(got["one_hot_features"], ref["one_hot_features"]):
        assert a["cat_index"] == b["cat_index"]
        np.testing.assert_array_equal(a["values"], b["values"])
    # the writer always stores the recomputed repacked bins (TModelTrees::FBSerialize)
    assert got["repacked_bins_in_file"].size == got["tree_splits"].size
    if ref["repacked_bins_in_file"].size:
        np.testing.assert_array_equal(got["repacked_bins_in_file"], ref["repacked_bins_in_file"])
    # a second generation is byte-identical
    assert cb.ModelCalcer(buffer=m.save_to_buffer()).save_to_buffer() == m.save_to_buffer()


def test_model_description_getters(golden_dir):
    m = cb.ModelCalcer(os.path.join(golden_dir, "rust_tmp_model.cbm"))
    assert (m.tree_count, m.dimensions_count, m.float_features_count, m.cat_features_count) == (1000, 1, 3, 1)
    assert m.get_float_feature_indices() == [0, 1, 3] and m.get_cat_feature_indices() == [2]
    assert m.get_used_features_names()[2] == "wind direction"
    assert m.check_metadata_has_key("params") and not m.check_metadata_has_key("nope")
    assert m.get_metadata_key_value("params").startswith("{")
    assert m.prediction_dimensions_count == 1
    iris = cb.ModelCalcer(os.path.join(golden_dir, "iris_model.cbm"))
    assert iris.prediction_dimensions_count == 3
    iris.set_prediction_type("Class")
    assert iris.prediction_dimensions_count == 1
    with pytest.raises(cb.CatBoostError):
        iris.set_prediction_type("NoSuchType")


def test_loader_rejects_bad_input(golden_dir):
    with pytest.raises(cb.CatBoostError, match="Incorrect model file descriptor"):
        cb.ModelCalcer(os.path.join(golden_dir, "not_a_model.cbm"))
    with pytest.raises(cb.CatBoostError, match="can't open"):
        cb.ModelCalcer(os.path.join(golden_dir, "no_such_file.cbm"))
    data = open(os.path.join(golden_dir, "numeric_only_model.cbm"), "rb").read()
    for cut in (3, 7, 8, 20, len(data) // 2, len(data) - 1):
        with pytest.raises(cb.CatBoostError):
            cb.ModelCalcer(buffer=data[:cut])
    # flip bytes inside the flatbuffer: must fail cleanly or load, never crash
    rng = np.random.default_rng(1)
    for _ in range(200):
        corrupted = bytearray(data)
        for pos in rng.integers(8, len(data), size=4):
            corrupted[pos] = int(rng.integers(0, 256))
        try:
            cb.ModelCalcer(buffer=bytes(corrupted))
        except cb.CatBoostError:
            pass
    # a damaged dimension field must not turn into gigabytes of bias before the loader gives up
    start = time.time()
    for pos, value in ((2243, 0x10), (2242, 0x7f)):
        corrupted = bytearray(data)
        corrupted[pos] = value
        with pytest.raises(cb.CatBoostError, match="dimension"):
            cb.ModelCalcer(buffer=bytes(corrupted))
    assert time.time() - start < 5
    # text features stay out of reach: the model part that carries their dictionaries is refused
    with pytest.raises(cb.CatBoostError, match="not supported"):
        cb.ModelCalcer(os.path.join(golden_dir, "jvm_model_with_text_features.cbm"))


def test_loader_reads_ctr_models(golden_dir):
    """Models with CTR features and the tables of their static CTR provider load; the counts are those
    the reference's binding tests expect (node-package/bindings/tests/model.ts:329-343)."""
    adult = cb.ModelCalcer(os.path.join(golden_dir, "node_adult.cbm"))
    assert adult.float_features_count == 6 and adult.cat_features_count == 8
    for name in rm.CTR_FIXTURES:
        m = cb.ModelCalcer(os.path.join(golden_dir, name))
        expected = read_cbm_file(os.path.join(golden_dir, name))
        borders = sum(len(f["borders"]) for f in expected["float_features"])
        buckets = sum((len(f["borders"]) + 253) // 254 for f in expected["float_features"]) + \
            sum((len(o["values"]) + 253) // 254 for o in expected["one_hot_features"]) + \
            sum((len(c["borders"]) + 253) // 254 for c in expected["ctr_features"])
        assert m.bucket_count == buckets and m.tree_count == len(expected["tree_sizes"]) and borders >= 0
        # saved again (CTR features in the core, the static CTR provider as a trailing part), the model
        # reads back with the same tables through the oracle's reader and through the library
        saved = m.save_to_buffer()
        again = read_cbm(saved)
        assert again["model_part_ids"] == ["static_provider_v1"]
        assert len(again["ctr_tables"]) == len({bytes(str(t["base"]), "utf8") for t in expected["ctr_tables"]})
        for a, b in zip(again["ctr_features"], expected["ctr_features"]):
            np.testing.assert_array_equal(a["borders"], b["borders"])
            assert str(a["base"]) == str(b["base"])
            assert [a[k] for k in ("target_border_idx", "prior_num", "prior_denom", "shift", "scale")] == \
                [b[k] for k in ("target_border_idx", "prior_num", "prior_denom", "shift", "scale")]
        floats, cats = rm.random_ctr_inputs(expected, 800, 9, rm.known_cat_hashes(expected))
        np.testing.assert_array_equal(OracleModel(again).calc(floats, cats, layout="split"),
                                      OracleModel(expected).calc(floats, cats, layout="split"))
        assert cb.ModelCalcer(buffer=saved).save_to_buffer() == saved
    # a damaged CTR part fails cleanly (or loads), and never crashes
    data = open(os.path.join(golden_dir, "jvm_model_with_ctr.cbm"), "rb").read()
    core = int.from_bytes(data[4:8], "little")
    for cut in (8 + core, 8 + core + 3, 8 + core + 4, 8 + core + 9, len(data) - 1):
        with pytest.raises(cb.CatBoostError):
            cb.ModelCalcer(buffer=data[:cut])
    rng = np.random.default_rng(2)
    for _ in range(300):
        corrupted = bytearray(data)
        for pos in rng.integers(8 + core, len(data), size=3):
            corrupted[pos] = int(rng.integers(0, 256))
        try:
            cb.ModelCalcer(buffer=bytes(corrupted))
        except cb.CatBoostError:
            pass


def test_oblivious_builder_matches_oracle_builder():
    rng = np.random.default_rng(11)
    ffs = [mb.float_feature(i, i, has_nans=bool(i % 2), nan_treatment=i % 3) for i in range(5)]
    cfs = [mb.cat_feature(0, 5), mb.cat_feature(1, 6)]
    cands = [np.unique(rng.normal(size=30).astype(np.float32)) for _ in range(5)]
    trees = []
    for _ in range(40):
        splits = []
        for _ in range(int(rng.integers(0, 7))):
            if rng.random() < 0.2:
                splits.append(("onehot", 1, int(rng.integers(-3, 5))))
            else:
                f = int(rng.integers(0, 5))
                splits.append(("float", f, float(rng.choice(cands[f]))))
        trees.append((splits, rng.normal(size=(1 << len(splits)) * 2)))
    ref = mb.build_oblivious(ffs, cfs, 2, trees, scale=2.0, bias=[0.5, -0.5])
    b = cb.ModelCalcer()
    b.build_oblivious(ffs, cfs, 2, trees, scale=2.0, bias=[0.5, -0.5])
    got = read_cbm(b.save_to_buffer())
    for k in ("tree_splits", "tree_sizes", "tree_start_offsets", "leaf_values", "bias", "scale"):
        np.testing.assert_array_equal(np.asarray(got[k]), np.asarray(ref[k]), err_msg=k)
    for a, c in zip(got["float_features"], ref["float_features"]):
        np.testing.assert_array_equal(a["borders"], c["borders"])
        assert (a["has_nans"], a["nan_treatment"]) == (c["has_nans"], c["nan_treatment"])
    assert [c["used"] for c in got["cat_features"]] == [False, True]
    np.testing.assert_array_equal(got["one_hot_features"][0]["values"], ref["one_hot_features"][0]["values"])
    # repacked bins written by the library equal the oracle's derivation
    from oracle.oracle import OracleModel
    feat, xor, split = OracleModel(ref).repacked_bins()
    packed = feat.astype(np.uint32) | (xor.astype(np.uint32) << 16) | (split.astype(np.uint32) << 24)
    np.testing.assert_array_equal(got["repacked_bins_in_file"], packed)


def test_non_symmetric_builder_matches_oracle_builder():
    rng = np.random.default_rng(5)

    def grow(depth):
        if depth >= 5 or rng.random() < 0.3:
            return mb.leaf_node([float(rng.normal()), float(rng.normal())])
        return mb.split_node(("float", int(rng.integers(0, 4)), float(np.float32(rng.normal()))), grow(depth + 1), grow(depth + 1))

    ffs = [mb.float_feature(i) for i in range(4)]
    heads = [grow(0) for _ in range(25)]
    ref = mb.build_non_symmetric(ffs, [], 2, heads)
    b = cb.ModelCalcer()
    b.build_non_symmetric(ffs, [], 2, heads)
    got = read_cbm(b.save_to_buffer())
    for k in ("tree_splits", "tree_sizes", "tree_start_offsets", "leaf_values", "step_nodes", "node_id_to_leaf_id"):
        np.testing.assert_array_equal(got[k], ref[k], err_msg=k)


def test_convert_oblivious_to_asymmetric_matches_oracle():
    model = rm.simple_float_model(tree_count=2)
    m = cb.ModelCalcer()
    m.load_from_dict(model)
    m.convert_oblivious_to_asymmetric()
    got = read_cbm(m.save_to_buffer())
    ref = mb.convert_oblivious_to_asymmetric(model)
    for k in ("tree_splits", "tree_sizes", "tree_start_offsets", "leaf_values", "step_nodes", "node_id_to_leaf_id"):
        np.testing.assert_array_equal(got[k], ref[k], err_msg=k)


def test_invalid_tables_are_refused():
    model = rm.simple_float_model()
    bad = dict(model, tree_splits=np.array([300, 301, 999], np.int32))
    with pytest.raises(cb.CatBoostError, match="out of range"):
        cb.ModelCalcer().load_from_dict(bad)
    bad = dict(model, leaf_values=model["leaf_values"][:5])
    with pytest.raises(cb.CatBoostError, match="leaf values"):
        cb.ModelCalcer().load_from_dict(bad)
    asym = mb.convert_oblivious_to_asymmetric(model)
    steps = asym["step_nodes"].copy()
    steps[0] = (200, 1)
    with pytest.raises(cb.CatBoostError, match="leaves its tree"):
        cb.ModelCalcer().load_from_dict(dict(asym, step_nodes=steps))
    m = cb.ModelCalcer()
    m.load_from_dict(model)
    with pytest.raises(cb.CatBoostError, match="bias"):
        m.set_scale_and_bias(1.0, np.zeros(3))


def test_prediction_without_gpu_fails_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    m = cb.ModelCalcer()
    m.load_from_dict(rm.simple_float_model())
    with pytest.raises(cb.CatBoostError, match="HIP"):
        m.calc_flat(rm.DATA)
    with pytest.raises(cb.CatBoostError, match="HIP"):
        m.enable_gpu_evaluation(0)


# --------------------------------------------------------------- prediction types ----

def test_library_exponent_matches_reference_fmath(golden_dir):
    """CbHipFastExpInplace against the vectors of the reference's fmath::expd_v, bit for bit."""
    g = np.load(os.path.join(golden_dir, "fmath_exp_vectors.npz"))
    for chunk in (1, 3, 4, 10, 128):
        np.testing.assert_array_equal(cb.fast_exp(g["x"], chunk).view(np.uint64), g["chunk_%d" % chunk].view(np.uint64))


def test_library_prediction_types_match_the_oracle():
    from oracle.oracle import PREDICTION_TYPES, apply_prediction_type

    rng = np.random.default_rng(8)
    cases = ((1, ("Probability", "Exponent", "Class", "RawFormulaVal")), (2, ("RMSEWithUncertainty", "Probability")),
             (3, ("Probability", "Class", "MultiProbability")), (10, ("Probability", "Class")))
    for dim, types in cases:
        for docs in (1, 5, 128, 129, 1000):
            raw = rng.normal(0, 5, size=docs * dim)
            raw[rng.random(raw.shape) < 0.01] = 800.0  # beyond the exponent's clamp
            for name in types:
                got = cb.apply_prediction_type(raw, dim, PREDICTION_TYPES[name])
                np.testing.assert_array_equal(got.view(np.uint64), apply_prediction_type(raw, dim, name).view(np.uint64))


# ------------------------------------------------------------------- json model format ----

def test_json_twin_of_the_numeric_only_fixture(golden_dir):
    """CatBoostModelTest.java:181-200 loads numeric_only_model.json; it must give the tables of its
    binary twin."""
    path = os.path.join(golden_dir, "numeric_only_model.json")
    from_json = read_cbm(cb.ModelCalcer(path, model_format="json").save_to_buffer())
    with open(path) as f:
        same = read_cbm(cb.ModelCalcer(buffer=f.read(), model_format="json").save_to_buffer())
    binary = read_cbm_file(os.path.join(golden_dir, "numeric_only_model.cbm"))
    for model in (from_json, same):
        for key in ("approx_dimension", "tree_splits", "tree_sizes", "tree_start_offsets", "leaf_values", "scale", "bias"):
            np.testing.assert_array_equal(np.asarray(model[key]), np.asarray(binary[key]), err_msg=key)
        for a, b in zip(model["float_features"], binary["float_features"]):
            np.testing.assert_array_equal(a["borders"], b["borders"])
            assert (a["index"], a["flat_index"], a["has_nans"], a["nan_treatment"]) == \
                (b["index"], b["flat_index"], b["has_nans"], b["nan_treatment"])
        assert "iterations" in model["info"]["params"]


@pytest.mark.parametrize("dim", [1, 3])
@pytest.mark.parametrize("asym", [False, True])
def test_json_import_of_random_models(dim, asym):
    """Random models (one-hot features, NaN modes, several dimensions, non-symmetric trees with nodes that
    are terminal on one side) written as json by the test's restatement of the reference's exporter:
    the imported model must predict what the original does (checked on the CPU oracle)."""
    from tests.test_oracle import _random_flat_data, _random_oblivious

    rng = np.random.default_rng(40 + dim + 10 * asym)
    model, cat_values = _random_oblivious(rng, dim=dim, trees=15, max_depth=5, scale=0.5, bias=list(rng.normal(size=dim)))
    if asym:
        model = mb.convert_oblivious_to_asymmetric(model)
    x = _random_flat_data(rng, model, cat_values, 500)
    imported = read_cbm(cb.ModelCalcer(buffer=rm.model_to_json(model), model_format="json").save_to_buffer())
    np.testing.assert_array_equal(OracleModel(imported).calc(x), OracleModel(model).calc(x))


def test_json_import_error_paths(golden_dir):
    text = open(os.path.join(golden_dir, "numeric_only_model.json")).read()
    for bad in ("", "[]", "{", text[:len(text) // 2], text.replace("oblivious_trees", "x"), text + "}",
                text.replace('"AsIs"', '"Maybe"', 1), text.replace("[", "[[[", 1)):
        with pytest.raises(cb.CatBoostError):
            cb.ModelCalcer(buffer=bad, model_format="json")
    rng = np.random.default_rng(3)
    raw = bytearray(text.encode())
    for _ in range(300):  # damaged text fails cleanly or loads; it never crashes
        corrupted = bytearray(raw)
        for pos in rng.integers(0, len(raw), size=3):
            corrupted[pos] = int(rng.integers(32, 127))
        try:
            cb.ModelCalcer(buffer=bytes(corrupted), model_format="json")
        except cb.CatBoostError:
            pass
    import json
    doc = json.loads(text)
    doc["features_info"]["ctrs"] = [{"borders": [0.5]}]  # a CTR feature without its description
    with pytest.raises(cb.CatBoostError, match="elements"):
        cb.ModelCalcer(buffer=json.dumps(doc), model_format="json")
    with pytest.raises(cb.CatBoostError, match="can't open"):
        cb.ModelCalcer(os.path.join(golden_dir, "no_such_model.json"), model_format="json")


def test_feature_layout_is_checked_when_it_is_set(golden_dir):
    """CbHipSetFeatureLayout needs an entry for every used feature in a list that is given
    (TFeatureLayout::GetRemappedPosition indexes the lists with at(), evaluation_interface.h:27-47)."""
    g = cb.ModelCalcer(os.path.join(golden_dir, "rust_tmp_model.cbm"))  # 3 float features, 1 categorical
    g.set_feature_layout(float_feature_indexes=[4, 0, 2], cat_feature_indexes=[1], flat_indexes=[3, 2, 1, 0])
    with pytest.raises(cb.CatBoostError, match="FloatFeatureIndexes has no entry"):
        g.set_feature_layout(float_feature_indexes=[4, 0])
    with pytest.raises(cb.CatBoostError, match="CatFeatureIndexes has no entry"):
        g.set_feature_layout(cat_feature_indexes=[])
    with pytest.raises(cb.CatBoostError, match="FlatIndexes has no entry"):
        g.set_feature_layout(flat_indexes=[0, 1, 2])
    g.set_feature_layout()


def json_view_of_ctr_model(model):
    """What the json format keeps of a model dict with CTR features: no TargetBorderClassifierIdx, and a
    mean CTR's sum only when it is a whole number (the reference reads it with GetInteger,
    json_model_helpers.cpp:562). None if two tables would share a key of ctr_data."""
    import copy

    kept = copy.deepcopy(model)
    keys = set()
    for t in kept["ctr_tables"]:
        t["base"]["target_border_classifier_idx"] = 0
        key = ctr_base_key(t["base"])
        if key in keys:
            return None
        keys.add(key)
        if t["base"]["ctr_type"] in (2, 3):
            rows = t["ctr_blob"].view(np.dtype([("sum", "<f4"), ("count", "<i4")]))
            whole = rows["sum"] == np.floor(rows["sum"])
            rows["sum"] = np.where(whole, rows["sum"], np.float32(0))
    for c in kept["ctr_features"]:
        c["base"]["target_border_classifier_idx"] = 0
    return kept


def test_json_import_of_ctr_models(golden_dir):
    """CTR features and their tables through the json format (CtrFeatureFromJson, CtrDataFromJson,
    json_model_helpers.cpp:119-136, 531-580): what the library saves afterwards holds the same features and,
    row for row, the same statistics as the model the json was written from."""
    from tests import ctr_models

    cases = [read_cbm_file(os.path.join(golden_dir, n)) for n in rm.CTR_FIXTURES]
    cases += [ctr_models.random_ctr_model(seed, **kwargs)[0] for seed, kwargs in ctr_models.CASES]
    checked = 0
    for model in cases:
        kept = json_view_of_ctr_model(model)
        if kept is None:
            continue
        checked += 1
        g = cb.ModelCalcer(buffer=rm.model_to_json(model), model_format="json")
        back = read_cbm(g.save_to_buffer())
        assert [ctr_base_key(c["base"]) for c in back["ctr_features"]] == [ctr_base_key(c["base"]) for c in kept["ctr_features"]]
        for a, b in zip(back["ctr_features"], kept["ctr_features"]):
            for k in ("target_border_idx", "prior_num", "prior_denom", "shift", "scale"):
                assert a[k] == b[k]
            np.testing.assert_array_equal(a["borders"], b["borders"])
        tables = {ctr_base_key(t["base"]): t for t in back["ctr_tables"]}
        assert len(tables) == len(kept["ctr_tables"])
        for t in kept["ctr_tables"]:
            got = tables[ctr_base_key(t["base"])]
            assert got["counter_denominator"] == t["counter_denominator"]
            if t["base"]["ctr_type"] in (0, 1):
                assert got["target_classes_count"] == t["target_classes_count"]

            def rows_by_hash(table):
                raw = np.asarray(table["index_hash_raw"], np.uint8).reshape(-1, 12)
                keys = raw[:, :8].copy().view(np.uint64).ravel()
                rows = raw[:, 8:].copy().view(np.uint32).ravel()
                width = {2: 8, 3: 8, 4: 4, 5: 4}.get(table["base"]["ctr_type"], 4 * max(table["target_classes_count"], 1))
                blob = np.asarray(table["ctr_blob"], np.uint8)
                return {int(k): blob[width * r:width * (r + 1)].tobytes() for k, r in zip(keys, rows)
                        if int(k) != 0xFFFFFFFFFFFFFFFF}

            assert rows_by_hash(got) == rows_by_hash(t)
    assert checked >= 8


def test_json_import_of_damaged_ctr_models(golden_dir):
    """Damaged text of a model with CTR features fails cleanly or loads; it never crashes."""
    import json

    model = read_cbm_file(os.path.join(golden_dir, "jvm_model_with_ctr.cbm"))
    text = rm.model_to_json(model)
    rng = np.random.default_rng(17)
    raw = bytearray(text.encode())
    for _ in range(400):
        corrupted = bytearray(raw)
        for pos in rng.integers(0, len(raw), size=3):
            corrupted[pos] = int(rng.integers(32, 127))
        try:
            cb.ModelCalcer(buffer=bytes(corrupted), model_format="json")
        except cb.CatBoostError:
            pass
    doc = json.loads(text)
    key = next(iter(doc["ctr_data"]))
    for change in ({"hash_stride": 0}, {"hash_stride": 7}, {"hash_map": ["12", 1]}, {"hash_map": [12, 1, 2]},
                   {"hash_map": ["-5", 1, 2]}, {"hash_map": ["18446744073709551615", 1, 2]}):
        bad = json.loads(text)
        bad["ctr_data"][key].update(change)
        with pytest.raises(cb.CatBoostError):
            cb.ModelCalcer(buffer=json.dumps(bad), model_format="json")
    bad = json.loads(text)
    del bad["ctr_data"][key]  # a CTR feature without its table
    with pytest.raises(cb.CatBoostError, match="CTR"):
        cb.ModelCalcer(buffer=json.dumps(bad), model_format="json")
