"""Pins the CPU oracle against what the reference itself holds: unit-test closed forms, .cbm
fixtures with golden predictions, hash known answers, and mathematical invariants.
CPU only (no GPU needed)."""
import json
import os

import numpy as np
import pytest

from oracle import model_builder as mb
from oracle.cbm_reader import ctr_base_key, read_cbm, read_cbm_file
from oracle.oracle import (OracleModel, apply_prediction_type, cat_feature_hash_signed, city_hash64,
                           integer_cat_feature_hash)
from tests import cbm_writer, ctr_models
from tests import refmodels as rm


# ------------------------------------------------------------------ hash known answers ----

def test_cat_feature_hash_known_answers():
    # CatBoostModelTest.java:122-134; covers the len<4 ("foo") and 4<=len<=8 ("😡") branches
    for s, expected in rm.HASH_KNOWN_ANSWERS.items():
        assert cat_feature_hash_signed(s) == expected


def test_city_hash_empty_string_is_k2():
    # HashLen0to16 returns k2 for the empty string, util/digest/city.cpp:99
    assert city_hash64("") == 0x9ae16a3b2f90404f


def test_integer_hash_is_hash_of_decimal_string():
    # c_api.cpp:944-949
    for v in (0, 1, 9, 10, -5, 123456789012345):
        assert integer_cat_feature_hash(v) == cat_feature_hash_signed(str(v))


def test_rust_fixture_one_hot_value_is_hash_of_north():
    # the single one-hot value stored in rust-package/tmp/model.bin must be the hash of one of
    # the two category strings of its test ("north"/"south", model.rs:337-341): a 5-byte string,
    # i.e. the 4<=len<=8 branch through a second, end-to-end, vector
    m = read_cbm_file(os.path.join(os.path.dirname(__file__), "golden", "rust_tmp_model.cbm"))
    value = int(m["one_hot_features"][0]["values"][0])
    assert value in (cat_feature_hash_signed("north"), cat_feature_hash_signed("south"))


# ------------------------------------------------------------ reference unit-test models ----

def _check(model, data, predictions, leaf_indexes):
    o = OracleModel(model)
    np.testing.assert_array_equal(o.calc(data), np.asarray(predictions, dtype=np.float64))
    np.testing.assert_array_equal(o.leaf_indexes(data), np.asarray(leaf_indexes, dtype=np.uint32))
    bf_pred, bf_idx = o.bruteforce(data)
    np.testing.assert_array_equal(bf_pred, np.asarray(predictions, dtype=np.float64))
    np.testing.assert_array_equal(bf_idx, np.asarray(leaf_indexes, dtype=np.uint32))
    # single-doc path (CalcFlatSingle / CalcLeafIndexesSingle)
    for i in range(data.shape[0]):
        np.testing.assert_array_equal(o.calc(data[i:i + 1]),
                                      np.asarray(predictions, dtype=np.float64).reshape(data.shape[0], -1)[i])


def _check_both_forms(model, data, predictions, leaf_indexes):
    _check(model, data, predictions, leaf_indexes)
    _check(mb.convert_oblivious_to_asymmetric(model), data, predictions, leaf_indexes)


def test_simple_float_model_301_borders_two_buckets():
    # formula_evaluator_ut.cpp:76-81
    model = rm.simple_float_model()
    o = OracleModel(model)
    assert o.bucket_count == 4
    feat, xor, split = o.repacked_bins()
    assert list(feat) == [1, 2, 3] and list(split) == [47, 1, 1] and list(xor) == [0, 0, 0]
    _check_both_forms(model, rm.DATA, np.arange(8.0), np.arange(8).reshape(8, 1))


def test_simple_float_model_scale_and_bias():
    # formula_evaluator_ut.cpp:83-95
    model = rm.simple_float_model(scale=0.5, bias=[0.125])
    _check_both_forms(model, rm.DATA, 0.5 * np.arange(8.0) + 0.125, np.arange(8).reshape(8, 1))


def test_two_trees():
    # formula_evaluator_ut.cpp:97-109
    model = rm.simple_float_model(tree_count=2)
    _check_both_forms(model, rm.DATA, 11.0 * np.arange(8.0), np.repeat(np.arange(8), 2).reshape(8, 2))


def test_deep_tree_depth_9():
    # formula_evaluator_ut.cpp:111-132
    model = rm.simple_deep_tree_model(9)
    _check_both_forms(model, rm.deep_tree_data(9), np.arange(512.0), np.arange(512).reshape(512, 1))


def test_multi_value_model():
    # formula_evaluator_ut.cpp:134-146
    model = rm.multi_value_float_model()
    expected = [0., 10., 20., 1., 11., 21., 2., 12., 22., 3., 13., 23.]
    _check_both_forms(model, rm.DATA[:4], expected, np.arange(4).reshape(4, 1))


def test_simple_asymmetric_model():
    # formula_evaluator_ut.cpp:284-307
    model = rm.simple_asymmetric_model()
    # pre-order layout with the lone leaf child folded into its parent, model_build_helper.cpp:249-304
    assert model["step_nodes"].tolist() == [[1, 0], [1, 2], [0, 0], [0, 0], [1, 2], [0, 0], [0, 0], [0, 1], [1, 2],
                                            [0, 0], [0, 0]]
    assert model["leaf_values"].tolist() == [3.0, 1.0, 2.0, 0.0, 10.0, 100.0, 200.0, 300.0]
    _check(model, rm.DATA, rm.ASYMMETRIC_PREDICTIONS, rm.ASYMMETRIC_LEAF_INDEXES)


def test_non_symmetric_builder_keeps_only_used_borders():
    # model_serialization_ut.cpp:112-224: only borders used by splits survive, split ids are the
    # ranks in the sorted split set
    ffs = [mb.float_feature(i) for i in range(3)]
    head = mb.split_node(("float", 2, 0.75), mb.leaf_node(1.0),
                         mb.split_node(("float", 0, 0.25), mb.leaf_node(2.0), mb.leaf_node(3.0)))
    model = mb.build_non_symmetric(ffs, [], 1, [head])
    assert [f["borders"].tolist() for f in model["float_features"]] == [[0.25], [], [0.75]]
    assert model["tree_splits"].tolist() == [1, 0, 0, 0]


def test_zero_trees_returns_bias():
    # cpu/formula_evaluator.cpp:29-41
    model = rm.simple_float_model(tree_count=0, bias=[0.75])
    o = OracleModel(model)
    np.testing.assert_array_equal(o.calc(rm.DATA), np.full(8, 0.75))


def test_staged_ranges_add_up_and_bias_only_at_tree_zero():
    # scale_and_bias.cpp:13-24
    model = rm.simple_float_model(tree_count=2, scale=0.5, bias=[0.125])
    o = OracleModel(model)
    full = o.calc(rm.DATA)
    first = o.calc(rm.DATA, tree_start=0, tree_end=1)
    second = o.calc(rm.DATA, tree_start=1, tree_end=2)
    np.testing.assert_array_equal(first, 0.5 * np.arange(8.0) + 0.125)
    np.testing.assert_array_equal(second, 0.5 * 10.0 * np.arange(8.0))
    np.testing.assert_allclose(first + second, full, rtol=0, atol=1e-12)


# ------------------------------------------------------------------- fixtures + goldens ----

def test_numeric_only_fixture(golden_dir):
    m = read_cbm_file(os.path.join(golden_dir, "numeric_only_model.cbm"))
    o = OracleModel(m)
    got = o.calc(rm.NUMERIC_ONLY_ROWS)
    np.testing.assert_array_equal(got, rm.NUMERIC_ONLY_EXPECTED)
    # transposed API, CatBoostModelTest.java:359-374
    got_t = o.calc(np.ascontiguousarray(rm.NUMERIC_ONLY_ROWS.T), layout="transposed")
    np.testing.assert_array_equal(got_t, rm.NUMERIC_ONLY_EXPECTED)


def test_numeric_only_fixture_matches_its_json_twin(golden_dir):
    """The .json export of the same model spells out borders, splits and leaf values; the
    binary reader must see the same model."""
    m = read_cbm_file(os.path.join(golden_dir, "numeric_only_model.cbm"))
    with open(os.path.join(golden_dir, "numeric_only_model.json")) as f:
        j = json.load(f)
    jf = j["features_info"]["float_features"]
    assert len(jf) == len(m["float_features"])
    for a, b in zip(jf, m["float_features"]):
        assert a["feature_index"] == b["index"] and a["flat_feature_index"] == b["flat_index"]
        np.testing.assert_array_equal(np.asarray(a["borders"], np.float32), b["borders"])
    trees = j["oblivious_trees"]
    assert len(trees) == len(m["tree_sizes"])
    leaves = np.concatenate([np.asarray(t["leaf_values"], np.float64) for t in trees])
    np.testing.assert_array_equal(leaves, m["leaf_values"])
    # each json split names (float_feature_index, border); the binary names a bin feature id
    flat_borders = [(f["index"], float(b)) for f in m["float_features"] for b in f["borders"]]
    k = 0
    for t in trees:
        for s in t["splits"]:
            fi, border = flat_borders[m["tree_splits"][k]]
            assert fi == s["float_feature_index"] and np.float32(border) == np.float32(s["border"])
            k += 1


def test_rust_fixture_with_one_hot_cat(golden_dir):
    m = read_cbm_file(os.path.join(golden_dir, "rust_tmp_model.cbm"))
    o = OracleModel(m)
    cats = np.array([[cat_feature_hash_signed(c) for c in row] for row in rm.RUST_CATS], np.int32)
    got = o.calc(rm.RUST_FLOATS, cats, layout="split")
    np.testing.assert_array_equal(got, rm.RUST_EXPECTED)
    bf, _ = o.bruteforce(rm.RUST_FLOATS, cats, layout="split")
    np.testing.assert_allclose(bf, rm.RUST_EXPECTED, rtol=1e-12, atol=0)


def test_querywise_fixture(golden_dir):
    m = read_cbm_file(os.path.join(golden_dir, "features_num__dataset_querywise.cbm"))
    o = OracleModel(m)
    got = o.calc(rm.querywise_rows())
    # printed to 16-17 significant digits in model.rs:449-454
    np.testing.assert_allclose(got, rm.QUERYWISE_EXPECTED, rtol=1e-14, atol=1e-17)


def test_iris_fixture_three_dims(golden_dir):
    # CatBoostModelEvaluatorTest.cs:20-44: argmax of the 3 raw values equals the label
    m = read_cbm_file(os.path.join(golden_dir, "iris_model.cbm"))
    assert m["approx_dimension"] == 3
    o = OracleModel(m)
    feats, labels = rm.load_iris(golden_dir)
    assert feats.shape == (150, 4)
    pred = o.calc(feats).reshape(-1, 3)
    np.testing.assert_array_equal(np.argmax(pred, axis=1), labels)
    bf, bf_idx = o.bruteforce(feats)
    np.testing.assert_allclose(bf, pred.ravel(), rtol=1e-12, atol=1e-12)
    np.testing.assert_array_equal(bf_idx, o.leaf_indexes(feats))


def test_boston_fixture(golden_dir):
    # CatBoostModelEvaluatorTest.cs:46-103: |pred - log(target)| >= 0.4 on at most 7 rows
    m = read_cbm_file(os.path.join(golden_dir, "boston_housing_model.cbm"))
    o = OracleModel(m)
    feats, target = rm.load_boston(golden_dir)
    pred = o.calc(feats)
    assert int(np.sum(np.abs(pred - np.log(target)) >= 0.4)) <= 7


@pytest.mark.parametrize("name", rm.CTR_FIXTURES)
def test_ctr_fixtures_are_recognised(golden_dir, name):
    m = read_cbm_file(os.path.join(golden_dir, name))
    assert m["ctr_feature_count"] > 0 and "static_provider_v1" in m["model_part_ids"]
    assert len(m["ctr_features"]) == m["ctr_feature_count"] and len(m["ctr_tables"]) > 0


def _hashed(rows):
    return np.array([[cat_feature_hash_signed(s) for s in r] for r in rows], np.int32)


def test_ctr_goldens_of_the_jvm_tests(golden_dir):
    # CatBoostModelTest.java:457-470, 528-547 (categorical features only) and :586-601, 720-743
    o = OracleModel(read_cbm_file(os.path.join(golden_dir, "categoric_only_model.cbm")))
    cats = _hashed(rm.JVM_CATEGORIC_ONLY_CATS)
    np.testing.assert_array_equal(o.calc(np.zeros((3, 0), np.float32), cats, layout="split"),
                                  rm.JVM_CATEGORIC_ONLY_EXPECTED)
    o = OracleModel(read_cbm_file(os.path.join(golden_dir, "jvm_model_with_ctr.cbm")))
    np.testing.assert_array_equal(o.calc(rm.JVM_CTR_FLOATS, _hashed(rm.JVM_CTR_CATS), layout="split"),
                                  rm.JVM_CTR_EXPECTED)


def test_ctr_goldens_of_the_rust_and_node_tests(golden_dir):
    # rust-package/src/model.rs:459-499: 26 CTRs of kinds Borders and Counter plus a one-hot feature
    o = OracleModel(read_cbm_file(os.path.join(golden_dir, "features_num_cat__dataset_adult.cbm")))
    pred = o.calc(rm.RUST_ADULT_FLOATS, _hashed(rm.RUST_ADULT_CATS), layout="split")
    np.testing.assert_allclose(pred, rm.RUST_ADULT_EXPECTED, rtol=0, atol=1e-15)
    # node-package/bindings/tests/model.ts:67-96
    o = OracleModel(read_cbm_file(os.path.join(golden_dir, "node_adult.cbm")))
    pred = o.calc(rm.NODE_ADULT_FLOATS, _hashed(rm.NODE_ADULT_CATS), layout="split")
    assert ["%.2f" % v for v in pred] == rm.NODE_ADULT_EXPECTED_2DP


def test_ctr_mushroom_labels(golden_dir):
    # CatBoostModelEvaluatorTest.cs:101-127: 159 CTRs over one to four categorical features, some with a
    # one-hot split in the projection; every one of the 8124 rows must get its label
    o = OracleModel(read_cbm_file(os.path.join(golden_dir, "mushroom_model.cbm")))
    labels, rows = rm.mushrooms(golden_dir)
    assert len(rows) == 8124
    pred = o.calc(np.zeros((len(rows), 0), np.float32), _hashed(rows), layout="split")
    np.testing.assert_array_equal(pred > 0, np.array(labels) == "p")


@pytest.mark.parametrize("name", rm.CTR_FIXTURES)
def test_ctr_models_against_the_raw_definition(golden_dir, name):
    """The block-wise path (bins of the projection's splits, transposed hashes) against a per-document
    evaluation from the raw features, in all three input layouts."""
    m = read_cbm_file(os.path.join(golden_dir, name))
    o = OracleModel(m)
    floats, cats = rm.random_ctr_inputs(m, 1500, 7, rm.known_cat_hashes(m))
    pred = o.calc(floats, cats, layout="split")
    bf, bf_idx = o.bruteforce(floats, cats, layout="split")
    np.testing.assert_array_equal(pred, bf)
    np.testing.assert_array_equal(o.leaf_indexes(floats, cats, layout="split"), bf_idx)
    flat = rm.flat_rows(m, floats, cats)
    np.testing.assert_array_equal(o.calc(flat), pred)
    np.testing.assert_array_equal(o.calc(np.ascontiguousarray(flat.T), layout="transposed"), pred)
    # known and unknown categories both occur
    ctrs = o.ctrs(floats, cats, layout="split")
    assert all(len(np.unique(row)) > 1 for row in ctrs)


def multiclass_classes_count_case(golden_dir, name):
    """(model path, features, expected probabilities of the model's own dimensions) of a canonical case of
    the reference's test_multiclass_classes_count (catboost/python-package/ut/medium/test.py:1979-2031):
    model.bin and predictions.txt are its canondata, the 100 x 10 features are the numpy RandomState(0)
    draw that the test makes. With labels 1 and 3 only ("missed") the model has two dimensions and the
    stored table four columns: the Python package spreads the two over the declared classes
    (class_to_label [1, 3] in the model's class_params) and leaves ~1e-308 in the others."""
    path = os.path.join(golden_dir, "multiclass_classes_count_%s.cbm" % name)
    features = np.random.RandomState(seed=0).random_sample(size=(100, 10)).astype(np.float32)
    expected = np.loadtxt(os.path.join(golden_dir, "multiclass_classes_count_%s.predictions.txt" % name))
    assert expected.shape == (100, 4)
    if name == "missed":
        assert np.abs(expected[:, [0, 2]]).max() < 1e-300
        expected = expected[:, [1, 3]]
    return path, features, expected


@pytest.mark.parametrize("name", ["all", "missed"])
def test_multiclass_probabilities_of_the_reference_canondata(golden_dir, name):
    """Softmax probabilities of a trained multi-class model against the 17-digit table that the
    reference's own test stores: equal to the last bit (multi-dimensional leaves, the sum over trees,
    CalcSoftmax with the reference's exponent)."""
    path, features, expected = multiclass_classes_count_case(golden_dir, name)
    o = OracleModel(read_cbm_file(path))
    assert o.dim == expected.shape[1]
    got = apply_prediction_type(o.calc(features), o.dim, "Probability").reshape(100, -1)
    np.testing.assert_array_equal(got, expected)


def test_model_of_the_backward_compatibility_test(golden_dir):
    """test_multiclass_model_backward_compatibility (catboost/pytest/test.py:7543-7571): a three-class model
    written by an old version (catboost/pytest/data/multiclass_model.bin, copied) applied to
    cloudness_small/train_small; the canonical outputs of `catboost calc` for the three prediction types
    are printed with 10 digits. The .npz holds the pool's numeric columns (categorical ones, which the
    model's tree does not look at, as zeros) and those tables."""
    v = np.load(os.path.join(golden_dir, "cloudness_backward_compatibility.npz"))
    m = read_cbm_file(os.path.join(golden_dir, "cloudness_backward_compatibility.cbm"))
    assert "class_params" not in m["info"]
    o = OracleModel(m)
    raw = o.calc(v["features"])
    np.testing.assert_allclose(raw.reshape(-1, 3), v["RawFormulaVal"], rtol=6e-10, atol=0)
    np.testing.assert_allclose(apply_prediction_type(raw, 3, "Probability").reshape(-1, 3), v["Probability"],
                               rtol=6e-10, atol=0)
    np.testing.assert_array_equal(apply_prediction_type(raw, 3, "Class"), v["Class"].ravel())


@pytest.mark.parametrize("name", ["cat", "nocat"])
def test_models_that_the_reference_holds_as_exported_cpp(golden_dir, name):
    """Two trained models that the reference keeps as exported C++ code, tables and applier in one file
    (canonical outputs of its export tests; run by tests/golden/make_export_vectors.py, which also put
    the tables together into tests/golden/cpp_export_<name>.cbm): predictions of the oracle against that
    applier's on 3000 documents, floats on and around the borders, known and unknown categories. The
    sums run in the same order, so the values are equal bit for bit. For the model with categorical
    features (20 trees, 13 Borders and Counter CTRs) also the (bucket, split index, xor mask) of every
    tree split against the arrays the reference's exporter wrote, and the string hash on the 58 category
    names of the code's own table."""
    v = np.load(os.path.join(golden_dir, "cpp_export_vectors.npz"))
    m = read_cbm_file(os.path.join(golden_dir, "cpp_export_%s.cbm" % name))
    o = OracleModel(m)
    floats, cats = v["floats_" + name], v["cats_" + name]
    expected, comparable = v["predictions_" + name], v["comparable_" + name]
    assert comparable.mean() > 0.8 and len(np.unique(expected)) > 500
    got = o.calc(floats, cats, layout="split")
    np.testing.assert_array_equal(got[comparable], expected[comparable])
    np.testing.assert_array_equal(got, o.bruteforce(floats, cats, layout="split")[0])
    if name == "cat":
        bucket, xor_mask, split_idx = o.repacked_bins()
        np.testing.assert_array_equal(bucket, v["split_bucket_cat"])
        np.testing.assert_array_equal(split_idx, v["split_idx_cat"])
        np.testing.assert_array_equal(xor_mask, v["split_xor_mask_cat"])
        assert len(v["hash_strings_cat"]) == 58
        for text, value in zip(v["hash_strings_cat"], v["hash_values_cat"]):
            assert cat_feature_hash_signed(str(text)) == int(value)


@pytest.mark.parametrize("seed", [seed for seed, _ in ctr_models.CASES])
def test_ctr_values_match_the_reference_ctr_calculator(golden_dir, seed):
    """CTR values on synthetic models with all six CTR types, tables with up to five target classes and
    projections over categorical features, float splits (also beyond the first 254 borders of a feature)
    and one-hot splits, against what the reference's own calculator for exported models printed
    (model_export/resources/ctr_calcer.cpp, run by tests/golden/make_ctr_vectors.py): bit for bit. Pairs
    where that calculator and the evaluator differ by design (a hash that a Counter or FeatureFreq
    table does not hold) are excluded by the stored mask and checked against Calc(0, denominator)."""
    g = np.load(os.path.join(golden_dir, "ctr_ref_vectors.npz"))
    m = read_cbm_file(os.path.join(golden_dir, "synthetic_ctr_%d.cbm" % seed))
    o = OracleModel(m)
    floats, cats = g["floats_%d" % seed], g["cats_%d" % seed]
    got = o.ctrs(floats, cats, layout="split")
    expected, comparable = g["ctrs_%d" % seed], g["comparable_%d" % seed]
    assert comparable.mean() > 0.7
    np.testing.assert_array_equal(got.view(np.uint32)[comparable], expected.view(np.uint32)[comparable])
    tables = {ctr_base_key(t["base"]): t for t in m["ctr_tables"]}
    for i, c in enumerate(m["ctr_features"]):
        rest = ~comparable[i]
        if rest.any():
            assert c["base"]["ctr_type"] in (4, 5)
            denominator = np.float32(tables[ctr_base_key(c["base"])]["counter_denominator"])
            value = (np.float32(c["prior_num"]) / (denominator + np.float32(c["prior_denom"])) +
                     np.float32(c["shift"])) * np.float32(c["scale"])
            np.testing.assert_array_equal(got[i][rest], np.full(int(rest.sum()), value, np.float32))
    # every CTR type and both kinds of split occur in the cases taken together
    assert {c["base"]["ctr_type"] for c in m["ctr_features"]} <= set(range(6))
    # the block path over these models equals the per-document definition
    pred = o.calc(floats, cats, layout="split")
    bf, bf_idx = o.bruteforce(floats, cats, layout="split")
    np.testing.assert_array_equal(pred, bf)
    np.testing.assert_array_equal(o.leaf_indexes(floats, cats, layout="split"), bf_idx)


def test_synthetic_ctr_cases_cover_every_kind(golden_dir):
    types, classes, float_splits, one_hot_splits, wide = set(), set(), 0, 0, 0
    for seed, kwargs in ctr_models.CASES:
        path = os.path.join(golden_dir, "synthetic_ctr_%d.cbm" % seed)
        m = read_cbm_file(path)
        # the committed files are what the seeded generator and the writer produce
        with open(path, "rb") as f:
            assert f.read() == cbm_writer.write_cbm(ctr_models.random_ctr_model(seed, **kwargs)[0])
        borders = {f["index"]: f["borders"] for f in m["float_features"]}
        for c in m["ctr_features"]:
            types.add(c["base"]["ctr_type"])
            float_splits += len(c["base"]["float_splits"])
            one_hot_splits += len(c["base"]["one_hot_splits"])
            wide += sum(int(np.searchsorted(borders[f], b)) >= 254 for f, b in c["base"]["float_splits"])
        for t in m["ctr_tables"]:
            if t["base"]["ctr_type"] in (0, 1):
                classes.add((t["base"]["ctr_type"], t["target_classes_count"]))
    assert types == set(range(6)) and float_splits > 10 and one_hot_splits > 5 and wide > 0
    assert {(0, 2), (0, 3), (0, 5)} <= classes and len([c for c in classes if c[0] == 1]) >= 2


def test_python_cbm_writer_round_trips_the_fixtures(golden_dir):
    """tests/cbm_writer.py writes what oracle/cbm_reader.py reads, on every fixture of the reference."""
    def same(a, b):
        if isinstance(a, dict):
            assert a.keys() == b.keys()
            for k in a:
                same(a[k], b[k])
        elif isinstance(a, (list, tuple)):
            assert len(a) == len(b)
            for x, y in zip(a, b):
                same(x, y)
        elif isinstance(a, np.ndarray):
            assert a.dtype == b.dtype and a.shape == b.shape and a.tobytes() == b.tobytes()
        else:
            assert a == b

    names = ["numeric_only_model.cbm", "rust_tmp_model.cbm", "iris_model.cbm", "boston_housing_model.cbm"]
    for name in names + rm.CTR_FIXTURES:
        m = read_cbm_file(os.path.join(golden_dir, name))
        again = read_cbm(cbm_writer.write_cbm(m))
        m.pop("repacked_bins_in_file")
        again.pop("repacked_bins_in_file")
        same(m, again)


def test_not_a_model_is_rejected(golden_dir):
    with open(os.path.join(golden_dir, "not_a_model.cbm"), "rb") as f:
        with pytest.raises(ValueError):
            read_cbm(f.read())


# ---------------------------------------------------------------------------- invariants ----

def _random_oblivious(rng, n_float=7, n_cat=2, trees=20, max_depth=6, dim=1, many_borders=False,
                      nan_modes=True, scale=1.0, bias=None):
    ffs = []
    flat = 0
    cfs = []
    layout = ["f"] * n_float + ["c"] * n_cat
    rng.shuffle(layout)
    fi = ci = 0
    for kind in layout:
        if kind == "f":
            ffs.append(mb.float_feature(fi, flat, has_nans=bool(rng.integers(0, 2)) if nan_modes else False,
                                        nan_treatment=int(rng.integers(0, 3)) if nan_modes else 0))
            fi += 1
        else:
            cfs.append(mb.cat_feature(ci, flat))
            ci += 1
        flat += 1
    cands = {}
    for f in ffs:
        k = 300 if (many_borders and f["index"] == 0) else int(rng.integers(1, 40))
        cands[f["index"]] = np.unique(rng.normal(size=k).astype(np.float32))
    cat_values = {c["index"]: [integer_cat_feature_hash(v) for v in range(int(rng.integers(2, 11)))] for c in cfs}
    tree_list = []
    for _ in range(trees):
        depth = int(rng.integers(1, max_depth + 1))
        splits = []
        for _ in range(depth):
            if cfs and rng.random() < 0.25:
                c = int(rng.integers(0, len(cfs)))
                splits.append(("onehot", c, int(rng.choice(cat_values[c]))))
            else:
                f = int(rng.integers(0, len(ffs)))
                splits.append(("float", f, float(rng.choice(cands[f]))))
        tree_list.append((splits, rng.normal(size=(1 << depth) * dim)))
    if many_borders:
        # force every candidate border of feature 0 into the model
        for b in cands[0]:
            tree_list.append(([("float", 0, float(b))], rng.normal(size=2 * dim)))
    return mb.build_oblivious(ffs, cfs, dim, tree_list, scale=scale, bias=bias), cat_values


def _random_flat_data(rng, model, cat_values, n):
    width = max([f["flat_index"] for f in model["float_features"]] + [c["flat_index"] for c in model["cat_features"]]) + 1
    x = rng.normal(size=(n, width)).astype(np.float32)
    x[rng.random(size=x.shape) < 0.1] = np.nan
    x[rng.random(size=x.shape) < 0.02] = np.inf
    x[rng.random(size=x.shape) < 0.02] = -np.inf
    for c in model["cat_features"]:
        vals = np.asarray(cat_values[c["index"]] + [12345], dtype=np.int32)
        x[:, c["flat_index"]] = rng.choice(vals, size=n).view(np.float32)
    return x


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("dim", [1, 3])
def test_block_path_equals_bruteforce_on_random_models(seed, dim):
    """The repacked-bin / bucket path and the raw-split brute force share no table: a wrong
    bucket split, XorMask, NaN gate or bit order fails here. Includes a >254-border feature
    together with one-hot splits and all three NaN treatments."""
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, dim=dim, many_borders=True, scale=0.5 if seed else 1.0,
                                          bias=rng.normal(size=dim) if seed else None)
    o = OracleModel(model)
    x = _random_flat_data(rng, model, cat_values, 300)
    pred = o.calc(x)
    bf, bf_idx = o.bruteforce(x)
    np.testing.assert_array_equal(o.leaf_indexes(x), bf_idx)
    np.testing.assert_allclose(pred, bf, rtol=1e-13, atol=1e-13)
    # the same model as a non-symmetric one gives identical answers (model.cpp:634-674; the
    # reference asserts this in every unit test)
    oa = OracleModel(mb.convert_oblivious_to_asymmetric(model))
    np.testing.assert_array_equal(oa.leaf_indexes(x), bf_idx)
    np.testing.assert_array_equal(oa.calc(x), pred)
    # threads do not change anything
    np.testing.assert_array_equal(o.calc(x, threads=3), pred)


def test_binarize_equals_searchsorted_and_nan_table():
    """bin == number of borders strictly below the value == numpy.searchsorted(borders, v, 'left')
    for sorted borders; NaN / +-inf by table (quantization.h:375-409)."""
    rng = np.random.default_rng(5)
    borders = np.unique(rng.normal(size=200).astype(np.float32))
    ffs = []
    for i, (has_nans, treatment) in enumerate([(False, 0), (True, 0), (True, 1), (True, 2), (False, 1), (False, 2)]):
        f = mb.float_feature(i, has_nans=has_nans, nan_treatment=treatment)
        ffs.append(f)
    trees = [([("float", i, float(b))], [0.0, 1.0]) for i in range(len(ffs)) for b in borders]
    model = mb.build_oblivious(ffs, [], 1, trees)
    o = OracleModel(model)
    assert o.bucket_count == len(ffs)
    v = np.concatenate([rng.normal(size=500).astype(np.float32), borders[:50],
                        np.array([np.nan, np.inf, -np.inf, 0.0, -0.0], np.float32)])
    x = np.repeat(v[:, None], len(ffs), axis=1)
    bins = o.binarize_doc_major(x)
    finite = ~np.isnan(v)
    expected = np.searchsorted(borders, v[finite], side="left")
    for i in range(len(ffs)):
        np.testing.assert_array_equal(bins[finite, i], expected)
    nan_row = bins[np.isnan(v)][0]
    # only HasNans && AsTrue turns NaN into +inf (all borders below); everything else gives 0
    assert nan_row.tolist() == [0, 0, 0, len(borders), 0, 0]
    assert bins[np.isposinf(v)][0].tolist() == [len(borders)] * len(ffs)
    assert bins[np.isneginf(v)][0].tolist() == [0] * len(ffs)


def test_one_hot_xor_mask_worked_example():
    """value id 2 of a cat feature => SplitIdx 0xff, XorMask ~3 & 0xff = 0xfc (model.cpp:567-572)."""
    cfs = [mb.cat_feature(0, 0)]
    values = sorted(integer_cat_feature_hash(v) for v in range(4))
    trees = [([("onehot", 0, v)], [0.0, float(i + 1)]) for i, v in enumerate(values)]
    model = mb.build_oblivious([], cfs, 1, trees)
    o = OracleModel(model)
    feat, xor, split = o.repacked_bins()
    assert list(split) == [0xff] * 4 and list(xor) == [0xfe, 0xfd, 0xfc, 0xfb] and list(feat) == [0] * 4
    x = np.asarray(values + [777], np.int32).view(np.float32).reshape(-1, 1)
    np.testing.assert_array_equal(o.binarize_doc_major(x).ravel(), [1, 2, 3, 4, 0])
    np.testing.assert_array_equal(o.calc(x), [1.0, 2.0, 3.0, 4.0, 0.0])


def test_last_block_is_packed_with_its_own_doc_count():
    # quantization.h:357-365: blocks of 128 docs, the tail block uses stride = its doc count
    model = rm.simple_float_model()
    o = OracleModel(model)
    rng = np.random.default_rng(0)
    x = rng.normal(scale=100, size=(130, 3)).astype(np.float32)
    raw = o.binarize(x)
    assert raw.size == 130 * 4
    first = raw[:128 * 4].reshape(4, 128)
    tail = raw[128 * 4:].reshape(4, 2)
    dm = o.binarize_doc_major(x)
    np.testing.assert_array_equal(first.T, dm[:128])
    np.testing.assert_array_equal(tail.T, dm[128:])


# --------------------------------------------------------------- prediction types ----

def test_fast_exp_matches_reference_fmath(golden_dir):
    """The exponent restatement against the reference's own fmath::expd_v (built from the reference
    tree by oracle/build_ref.sh; vectors by tests/golden/make_fmath_vectors.py): bit for bit,
    for every run length the result processor uses, clamps, infinities and NaN included."""
    from oracle.oracle import fast_exp

    g = np.load(os.path.join(golden_dir, "fmath_exp_vectors.npz"))
    x = g["x"]
    for chunk in (1, 3, 4, 10, 128):
        np.testing.assert_array_equal(fast_exp(x, chunk).view(np.uint64), g["chunk_%d" % chunk].view(np.uint64))


def test_fast_exp_is_an_exponent():
    """Independent of the vectors: a relative error of a few 1e-16 against libm over the range
    raw formula values live in, exact at 0, monotone."""
    from oracle.oracle import fast_exp

    x = np.linspace(-50.0, 50.0, 200001)
    y = fast_exp(x)
    assert np.max(np.abs(y / np.exp(x) - 1.0)) < 1e-14
    assert fast_exp([0.0, 0.0, 0.0, 0.0, 0.0])[0] == 1.0 and fast_exp([0.0])[0] == 1.0
    assert np.all(np.diff(y) >= 0)


def test_prediction_types_closed_forms():
    """TestFlatCalcMultiValMultiProba (formula_evaluator_ut.cpp:148-165): sigmoid of the raw values
    within 1e-6; softmax sums to one and keeps the order; Class is the arg max / the sign."""
    from oracle.oracle import apply_prediction_type

    raw = np.array([0., 10., 20., 1., 11., 21., 2., 12., 22., 3., 13., 23.])
    np.testing.assert_allclose(apply_prediction_type(raw, 3, "MultiProbability"), 1 / (1 + np.exp(-raw)), atol=1e-6)
    rng = np.random.default_rng(5)
    raw = rng.normal(0, 4, size=(333, 7))
    p = apply_prediction_type(raw, 7, "Probability").reshape(333, 7)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, atol=1e-12)
    np.testing.assert_allclose(p, np.exp(raw - raw.max(axis=1, keepdims=True)) /
                               np.exp(raw - raw.max(axis=1, keepdims=True)).sum(axis=1, keepdims=True), rtol=1e-12)
    np.testing.assert_array_equal(apply_prediction_type(raw, 7, "Class"), raw.argmax(axis=1))
    one = rng.normal(0, 4, size=1000)
    np.testing.assert_allclose(apply_prediction_type(one, 1, "Probability"), 1 / (1 + np.exp(-one)), rtol=1e-12)
    np.testing.assert_allclose(apply_prediction_type(one, 1, "Exponent"), np.exp(one), rtol=1e-12)
    np.testing.assert_array_equal(apply_prediction_type(one, 1, "Class"), one > 0)
    two = rng.normal(0, 1, size=(50, 2))
    u = apply_prediction_type(two, 2, "RMSEWithUncertainty").reshape(50, 2)
    np.testing.assert_array_equal(u[:, 0], two[:, 0])
    np.testing.assert_allclose(u[:, 1], np.exp(2 * two[:, 1]), rtol=1e-12)
