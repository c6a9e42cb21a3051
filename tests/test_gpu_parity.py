"""Parity of the HIP evaluator against the CPU oracle, through the C ABI. Needs an MI355X.

Bar: bins and leaf indexes bit-exact; predictions within 1e-9 relative / 1e-12 absolute.
"""
import ctypes
import os

import numpy as np
import pytest

import catboost_amd as cb
from catboost_amd import synthetic as syn
from oracle import model_builder as mb
from oracle.cbm_reader import read_cbm, read_cbm_file
from oracle.oracle import OracleModel, cat_feature_hash_signed
from tests import ctr_models
from tests import refmodels as rm
from tests.test_oracle import _random_flat_data, _random_oblivious

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-9, 1e-12


def _close(got, expected):
    np.testing.assert_allclose(got, expected, rtol=RTOL, atol=ATOL)


def _gpu_model(model_dict):
    m = cb.ModelCalcer()
    m.load_from_dict(model_dict)
    m.enable_gpu_evaluation(0)
    return m


def _check_flat(model_dict, x, exact=None):
    """bins, leaf indexes and predictions of flat rows against the oracle."""
    o = OracleModel(model_dict)
    g = _gpu_model(model_dict)
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    pred = g.calc_flat(x)
    _close(pred, o.calc(x))
    if exact is not None:
        np.testing.assert_array_equal(pred, np.asarray(exact, np.float64))
    return g, o


# ------------------------------------------------------------ reference unit-test models ----

def test_library_loaded_is_the_in_tree_hip_build():
    lib = cb.load_library()
    assert os.path.samefile(lib._name, cb.library_path())
    assert cb.ModelCalcer().get_supported_evaluator_types() == [1]  # CBA_FET_GPU only


@pytest.mark.both_batch_modes
@pytest.mark.parametrize("asym", [False, True])
def test_simple_float_model(asym):
    model = rm.simple_float_model()
    if asym:
        model = mb.convert_oblivious_to_asymmetric(model)
    _check_flat(model, rm.DATA, exact=np.arange(8.0))


@pytest.mark.both_batch_modes
@pytest.mark.parametrize("asym", [False, True])
def test_scale_bias_two_trees(asym):
    model = rm.simple_float_model(tree_count=2, scale=0.5, bias=[0.125])
    if asym:
        model = mb.convert_oblivious_to_asymmetric(model)
    g, _ = _check_flat(model, rm.DATA, exact=0.5 * 11.0 * np.arange(8.0) + 0.125)
    # staged ranges: bias only with tree 0 (scale_and_bias.cpp:13-24)
    np.testing.assert_array_equal(g.calc_flat(rm.DATA, tree_start=0, tree_end=1), 0.5 * np.arange(8.0) + 0.125)
    np.testing.assert_array_equal(g.calc_flat(rm.DATA, tree_start=1, tree_end=2), 5.0 * np.arange(8.0))
    np.testing.assert_array_equal(g.calc_flat(rm.DATA, tree_start=1, tree_end=1), np.zeros(8))


@pytest.mark.both_batch_modes
@pytest.mark.parametrize("asym", [False, True])
def test_deep_tree(asym):
    model = rm.simple_deep_tree_model(9)
    if asym:
        model = mb.convert_oblivious_to_asymmetric(model)
    g, _ = _check_flat(model, rm.deep_tree_data(9), exact=np.arange(512.0))
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(rm.deep_tree_data(9)).ravel(), np.arange(512))


@pytest.mark.both_batch_modes
@pytest.mark.parametrize("asym", [False, True])
def test_multi_value_model(asym):
    model = rm.multi_value_float_model()
    if asym:
        model = mb.convert_oblivious_to_asymmetric(model)
    g, _ = _check_flat(model, rm.DATA[:4], exact=[0., 10., 20., 1., 11., 21., 2., 12., 22., 3., 13., 23.])
    np.testing.assert_array_equal(g.predict_specific_class_flat(rm.DATA[:4], 1), [10., 11., 12., 13.])


@pytest.mark.both_batch_modes
def test_simple_asymmetric_model():
    g, _ = _check_flat(rm.simple_asymmetric_model(), rm.DATA, exact=rm.ASYMMETRIC_PREDICTIONS)
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(rm.DATA), rm.ASYMMETRIC_LEAF_INDEXES)
    # built by the library's own non-symmetric builder and reloaded from its .cbm
    ffs, heads = rm.simple_asymmetric_trees()
    b = cb.ModelCalcer()
    b.build_non_symmetric(ffs, [], 1, heads)
    r = cb.ModelCalcer(buffer=b.save_to_buffer())
    np.testing.assert_array_equal(r.calc_flat(rm.DATA), rm.ASYMMETRIC_PREDICTIONS)


@pytest.mark.parametrize("seed,n_float,n_cat,trees,max_depth,docs", [
    (1, 20, 6, 90, 8, 3000), (2, 150, 3, 40, 9, 1000), (3, 4, 10, 25, 6, 257), (4, 30, 2, 300, 5, 5000),
])
def test_non_symmetric_models_with_one_hot_splits(seed, n_float, n_cat, trees, max_depth, docs):
    """One-dimensional non-symmetric models with one-hot splits walk out of LDS like float-only ones: the tables
    of that kernel hold a one-hot split (bin == v) as two tests, bin >= v and behind it bin >= v + 1, with the
    left side's entry repeated. Bins and leaf indexes equal the oracle's, predictions within the tolerance
    (partial sums per wave)."""
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth,
                                          scale=0.5, bias=rng.normal(size=1))
    model = mb.convert_oblivious_to_asymmetric(model)
    assert any(len(f["values"]) for f in model["one_hot_features"]), "the model needs one-hot splits"
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = _gpu_model(model)
    assert "EvalNonSymmetricLdsKernel" in g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)["evaluate"]
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    _close(g.calc_flat(x), o.calc(x))


@pytest.mark.parametrize("seed,dim,n_float,n_cat,trees,max_depth,docs", [
    (1, 2, 30, 0, 120, 8, 3000), (2, 3, 150, 3, 60, 9, 1000), (3, 4, 8, 4, 25, 6, 257), (4, 5, 40, 0, 200, 5, 5000),
    (5, 10, 60, 2, 90, 7, 2049), (6, 13, 12, 0, 33, 10, 64),
])
def test_non_symmetric_models_of_several_dimensions(seed, dim, n_float, n_cat, trees, max_depth, docs):
    """Non-symmetric models of several dimensions walk out of LDS as well: a workgroup sums two or four
    dimensions (a slice), the model's slices are rows of the grid. Two dimensions, one slice with a dimension
    to spare, and several slices the last of which is short; with and without one-hot splits."""
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth, dim=dim,
                                          scale=-0.5, bias=rng.normal(size=dim))
    model = mb.convert_oblivious_to_asymmetric(model)
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = _gpu_model(model)
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    assert "EvalNonSymmetricLdsKernel" in kernels["evaluate"] and kernels["evaluate"].endswith(", %d>" % (2 if dim == 2 else 4))
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    _close(g.calc_flat(x), o.calc(x))
    # most of the trees: the same kernel adds only the values of the range's trees; a few trees: the kernel that
    # walks those alone; no bias unless the range starts at tree 0
    for begin, end in ((1, trees - 1), (0, trees - 2), (trees // 2, trees // 2 + max(1, trees // 10)), (0, 2)):
        _close(g.calc_flat(x, tree_start=begin, tree_end=end), o.calc(x, tree_start=begin, tree_end=end))


def test_non_symmetric_tree_whose_nodes_share_children():
    """A chain of 60 nodes in which both steps of every node lead to the next one passes the loader's
    range checks; unfolded level by level it would have 2^60 entries. The level-order tables give up
    on it and the model runs on the kernel that follows the step nodes, like the reference."""
    depth = 60
    head = mb.leaf_node(float(depth))
    for level in reversed(range(depth)):
        head = mb.split_node(("float", level % 3, 0.5), mb.leaf_node(float(level)), head)
    model = mb.build_non_symmetric([mb.float_feature(i) for i in range(3)], [], 1, [head])
    steps = np.array(model["step_nodes"])
    chain = (steps == [0, 1]).all(axis=1)
    assert chain.sum() == depth - 1
    steps[chain] = [1, 1]
    model["step_nodes"] = steps
    _, o = _check_flat(model, rm.DATA)
    assert set(o.calc(rm.DATA)) == {depth - 1.0, float(depth)}


def test_zero_trees_gives_bias():
    g = _gpu_model(rm.simple_float_model(tree_count=0, bias=[0.75]))
    np.testing.assert_array_equal(g.calc_flat(rm.DATA), np.full(8, 0.75))


def test_zero_trees_ignore_the_prediction_type():
    """The reference fills the results with the bias and returns before TEvalResultProcessor runs
    (cpu/formula_evaluator.cpp:29-41): Probability, Exponent and Class of a model without trees are the raw bias."""
    g = _gpu_model(rm.simple_float_model(tree_count=0, bias=[0.75]))
    for kind in ("Probability", "Exponent", "Class", "RawFormulaVal"):
        g.set_prediction_type(kind)
        np.testing.assert_array_equal(g.calc_flat(rm.DATA), np.full(8, 0.75))
        np.testing.assert_array_equal(g.calc_flat_transposed(np.ascontiguousarray(rm.DATA.T)), np.full(8, 0.75))


def test_single_document_and_ragged_sizes():
    model = rm.simple_float_model(tree_count=2)
    o = OracleModel(model)
    g = _gpu_model(model)
    rng = np.random.default_rng(3)
    for n in (1, 2, 63, 64, 65, 127, 128, 129, 255, 256, 257, 1000):
        x = rng.normal(scale=150, size=(n, 3)).astype(np.float32)
        np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
        np.testing.assert_array_equal(g.calc_flat(x), o.calc(x))
        np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    assert g.calc_flat(np.zeros((0, 3), np.float32)).size == 0


def test_empty_batches(golden_dir):
    """No documents: every entry point returns without touching the GPU buffers, whatever the model holds
    (CTR features, several dimensions, a prediction type)."""
    import torch

    for name in ("numeric_only_model.cbm", "features_num_cat__dataset_adult.cbm", "iris_model.cbm"):
        g = cb.ModelCalcer(os.path.join(golden_dir, name))
        width = max(g.get_float_feature_indices() + g.get_cat_feature_indices()) + 1
        for kind in ("RawFormulaVal", "Probability", "Class"):
            g.set_prediction_type(kind)
            assert g.calc_flat(np.zeros((0, width), np.float32)).size == 0
            assert g.calc_flat_transposed(np.zeros((width, 0), np.float32)).size == 0
        assert g.quantize_flat(np.zeros((0, width), np.float32)).size == 0
        assert g.calc_leaf_indexes_flat(np.zeros((0, width), np.float32)).size == 0
        ev = g.evaluator()
        guard = torch.full((16,), 7.0, dtype=torch.float64, device="cuda:0")
        torch.cuda.synchronize()
        feats = ev.features(cb.LAYOUT_FLAT_ROWS, guard.data_ptr(), width)
        ev.eval_data(feats, 0, guard.data_ptr())
        ev.quantize(feats, 0, guard.data_ptr())
        ev.eval_quantized(guard.data_ptr(), 0, guard.data_ptr())
        ev.apply_prediction_type(cb.APT_PROBABILITY, 0, guard.data_ptr(), guard.data_ptr())
        ev.synchronize()
        assert bool((guard == 7.0).all())


# ------------------------------------------------------------------- fixtures + goldens ----

@pytest.mark.both_batch_modes
def test_numeric_only_fixture(golden_dir):
    g = cb.ModelCalcer(os.path.join(golden_dir, "numeric_only_model.cbm"))
    g.enable_gpu_evaluation(0)
    _close(g.calc_flat(rm.NUMERIC_ONLY_ROWS), rm.NUMERIC_ONLY_EXPECTED)
    _close(g.calc_flat_transposed(np.ascontiguousarray(rm.NUMERIC_ONLY_ROWS.T)), rm.NUMERIC_ONLY_EXPECTED)
    _close(g.calc_flat(rm.NUMERIC_ONLY_ROWS[0]), rm.NUMERIC_ONLY_EXPECTED[:1])
    _close(g.calc(rm.NUMERIC_ONLY_ROWS, [[] for _ in range(4)]), rm.NUMERIC_ONLY_EXPECTED)
    _close(g.calc_single(rm.NUMERIC_ONLY_ROWS[0], []), rm.NUMERIC_ONLY_EXPECTED[:1])


@pytest.mark.both_batch_modes
def test_json_model_format(golden_dir):
    # the json twin of the numeric-only model (CatBoostModelTest.java:181-200) predicts the binary's goldens
    g = cb.ModelCalcer(os.path.join(golden_dir, "numeric_only_model.json"), model_format="json")
    _close(g.calc_flat(rm.NUMERIC_ONLY_ROWS), rm.NUMERIC_ONLY_EXPECTED)
    rng = np.random.default_rng(8)
    model, cat_values = _random_oblivious(rng, dim=3, trees=40, max_depth=6)
    model = mb.convert_oblivious_to_asymmetric(model)
    x = _random_flat_data(rng, model, cat_values, 700)
    g = cb.ModelCalcer(buffer=rm.model_to_json(model), model_format="json")
    _close(g.calc_flat(x), OracleModel(model).calc(x))


@pytest.mark.both_batch_modes
def test_json_model_format_with_ctr_features(golden_dir):
    """Models with CTR features through the json format: bins and predictions equal the oracle's on what
    the format keeps of the model (tests/test_host_logic.py::json_view_of_ctr_model)."""
    from tests.test_host_logic import json_view_of_ctr_model

    cases = [(read_cbm_file(os.path.join(golden_dir, n)), None) for n in ("mushroom_model.cbm", "jvm_model_with_ctr.cbm",
                                                                          "features_num_cat__dataset_adult.cbm")]
    cases += [ctr_models.random_ctr_model(seed, **kwargs) for seed, kwargs in ctr_models.CASES]
    checked = 0
    for model, known in cases:
        kept = json_view_of_ctr_model(model)
        if kept is None:
            continue
        checked += 1
        g = cb.ModelCalcer(buffer=rm.model_to_json(model), model_format="json")
        o = OracleModel(kept)
        if known is None:
            floats, cats = rm.random_ctr_inputs(model, 1500, 21, rm.known_cat_hashes(model))
        else:
            floats, cats = ctr_models.random_documents(model, known, 1500, 21)
        np.testing.assert_array_equal(g.quantize_hashed(floats, cats), o.binarize(floats, cats, layout="split"))
        _close(g.calc_hashed(floats, cats), o.calc(floats, cats, layout="split"))
    assert checked >= 5


@pytest.mark.both_batch_modes
def test_rust_fixture_with_one_hot_string_cats(golden_dir):
    g = cb.ModelCalcer(os.path.join(golden_dir, "rust_tmp_model.cbm"))
    _close(g.calc(rm.RUST_FLOATS, rm.RUST_CATS), rm.RUST_EXPECTED)
    hashed = np.array([[cb.string_cat_feature_hash(c) for c in row] for row in rm.RUST_CATS], np.int32)
    _close(g.calc_hashed(rm.RUST_FLOATS, hashed), rm.RUST_EXPECTED)
    # flat layout: the hash bit-cast into the categorical slot (flat index 2), floats at 0, 1, 3
    flat = np.zeros((3, 4), np.float32)
    flat[:, [0, 1, 3]] = rm.RUST_FLOATS
    flat[:, 2] = hashed[:, 0].view(np.float32)
    _close(g.calc_flat(flat), rm.RUST_EXPECTED)
    o = OracleModel(read_cbm_file(os.path.join(golden_dir, "rust_tmp_model.cbm")))
    np.testing.assert_array_equal(g.quantize_hashed(rm.RUST_FLOATS, hashed), o.binarize(rm.RUST_FLOATS, hashed, layout="split"))


def _same_bits(got, expected, what):
    """Bit for bit, except that a NaN only has to be a NaN (x86 and the GPU give the NaN they make a
    different sign)."""
    nan = np.isnan(expected)
    np.testing.assert_array_equal(np.isnan(got), nan, err_msg=what)
    np.testing.assert_array_equal(got[~nan].view(np.uint64), expected[~nan].view(np.uint64), err_msg=what)


@pytest.mark.parametrize("dim", [1, 2, 3, 10])
def test_prediction_types_on_the_device(golden_dir, dim):
    """CbHipApplyPredictionTypeDevice against the oracle's TEvalResultProcessor, bit for bit: the inputs of
    the reference exponent's vectors (clamps, infinities, NaN, table boundaries) as raw values, and
    document counts around the 128-document block and the 4-value vector width."""
    import torch

    from oracle.oracle import apply_prediction_type

    rng = np.random.default_rng(dim)
    ev = _gpu_model(_random_oblivious(rng, trees=2, dim=dim)[0]).evaluator()
    pool = np.load(os.path.join(golden_dir, "fmath_exp_vectors.npz"))["x"]
    names = {"RawFormulaVal": cb.APT_RAW_FORMULA_VAL, "Exponent": cb.APT_EXPONENT, "Probability": cb.APT_PROBABILITY,
             "Class": cb.APT_CLASS}
    if dim > 1:
        names["MultiProbability"] = cb.APT_MULTI_PROBABILITY
    if dim == 2:
        names["RMSEWithUncertainty"] = cb.APT_RMSE_WITH_UNCERTAINTY
    for docs in (1, 2, 3, 4, 5, 127, 128, 129, 131, 1000, len(pool) // dim):
        raw = pool[rng.permutation(len(pool))[:docs * dim]].copy()
        if dim > 1 and docs > 4:
            raw[:dim] = raw[0]  # a tie for the first largest
        for name, kind in names.items():
            if name == "Exponent" and dim > 1:
                continue  # several dimensions: the reference leaves the raw values (covered by the raw case)
            expected = apply_prediction_type(raw, dim, name)
            x = torch.from_numpy(raw).to("cuda:0")
            out = torch.full((len(expected),), 777.0, dtype=torch.float64, device="cuda:0")
            torch.cuda.synchronize()
            ev.apply_prediction_type(kind, docs, x.data_ptr(), out.data_ptr())
            ev.synchronize()
            _same_bits(out.cpu().numpy(), expected, "%s dim %d docs %d" % (name, dim, docs))
            if not (name == "Class" and dim > 1):  # in place
                ev.apply_prediction_type(kind, docs, x.data_ptr(), x.data_ptr())
                ev.synchronize()
                _same_bits(x.cpu().numpy()[:len(expected)], expected, "in place")
    with pytest.raises(cb.CatBoostError):
        ev.apply_prediction_type(99, 1, 0, 0)
    if dim == 1:
        with pytest.raises(cb.CatBoostError, match="unsupported prediction type"):
            ev.apply_prediction_type(cb.APT_MULTI_PROBABILITY, 1, 0, 0)


# -------------------------------------------------------- CTR (target statistics) features ----

def _hashed(rows):
    return np.array([[cb.string_cat_feature_hash(c) for c in row] for row in rows], np.int32)


@pytest.mark.both_batch_modes
def test_ctr_goldens_of_the_jvm_tests(golden_dir):
    # CatBoostModelTest.java:457-470, 528-547, 586-601, 720-743; the reference's CUDA evaluator refuses
    # both models (cuda/evaluator.cpp:22-28)
    g = cb.ModelCalcer(os.path.join(golden_dir, "categoric_only_model.cbm"))
    none = np.zeros((3, 0), np.float32)
    _close(g.calc(none, rm.JVM_CATEGORIC_ONLY_CATS), rm.JVM_CATEGORIC_ONLY_EXPECTED)
    _close(g.calc_single(none[0], rm.JVM_CATEGORIC_ONLY_CATS[0]), rm.JVM_CATEGORIC_ONLY_EXPECTED[:1])
    _close(g.calc_hashed(none, _hashed(rm.JVM_CATEGORIC_ONLY_CATS)), rm.JVM_CATEGORIC_ONLY_EXPECTED)
    with pytest.raises(cb.CatBoostError):
        g.calc(none, [row[:2] for row in rm.JVM_CATEGORIC_ONLY_CATS])  # :508-524, too few categorical features
    g = cb.ModelCalcer(os.path.join(golden_dir, "jvm_model_with_ctr.cbm"))
    _close(g.calc(rm.JVM_CTR_FLOATS, rm.JVM_CTR_CATS), rm.JVM_CTR_EXPECTED)
    _close(g.calc_single(rm.JVM_CTR_FLOATS[0], rm.JVM_CTR_CATS[0]), rm.JVM_CTR_EXPECTED[:1])


@pytest.mark.both_batch_modes
def test_ctr_goldens_of_the_rust_and_node_tests(golden_dir):
    g = cb.ModelCalcer(os.path.join(golden_dir, "features_num_cat__dataset_adult.cbm"))
    _close(g.calc(rm.RUST_ADULT_FLOATS, rm.RUST_ADULT_CATS), rm.RUST_ADULT_EXPECTED)
    g = cb.ModelCalcer(os.path.join(golden_dir, "node_adult.cbm"))
    assert ["%.2f" % v for v in g.calc(rm.NODE_ADULT_FLOATS, rm.NODE_ADULT_CATS)] == rm.NODE_ADULT_EXPECTED_2DP


@pytest.mark.both_batch_modes
def test_ctr_mushroom_labels(golden_dir):
    # CatBoostModelEvaluatorTest.cs:101-127
    g = cb.ModelCalcer(os.path.join(golden_dir, "mushroom_model.cbm"))
    labels, rows = rm.mushrooms(golden_dir)
    pred = g.calc(np.zeros((len(rows), 0), np.float32), rows)
    np.testing.assert_array_equal(pred > 0, np.array(labels) == "p")
    o = OracleModel(read_cbm_file(os.path.join(golden_dir, "mushroom_model.cbm")))
    _close(pred, o.calc(np.zeros((len(rows), 0), np.float32), _hashed(rows), layout="split"))


@pytest.mark.parametrize("name", rm.CTR_FIXTURES)
@pytest.mark.parametrize("docs", [1, 257, 5000])
def test_ctr_models_against_the_oracle(golden_dir, name, docs):
    """Random documents (known and unknown categories, floats on and around the borders) through the
    hashed, flat and transposed host entry points: bins bit-exact, predictions within the bar."""
    path = os.path.join(golden_dir, name)
    m = read_cbm_file(path)
    o = OracleModel(m)
    g = cb.ModelCalcer(path)
    floats, cats = rm.random_ctr_inputs(m, docs, 100 + docs, rm.known_cat_hashes(m))
    expected = o.calc(floats, cats, layout="split")
    np.testing.assert_array_equal(g.quantize_hashed(floats, cats), o.binarize(floats, cats, layout="split"))
    _close(g.calc_hashed(floats, cats), expected)
    flat = rm.flat_rows(m, floats, cats)
    np.testing.assert_array_equal(g.quantize_flat(flat), o.binarize(flat))
    _close(g.calc_flat(flat), expected)
    _close(g.calc_flat_transposed(np.ascontiguousarray(flat.T)), expected)
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(flat), o.leaf_indexes(flat))
    half = o.tree_count // 2
    _close(g.calc_flat(flat, tree_start=half, tree_end=o.tree_count),
           o.calc(flat, tree_start=half, tree_end=o.tree_count))


@pytest.mark.parametrize("seed", [seed for seed, _ in ctr_models.CASES])
@pytest.mark.parametrize("tile", ["1", "0"])
def test_synthetic_ctr_models_of_every_kind(golden_dir, monkeypatch, seed, tile):
    """Synthetic models with all six CTR types, tables with up to five target classes and projections
    over categorical features, float splits and one-hot splits (tests/ctr_models.py), through both CTR
    kernels. The CTR buckets of the quantized documents must equal, bit for bit, the bins of the CTR
    values that the reference's own calculator printed for the stored documents; on more documents the
    oracle (which reproduces those values) is the checker."""
    monkeypatch.setenv("CATBOOST_AMD_CTR_TILE", tile)
    path = os.path.join(golden_dir, "synthetic_ctr_%d.cbm" % seed)
    m = read_cbm_file(path)
    o = OracleModel(m)
    g = cb.ModelCalcer(path)
    ref = np.load(os.path.join(golden_dir, "ctr_ref_vectors.npz"))
    floats, cats = ref["floats_%d" % seed], ref["cats_%d" % seed]
    bins = g.quantize_hashed(floats, cats)
    np.testing.assert_array_equal(bins, o.binarize(floats, cats, layout="split"))
    # straight against the reference's values: a CTR bucket holds the count of borders below the value
    # (one bucket per CTR here, none has more than 254 borders)
    doc_major = np.zeros((floats.shape[0], o.bucket_count), np.uint8)
    for start in range(0, floats.shape[0], 128):
        dc = min(128, floats.shape[0] - start)
        doc_major[start:start + dc] = bins[start * o.bucket_count:(start + dc) * o.bucket_count].reshape(-1, dc).T
    first = o.bucket_count - len(m["ctr_features"])
    values, comparable = ref["ctrs_%d" % seed], ref["comparable_%d" % seed]
    for i, c in enumerate(m["ctr_features"]):
        expected = (values[i][:, None] > np.asarray(c["borders"], np.float32)[None, :]).sum(axis=1)
        np.testing.assert_array_equal(doc_major[comparable[i], first + i], expected[comparable[i]])
    _close(g.calc_hashed(floats, cats), o.calc(floats, cats, layout="split"))
    # more documents, ragged tail, every host layout
    model, known = ctr_models.random_ctr_model(seed, **dict(ctr_models.CASES)[seed])
    for docs in (1, 3000):
        floats, cats = ctr_models.random_documents(model, known, docs, 50 + docs)
        expected = o.calc(floats, cats, layout="split")
        np.testing.assert_array_equal(g.quantize_hashed(floats, cats), o.binarize(floats, cats, layout="split"))
        _close(g.calc_hashed(floats, cats), expected)
        flat = rm.flat_rows(m, floats, cats)
        _close(g.calc_flat(flat), expected)
        _close(g.calc_flat_transposed(np.ascontiguousarray(flat.T)), expected)
        np.testing.assert_array_equal(g.calc_leaf_indexes_flat(flat), o.leaf_indexes(flat))


@pytest.mark.both_batch_modes
@pytest.mark.parametrize("name", ["cat", "nocat"])
def test_models_that_the_reference_holds_as_exported_cpp(golden_dir, name):
    """The two models that the reference keeps as exported C++ code (tests/golden/make_export_vectors.py):
    the library's predictions against that code's own applier on the stored documents, bins and leaf
    indexes against the oracle, the split tables the library derives against the exporter's arrays."""
    v = np.load(os.path.join(golden_dir, "cpp_export_vectors.npz"))
    path = os.path.join(golden_dir, "cpp_export_%s.cbm" % name)
    m = read_cbm_file(path)
    o = OracleModel(m)
    g = cb.ModelCalcer(path)
    floats, cats = v["floats_" + name], v["cats_" + name]
    expected, comparable = v["predictions_" + name], v["comparable_" + name]
    got = g.calc_hashed(floats, cats)
    _close(got[comparable], expected[comparable])
    _close(got, o.calc(floats, cats, layout="split"))
    np.testing.assert_array_equal(g.quantize_hashed(floats, cats), o.binarize(floats, cats, layout="split"))
    flat = rm.flat_rows(m, floats, cats)
    _close(g.calc_flat(flat), got)
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(flat), o.leaf_indexes(flat))
    if name == "cat":
        # the strings of the code's own table through the string entry point
        strings = {int(h): str(s) for s, h in zip(v["hash_strings_cat"], v["hash_values_cat"])}
        rows = [i for i in range(200) if all(int(h) in strings for h in cats[i])]
        assert len(rows) > 50
        as_text = [[strings[int(h)] for h in cats[i]] for i in rows]
        _close(g.calc(floats[rows], as_text), got[rows])


def test_synthetic_ctr_model_survives_save_and_load(golden_dir, tmp_path):
    """The library's own writer keeps CTR features of every kind: load, save, load again, same bins."""
    path = os.path.join(golden_dir, "synthetic_ctr_5.cbm")
    ref = np.load(os.path.join(golden_dir, "ctr_ref_vectors.npz"))
    floats, cats = ref["floats_5"], ref["cats_5"]
    g = cb.ModelCalcer(path)
    again = cb.ModelCalcer(buffer=g.save_to_buffer())
    np.testing.assert_array_equal(g.quantize_hashed(floats, cats), again.quantize_hashed(floats, cats))
    np.testing.assert_array_equal(g.calc_hashed(floats, cats), again.calc_hashed(floats, cats))


def test_feature_layout_remaps_positions(golden_dir):
    """TFeatureLayout (evaluation_interface.h:17-69): with a layout installed, a feature at model
    position p is read at list[p] of the caller's data. Documents whose columns are scattered that way
    must give what the unscattered documents give without a layout, bit for bit (same kernels, same
    bins), through flat rows, flat columns, separate float / hashed categorical arrays and strings."""
    rng = np.random.default_rng(42)
    for name in ("synthetic_ctr_2.cbm", "rust_tmp_model.cbm", "features_num__dataset_querywise.cbm"):
        path = os.path.join(golden_dir, name)
        m = read_cbm_file(path)
        o = OracleModel(m)
        g = cb.ModelCalcer(path)
        floats, cats = rm.random_ctr_inputs(m, 700, 3, rm.known_cat_hashes(m))
        flat = rm.flat_rows(m, floats, cats)
        expected = g.calc_flat(flat)
        _close(expected, o.calc(flat))
        expected_bins = g.quantize_flat(flat)
        # flat vectors: scatter into wider rows
        width = flat.shape[1] + 5
        where = rng.permutation(width)[:flat.shape[1]].astype(np.uint32)
        scattered = rng.normal(size=(flat.shape[0], width)).astype(np.float32)
        scattered[:, where] = flat
        g.set_feature_layout(flat_indexes=where)
        used = [f["flat_index"] for f in m["float_features"] if len(f["borders"])] + \
               [c["flat_index"] for c in m["cat_features"] if c.get("used", True)]
        need = int(where[used].max()) + 1
        np.testing.assert_array_equal(g.calc_flat(scattered), expected)
        np.testing.assert_array_equal(g.calc_flat(scattered[:, :need]), expected)
        np.testing.assert_array_equal(g.quantize_flat(scattered), expected_bins)
        np.testing.assert_array_equal(g.calc_flat_transposed(np.ascontiguousarray(scattered.T)), expected)
        with pytest.raises(cb.CatBoostError, match="insufficient"):
            g.calc_flat(scattered[:, :need - 1])
        # separate arrays: scatter the float and the categorical columns on their own
        fw, cw = floats.shape[1] + 3, cats.shape[1] + 2
        fwhere = rng.permutation(fw)[:floats.shape[1]].astype(np.uint32)
        cwhere = rng.permutation(cw)[:cats.shape[1]].astype(np.uint32)
        sf = rng.normal(size=(floats.shape[0], fw)).astype(np.float32)
        sc = rng.integers(-5, 5, size=(cats.shape[0], cw)).astype(np.int32)
        sf[:, fwhere] = floats
        sc[:, cwhere] = cats
        g.set_feature_layout(float_feature_indexes=fwhere, cat_feature_indexes=cwhere)
        np.testing.assert_array_equal(g.calc_hashed(sf, sc), expected)
        np.testing.assert_array_equal(g.calc_flat(flat), expected)  # flat positions untouched by these lists
        # a list without an entry for a used feature is refused and changes nothing
        if floats.shape[1] > 1:
            with pytest.raises(cb.CatBoostError, match="feature layout"):
                g.set_feature_layout(float_feature_indexes=fwhere[:0])
            np.testing.assert_array_equal(g.calc_hashed(sf, sc), expected)
        g.set_feature_layout()
        np.testing.assert_array_equal(g.calc_hashed(floats, cats), expected)
    # strings: the rust fixture's one categorical feature moved to the third of three strings
    g = cb.ModelCalcer(os.path.join(golden_dir, "rust_tmp_model.cbm"))
    g.set_feature_layout(cat_feature_indexes=np.array([2], np.uint32))
    _close(g.calc(rm.RUST_FLOATS, [["x", "y", c[0]] for c in rm.RUST_CATS]), rm.RUST_EXPECTED)


def test_ctr_kernel_without_the_staged_tile(golden_dir, monkeypatch):
    """Models whose projections read more categorical columns than the LDS tile holds take the plain CTR
    kernel; the switch forces it for models that would not."""
    monkeypatch.setenv("CATBOOST_AMD_CTR_TILE", "0")
    for name in ("mushroom_model.cbm", "features_num_cat__dataset_adult.cbm", "cloudness_small.cbm"):
        path = os.path.join(golden_dir, name)
        m = read_cbm_file(path)
        o = OracleModel(m)
        g = cb.ModelCalcer(path)
        floats, cats = rm.random_ctr_inputs(m, 3000, 77, rm.known_cat_hashes(m))
        np.testing.assert_array_equal(g.quantize_hashed(floats, cats), o.binarize(floats, cats, layout="split"))
        flat = rm.flat_rows(m, floats, cats)
        _close(g.calc_flat_transposed(np.ascontiguousarray(flat.T)), o.calc(flat))


def test_ctr_model_on_the_device_path(golden_dir):
    """The device entry points (features already in HBM) on the adult model, 200 000 documents."""
    import torch

    path = os.path.join(golden_dir, "features_num_cat__dataset_adult.cbm")
    m = read_cbm_file(path)
    o = OracleModel(m)
    g = cb.ModelCalcer(path)
    ev = g.evaluator()
    docs = 200_000
    floats, cats = rm.random_ctr_inputs(m, docs, 5, rm.known_cat_hashes(m))
    flat = rm.flat_rows(m, floats, cats)
    x = torch.from_numpy(flat).to("cuda:0")
    f = torch.from_numpy(floats).to("cuda:0")
    c = torch.from_numpy(cats).to("cuda:0")
    out = torch.zeros(docs, dtype=torch.float64, device="cuda:0")
    out2 = torch.zeros_like(out)
    bins = torch.zeros(ev.quantized_bytes(docs), dtype=torch.uint8, device="cuda:0")
    exported = torch.zeros(docs * ev.bucket_count, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]), docs, out.data_ptr())
    split = ev.features(cb.LAYOUT_SPLIT_ROWS, f.data_ptr(), f.shape[1], c.data_ptr(), c.shape[1])
    ev.quantize(split, docs, bins.data_ptr())
    ev.eval_quantized(bins.data_ptr(), docs, out2.data_ptr())
    ev.export_quantized(bins.data_ptr(), docs, exported.data_ptr())
    ev.synchronize()
    assert torch.equal(out, out2)
    _close(out.cpu().numpy(), o.calc(flat, threads=8))
    np.testing.assert_array_equal(exported.cpu().numpy(), o.binarize(flat))


def test_device_entry_points_in_a_hip_graph(golden_dir):
    """CbHipQuantize, CbHipEvalQuantized, CbHipLeafIndexesQuantized and CbHipApplyPredictionTypeDevice only
    launch kernels on the caller's stream (no allocation, no synchronisation, no memset), so a caller may
    capture them into a HIP graph. Every replay, with new documents in the captured input buffer and eager
    work in between, must equal the eager one-call path bit for bit."""
    import torch

    cases = []
    for cfg, docs in (("C1", 10_000), ("C3", 3000), ("C4", 3000), ("C5", 2000)):
        model, info = syn.build_model(cfg, trees=100)
        cases.append((cfg, model, syn.device_features(info, docs), None, info["dim"]))
    path = os.path.join(golden_dir, "features_num_cat__dataset_adult.cbm")
    m = read_cbm_file(path)
    floats, cats = rm.random_ctr_inputs(m, 5000, 9, rm.known_cat_hashes(m))
    cases.append(("adult", cb.ModelCalcer(path), torch.from_numpy(floats).to("cuda:0"),
                  torch.from_numpy(cats).to("cuda:0"), 1))
    no_splits = cb.ModelCalcer()
    no_splits.build_oblivious([dict(index=0, flat_index=0)], [], 1, [([], [0.25]), ([], [0.5])], bias=[1.0])
    cases.append(("no splits", no_splits, torch.zeros(1000, 1, device="cuda:0"), None, 1))
    for name, model, x, c, dim in cases:
        model.enable_gpu_evaluation(0)
        ev = model.evaluator()
        docs = x.shape[0]
        static_x = x.clone()
        static_c = c.clone() if c is not None else None
        bins = torch.zeros(ev.quantized_bytes(docs), dtype=torch.uint8, device="cuda:0")
        out = torch.zeros(docs * dim, dtype=torch.float64, device="cuda:0")
        proba = torch.zeros_like(out)
        leaves = torch.zeros(docs * ev.tree_count, dtype=torch.int32, device="cuda:0")

        def features(a, b):
            if b is None:
                return ev.features(cb.LAYOUT_FLAT_ROWS, a.data_ptr(), a.shape[1])
            return ev.features(cb.LAYOUT_SPLIT_ROWS, a.data_ptr(), a.shape[1], b.data_ptr(), b.shape[1])

        prediction = cb.APT_PROBABILITY if dim == 1 else cb.APT_MULTI_PROBABILITY

        def run(stream):
            ev.quantize(features(static_x, static_c), docs, bins.data_ptr(), stream=stream)
            ev.eval_quantized(bins.data_ptr(), docs, out.data_ptr(), stream=stream)
            ev.leaf_indexes_quantized(bins.data_ptr(), docs, leaves.data_ptr(), stream=stream)
            ev.apply_prediction_type(prediction, docs, out.data_ptr(), proba.data_ptr(), stream=stream)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            run(side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run(torch.cuda.current_stream().cuda_stream)
        eager = torch.zeros_like(out)
        eager_proba = torch.zeros_like(out)
        eager_bins = torch.zeros_like(bins)
        eager_leaves = torch.zeros_like(leaves)
        for replay in range(3):
            order = torch.randperm(docs, device="cuda:0")
            static_x.copy_(x[order])
            if c is not None:
                static_c.copy_(c[order])
            out.zero_()
            proba.zero_()
            leaves.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            # eager, through the one-call entry point and separate buffers
            xe = x[order].contiguous()
            ce = c[order].contiguous() if c is not None else None
            ev.eval_data(features(xe, ce), docs, eager.data_ptr())
            ev.quantize(features(xe, ce), docs, eager_bins.data_ptr())
            ev.leaf_indexes_quantized(eager_bins.data_ptr(), docs, eager_leaves.data_ptr())
            ev.apply_prediction_type(prediction, docs, eager.data_ptr(), eager_proba.data_ptr())
            ev.synchronize()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), (name, replay)
            assert torch.equal(leaves, eager_leaves), (name, replay)
            assert torch.equal(proba, eager_proba), (name, replay)
        if name == "no splits":
            assert torch.equal(out, torch.full_like(out, 1.75))


@pytest.mark.both_batch_modes
def test_querywise_fixture(golden_dir):
    g = cb.ModelCalcer(os.path.join(golden_dir, "features_num__dataset_querywise.cbm"))
    np.testing.assert_allclose(g.calc_flat(rm.querywise_rows()), rm.QUERYWISE_EXPECTED, rtol=1e-12, atol=1e-15)


@pytest.mark.both_batch_modes
def test_iris_fixture(golden_dir):
    path = os.path.join(golden_dir, "iris_model.cbm")
    g = cb.ModelCalcer(path)
    feats, labels = rm.load_iris(golden_dir)
    pred = g.calc_flat(feats).reshape(-1, 3)
    np.testing.assert_array_equal(np.argmax(pred, axis=1), labels)
    o = OracleModel(read_cbm_file(path))
    _close(pred.ravel(), o.calc(feats))
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(feats), o.leaf_indexes(feats))
    np.testing.assert_array_equal(g.quantize_flat(feats), o.binarize(feats))
    g.set_prediction_type("Class")
    np.testing.assert_array_equal(g.calc_flat(feats), labels.astype(np.float64))
    # the other prediction types of a multi-class model: the oracle's result processor on the
    # library's own raw values, bit for bit
    from oracle.oracle import apply_prediction_type
    for name in ("Probability", "MultiProbability"):
        g.set_prediction_type(name)
        np.testing.assert_array_equal(g.calc_flat(feats), apply_prediction_type(pred.ravel(), 3, name))
    g.set_prediction_type("Probability")
    np.testing.assert_allclose(g.calc_flat(feats).reshape(-1, 3).sum(axis=1), 1.0, atol=1e-12)


@pytest.mark.both_batch_modes
@pytest.mark.parametrize("name", ["all", "missed"])
def test_multiclass_probabilities_of_the_reference_canondata(golden_dir, name):
    """The multi-class model and the 17-digit probability table of the reference's own
    test_multiclass_classes_count: the library's Probability predictions, host and device post-processing."""
    from tests.test_oracle import multiclass_classes_count_case
    path, features, expected = multiclass_classes_count_case(golden_dir, name)
    g = cb.ModelCalcer(path)
    g.set_prediction_type("Probability")
    got = g.calc_flat(features).reshape(100, -1)
    np.testing.assert_allclose(got, expected, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(g.calc_flat_transposed(np.ascontiguousarray(features.T)).reshape(100, -1), expected,
                               rtol=1e-9, atol=1e-12)
    g.set_prediction_type("Class")
    # classes from the raw values (documents with equal stored probabilities may differ in the raw ones)
    raw = OracleModel(read_cbm_file(path)).calc(features).reshape(100, -1)
    np.testing.assert_array_equal(g.calc_flat(features), np.argmax(raw, axis=1).astype(np.float64))
    # on the device: raw values, then the prediction type applied in place by the library's kernel
    import torch
    ev = g.evaluator()
    dim = expected.shape[1]
    x = torch.from_numpy(features).cuda()
    out = torch.zeros(100 * dim, dtype=torch.float64, device="cuda")
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]), 100, out.data_ptr())
    ev.apply_prediction_type(cb.APT_PROBABILITY, 100, out.data_ptr(), out.data_ptr())
    ev.synchronize()
    np.testing.assert_allclose(out.cpu().numpy().reshape(100, dim), expected, rtol=1e-9, atol=1e-12)


@pytest.mark.both_batch_modes
def test_model_of_the_backward_compatibility_test(golden_dir):
    """The old-version three-class model of the reference's test_multiclass_model_backward_compatibility and
    the canonical outputs of `catboost calc` for it (10 digits), through the library."""
    v = np.load(os.path.join(golden_dir, "cloudness_backward_compatibility.npz"))
    g = cb.ModelCalcer(os.path.join(golden_dir, "cloudness_backward_compatibility.cbm"))
    for kind in ("RawFormulaVal", "Probability", "Class"):
        g.set_prediction_type(kind)
        np.testing.assert_allclose(g.calc_flat(v["features"]), v[kind].ravel(), rtol=6e-10, atol=0)


@pytest.mark.both_batch_modes
def test_prediction_types_of_the_reference_unit_test():
    """TestFlatCalcMultiValMultiProba (formula_evaluator_ut.cpp:148-165) through the C API, and the
    one-dimensional types on the two-tree model with scale and bias."""
    from oracle.oracle import apply_prediction_type
    g = _gpu_model(rm.multi_value_float_model())
    raw = np.array([0., 10., 20., 1., 11., 21., 2., 12., 22., 3., 13., 23.])
    g.set_prediction_type("MultiProbability")
    probs = g.calc_flat(rm.DATA[:4])
    np.testing.assert_allclose(probs, 1 / (1 + np.exp(-raw)), atol=1e-6)
    np.testing.assert_array_equal(probs, apply_prediction_type(raw, 3, "MultiProbability"))
    rng = np.random.default_rng(12)
    model, cat_values = _random_oblivious(rng, dim=1, trees=30, max_depth=6, scale=0.5, bias=[0.25])
    x = _random_flat_data(rng, model, cat_values, 1000)
    g = _gpu_model(model)
    raw = g.calc_flat(x)
    for name in ("Probability", "Exponent", "Class"):
        g.set_prediction_type(name)
        np.testing.assert_array_equal(g.calc_flat(x), apply_prediction_type(raw, 1, name))
    g.set_prediction_type("Probability")
    np.testing.assert_allclose(g.calc_flat(x), 1 / (1 + np.exp(-raw)), rtol=1e-12)


@pytest.mark.both_batch_modes
def test_boston_fixture(golden_dir):
    path = os.path.join(golden_dir, "boston_housing_model.cbm")
    g = cb.ModelCalcer(path)
    feats, target = rm.load_boston(golden_dir)
    pred = g.calc_flat(feats)
    assert int(np.sum(np.abs(pred - np.log(target)) >= 0.4)) <= 7
    _close(pred, OracleModel(read_cbm_file(path)).calc(feats))


# ------------------------------------------------------------------------- random models ----

@pytest.mark.parametrize("seed", [0, 1, 2, 3])
@pytest.mark.parametrize("dim", [1, 3, 10, 20])
def test_random_oblivious_models(seed, dim):
    rng = np.random.default_rng(100 * dim + seed)
    model, cat_values = _random_oblivious(rng, dim=dim, trees=40, max_depth=8, many_borders=(seed % 2 == 0),
                                          scale=0.5 if seed else 1.0, bias=rng.normal(size=dim) if seed else None)
    x = _random_flat_data(rng, model, cat_values, 777)
    g, o = _check_flat(model, x)
    # one-hot splits and features with more than 127 borders: the mixed register-resident kernels,
    # which add in tree order like the CPU evaluator
    np.testing.assert_array_equal(g.calc_flat(x), o.calc(x))
    # the same model as a non-symmetric one
    _check_flat(mb.convert_oblivious_to_asymmetric(model), x)
    # transposed input and a tree sub-range
    _close(g.calc_flat_transposed(np.ascontiguousarray(x.T)), o.calc(x))
    _close(g.calc_flat(x, tree_start=3, tree_end=17), o.calc(x, tree_start=3, tree_end=17))
    # split float / hashed categorical rows
    ff, cf = model["float_features"], model["cat_features"]
    floats = x[:, [f["flat_index"] for f in ff]]
    cats = x[:, [c["flat_index"] for c in cf]].view(np.int32)
    _close(g.calc_hashed(floats, cats), o.calc(floats, cats, layout="split"))


def _float_only_model(rng, n_float, trees, max_depth, scale=1.0, bias=None, dim=1, max_borders=40):
    """Oblivious model over float features only (fewer than `max_borders` borders each), every feature used."""
    ffs = [mb.float_feature(i, i) for i in range(n_float)]
    cands = [np.unique(rng.normal(size=int(rng.integers(1, max_borders))).astype(np.float32)) for _ in range(n_float)]
    tree_list = []
    order = rng.permutation(n_float)
    next_feature = 0
    t = 0
    while t < trees or next_feature < n_float:
        depth = int(rng.integers(1, max_depth + 1))
        splits = []
        for _ in range(depth):
            if next_feature < n_float:
                f = int(order[next_feature])
                next_feature += 1
            else:
                f = int(rng.integers(0, n_float))
            splits.append(("float", f, float(rng.choice(cands[f]))))
        tree_list.append((splits, rng.normal(size=(1 << depth) * dim)))
        t += 1
    return mb.build_oblivious(ffs, [], dim, tree_list, scale=scale, bias=bias)


# Models of this kind (one-dimensional, float features with < 128 borders, depth <= 8, at most
# 224 buckets) run on the register-resident kernels (97 to 208 buckets: on the fused kernel), which add leaf
# values in tree order like the CPU evaluator: their predictions are compared bit for bit. 225 buckets fall back
# to the LDS tile kernel (sums per wave, then across waves), which only meets the tolerance. Models whose features all
# have fewer than 64 borders take the six-bit form of these kernels (two levels share a merge); the
# switch sends them through the 7-bit form as well.
@pytest.mark.parametrize("six", ["1", "0"])
@pytest.mark.parametrize("n_float,trees,max_depth,docs", [
    (1, 1, 1, 1), (1, 1, 8, 255), (3, 15, 8, 256), (5, 16, 8, 257), (7, 17, 6, 2049), (20, 33, 8, 1000),
    (96, 40, 8, 3000), (97, 40, 8, 3000), (208, 70, 8, 5000), (209, 70, 8, 1500), (224, 70, 8, 2000),
    (225, 70, 8, 1500), (50, 200, 4, 70001),
])
def test_register_kernel_shapes(monkeypatch, n_float, trees, max_depth, docs, six):
    monkeypatch.setenv("CATBOOST_AMD_REG_SIX", six)
    rng = np.random.default_rng(1000 * n_float + trees)
    model = _float_only_model(rng, n_float, trees, max_depth, scale=0.75, bias=[0.125])
    x = rng.normal(size=(docs, n_float)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] = np.nan
    o = OracleModel(model)
    g = _gpu_model(model)
    expected = o.calc(x)
    got = g.calc_flat(x)
    if n_float <= 224:
        np.testing.assert_array_equal(got, expected)
    else:
        _close(got, expected)
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
    # a tree sub-range
    if len(model["tree_sizes"]) >= 3:
        _close(g.calc_flat(x, tree_start=1, tree_end=len(model["tree_sizes"]) - 1),
               o.calc(x, tree_start=1, tree_end=len(model["tree_sizes"]) - 1))


@pytest.mark.parametrize("six", ["1", "0"])
@pytest.mark.parametrize("n_float,trees,max_depth,docs,small_batch", [
    (30, 60, 10, 3000, "0"), (96, 37, 9, 700, "0"), (97, 41, 10, 2500, "0"), (208, 45, 10, 1500, "0"),
    (12, 300, 10, 70001, "0"), (12, 300, 10, 900, "1"), (5, 3, 10, 1, "0"),
])
def test_register_kernel_deep_trees(monkeypatch, n_float, trees, max_depth, docs, small_batch, six):
    """One-dimensional float-only models with trees of depth 9 and 10: register-resident kernels with 1024 leaf
    rows per tree (the index of a document is a 16-bit word of two byte-parallel index bytes), bit for bit like
    the shallower ones; small batches in slices of the trees within the tolerance."""
    monkeypatch.setenv("CATBOOST_AMD_REG_SIX", six)
    monkeypatch.setenv("CATBOOST_AMD_SMALL_BATCH", small_batch)
    rng = np.random.default_rng(31 * n_float + trees + max_depth)
    model = _float_only_model(rng, n_float, trees, max_depth, scale=-0.5, bias=[2.0])
    assert max(model["tree_sizes"]) > 8
    x = rng.normal(size=(docs, n_float)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] = np.nan
    o = OracleModel(model)
    g = _gpu_model(model)
    evaluate = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)["evaluate"]
    kernel = evaluate.split(" ")[0]
    assert "_l1024" in kernel and kernel.endswith("_s") == (six == "1"), evaluate
    expected = o.calc(x)
    got = g.calc_flat(x)
    if small_batch == "0":
        np.testing.assert_array_equal(got, expected)
    else:
        assert " slices" in evaluate, evaluate
        _close(got, expected)
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    n = len(model["tree_sizes"])
    for begin, end in ((1, n - 1), (0, n // 2), (n // 2, n), (5, 6)):
        if begin < end <= n:
            np.testing.assert_array_equal(g.calc_flat(x, tree_start=begin, tree_end=end),
                                          o.calc(x, tree_start=begin, tree_end=end), err_msg="trees %d..%d" % (begin, end))


@pytest.mark.parametrize("six", ["1", "0"])
@pytest.mark.parametrize("dim,max_depth,n_float,trees,docs", [
    (2, 6, 10, 20, 1000), (3, 6, 30, 33, 3000), (5, 8, 12, 9, 700), (6, 6, 128, 50, 2500), (7, 8, 100, 21, 1300),
    (10, 6, 100, 100, 5000), (13, 8, 60, 18, 900), (20, 6, 40, 30, 2049), (4, 6, 160, 60, 600), (2, 8, 192, 70, 600),
])
def test_register_kernel_multi_dimensional(monkeypatch, dim, max_depth, n_float, trees, docs, six):
    """Multi-dimensional float-only models: several launches of a register-resident kernel, each
    adding its dimensions in tree order like the CPU evaluator, hence bit for bit."""
    monkeypatch.setenv("CATBOOST_AMD_REG_SIX", six)
    rng = np.random.default_rng(77 * dim + trees)
    model = _float_only_model(rng, n_float, trees, max_depth, scale=1.25, bias=list(rng.normal(size=dim)), dim=dim)
    x = rng.normal(size=(docs, n_float)).astype(np.float32)
    o = OracleModel(model)
    g = _gpu_model(model)
    np.testing.assert_array_equal(g.calc_flat(x), o.calc(x))
    _close(g.calc_flat(x, tree_start=1, tree_end=len(model["tree_sizes"])),
           o.calc(x, tree_start=1, tree_end=len(model["tree_sizes"])))
    # the last launch takes the narrowest kernel that holds the dimensions left over
    evaluate = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, 1 << 20)["evaluate"]
    expected_tail = {10: "_p4_", 13: "_p2_", 20: "_p2_"}.get(dim)
    if expected_tail:
        assert "_p6_" in evaluate.split(" + ")[0] and expected_tail in evaluate.split(" + ")[1], evaluate
    else:
        assert " + " not in evaluate, evaluate


@pytest.mark.parametrize("max_borders", [64, 65, 128])
def test_register_kernel_border_counts(max_borders):
    """Features with exactly 63 borders still take the six-bit form, one feature with 64 or more sends
    the model to the 7-bit form (127 is its limit): bit for bit either way."""
    rng = np.random.default_rng(max_borders)
    model = _float_only_model(rng, 24, 60, 8, scale=1.5, bias=[-0.25], max_borders=max_borders)
    # one feature with every border the form allows, all of them used by some tree
    full = np.unique(rng.normal(size=4 * max_borders).astype(np.float32))[:max_borders - 1]
    ffs = [mb.float_feature(i, i) for i in range(25)]
    trees = [([("float", 24, float(b)), ("float", int(rng.integers(0, 24)), 0.0)], rng.normal(size=4)) for b in full]
    extra = mb.build_oblivious(ffs, [], 1, trees)
    assert max(len(f["borders"]) for f in extra["float_features"]) == max_borders - 1
    x = rng.normal(size=(3000, 25)).astype(np.float32)
    x[:1000, 24] = rng.choice(full, size=1000)  # on the borders
    for m in (model, extra):
        xx = x[:, :len(m["float_features"])]
        np.testing.assert_array_equal(_gpu_model(m).calc_flat(xx), OracleModel(m).calc(xx))
        np.testing.assert_array_equal(_gpu_model(m).quantize_flat(xx), OracleModel(m).binarize(xx))


@pytest.mark.parametrize("split", ["1", "0"])
@pytest.mark.parametrize("borders,n_float,dim,depth", [(128, 6, 1, 8), (200, 20, 1, 8), (254, 3, 1, 6), (254, 40, 3, 6),
                                                       (300, 10, 1, 10)])
def test_register_kernel_buckets_of_many_values(monkeypatch, split, borders, n_float, dim, depth):
    """Float features with 128 and more used borders (values on the borders included, around the 127th above
    all): a bucket of more than 127 values takes two bins registers, min(bin, 127) and max(bin - 127, 0), and the
    model keeps the 7-bit compare; with the switch off it takes the 8-bit one of the mixed kernels. Bit for bit
    either way (trees of depth 10 have no mixed kernel: those go to the tile kernel for deep trees, whose waves
    add partial sums: within the tolerance)."""
    monkeypatch.setenv("CATBOOST_AMD_REG_SPLIT", split)
    rng = np.random.default_rng(borders + n_float)
    ffs = [mb.float_feature(i, i) for i in range(n_float)]
    cands = [np.unique(rng.normal(size=4 * borders).astype(np.float32))[:borders] for _ in range(n_float)]
    trees = []
    for f in range(n_float):  # every border of every feature is used by some tree
        for start in range(0, borders, depth):
            splits = [("float", f, float(b)) for b in cands[f][start:start + depth]]
            trees.append((splits, rng.normal(size=(1 << len(splits)) * dim)))
    model = mb.build_oblivious(ffs, [], dim, trees, scale=0.5, bias=list(rng.normal(size=dim)))
    assert max(len(f["borders"]) for f in model["float_features"]) == borders
    x = rng.normal(size=(2500, n_float)).astype(np.float32)
    for f in range(n_float):
        x[:600, f] = rng.choice(cands[f][max(0, 120):min(borders, 135)], size=600)  # on the borders around the 127th
    x[rng.random(x.shape) < 0.01] = np.nan
    o = OracleModel(model)
    g = _gpu_model(model)
    evaluate = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, 2500)["evaluate"]
    if depth <= 8 or split == "1":
        assert evaluate.startswith("cbamd_eval_reg_"), evaluate
        assert ("_m" in evaluate.split(" ")[0]) == (split == "0"), evaluate
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
    if evaluate.startswith("cbamd_eval_reg_"):
        np.testing.assert_array_equal(g.calc_flat(x), o.calc(x))
    else:
        _close(g.calc_flat(x), o.calc(x))
    n = len(model["tree_sizes"])
    if evaluate.startswith("cbamd_eval_reg_"):
        np.testing.assert_array_equal(g.calc_flat(x, tree_start=3, tree_end=n - 2), o.calc(x, tree_start=3, tree_end=n - 2))
    else:
        _close(g.calc_flat(x, tree_start=3, tree_end=n - 2), o.calc(x, tree_start=3, tree_end=n - 2))


def test_register_kernel_against_tile_kernel():
    """The same model with the register-resident kernels switched off: both paths agree."""
    rng = np.random.default_rng(5)
    model = _float_only_model(rng, 120, 300, 8)
    x = rng.normal(size=(20000, 120)).astype(np.float32)
    reg = _gpu_model(model).calc_flat(x)
    os.environ["CATBOOST_AMD_REG_KERNEL"] = "0"
    try:
        tile = _gpu_model(model).calc_flat(x)
    finally:
        del os.environ["CATBOOST_AMD_REG_KERNEL"]
    np.testing.assert_array_equal(reg, OracleModel(model).calc(x))
    _close(tile, reg)


def test_library_builder_matches_oracle_builder_and_roundtrips():
    rng = np.random.default_rng(11)
    ffs = [mb.float_feature(i, i) for i in range(5)]
    cfs = [mb.cat_feature(0, 5)]
    cands = [np.unique(rng.normal(size=30).astype(np.float32)) for _ in range(5)]
    trees = []
    for _ in range(30):
        splits = []
        for _ in range(int(rng.integers(1, 7))):
            if rng.random() < 0.2:
                splits.append(("onehot", 0, int(rng.integers(0, 5))))
            else:
                f = int(rng.integers(0, 5))
                splits.append(("float", f, float(rng.choice(cands[f]))))
        trees.append((splits, rng.normal(size=(1 << len(splits)) * 2)))
    ref = mb.build_oblivious(ffs, cfs, 2, trees, scale=2.0, bias=[0.5, -0.5])
    b = cb.ModelCalcer()
    b.build_oblivious(ffs, cfs, 2, trees, scale=2.0, bias=[0.5, -0.5])
    got = read_cbm(b.save_to_buffer())
    for k in ("tree_splits", "tree_sizes", "tree_start_offsets", "leaf_values", "bias"):
        np.testing.assert_array_equal(got[k], ref[k])
    for a, c in zip(got["float_features"], ref["float_features"]):
        np.testing.assert_array_equal(a["borders"], c["borders"])
    x = rng.normal(size=(300, 6)).astype(np.float32)
    x[:, 5] = rng.integers(0, 6, size=300).astype(np.int32).view(np.float32)
    _close(b.calc_flat(x), OracleModel(ref).calc(x))


# --------------------------------------------------------------------- the five workloads ----

@pytest.mark.both_batch_modes
@pytest.mark.parametrize("name,docs", [("C1", 30000), ("C2", 20000), ("C3", 10000), ("C4", 20000), ("C5", 6000)])
def test_workload_configs_host_path(name, docs):
    model, info = syn.build_model(name)
    o = OracleModel(read_cbm(model.save_to_buffer()))
    x = syn.host_features(info, docs)
    np.testing.assert_array_equal(model.quantize_flat(x), o.binarize(x))
    sample = slice(0, 2000)
    np.testing.assert_array_equal(model.calc_leaf_indexes_flat(x[sample]), o.leaf_indexes(x[sample]))
    _close(model.calc_flat(x), o.calc(x, threads=8))


@pytest.mark.parametrize("name,docs", [("C1", 100000), ("C2", 50000), ("C3", 20000), ("C4", 30000), ("C5", 10000)])
def test_workload_configs_device_path(name, docs):
    import torch

    model, info = syn.build_model(name)
    o = OracleModel(read_cbm(model.save_to_buffer()))
    ev = model.evaluator()
    x = syn.device_features(info, docs)
    out = torch.zeros(docs * info["dim"], dtype=torch.float64, device="cuda:0")
    out2 = torch.zeros_like(out)
    bins = torch.zeros(ev.quantized_bytes(docs), dtype=torch.uint8, device="cuda:0")
    exported = torch.zeros(docs * ev.bucket_count, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()  # the evaluator runs on its own stream: torch's fills must be done first
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    ev.eval_data(feats, docs, out.data_ptr())
    host = x.cpu().numpy()
    _close(out.cpu().numpy(), o.calc(host, threads=8))
    # separate quantize + evaluate on a caller-owned buffer, and the reference-layout export
    ev.quantize(feats, docs, bins.data_ptr())
    ev.eval_quantized(bins.data_ptr(), docs, out2.data_ptr())
    ev.export_quantized(bins.data_ptr(), docs, exported.data_ptr())
    ev.synchronize()
    assert torch.equal(out, out2)
    np.testing.assert_array_equal(exported.cpu().numpy(), o.binarize(host))
    binarize_ms, eval_ms = ev.last_kernel_times()
    assert binarize_ms >= 0 and eval_ms > 0  # a fused kernel reports its whole time as the evaluate time


def test_concurrent_callers():
    """Callers on threads of their own: the device entry points with caller-owned buffers and streams run
    side by side without sharing state; the host entry points of one handle borrow one of a few staging contexts
    each (a stream, pinned and device buffers), so flat, transposed and leaf-index calls overlap too, over several
    pipeline chunks each. Every result must equal the single-threaded one."""
    import threading

    import torch

    model, info = syn.build_model("C1")
    ev = model.evaluator()
    docs = 40_000
    x = syn.device_features(info, docs)
    expected = torch.zeros(docs, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    ev.eval_data(feats, docs, expected.data_ptr())
    ev.synchronize()
    host = x.cpu().numpy()
    expected_host = expected.cpu().numpy()
    errors = []

    def device_worker(k):
        try:
            stream = torch.cuda.Stream()
            bins = torch.zeros(ev.quantized_bytes(docs), dtype=torch.uint8, device="cuda:0")
            out = torch.zeros(docs, dtype=torch.float64, device="cuda:0")
            torch.cuda.synchronize()
            for _ in range(20):
                ev.quantize(feats, docs, bins.data_ptr(), stream=stream.cuda_stream)
                ev.eval_quantized(bins.data_ptr(), docs, out.data_ptr(), stream=stream.cuda_stream)
            ev.synchronize(stream=stream.cuda_stream)
            if not torch.equal(out, expected):
                errors.append("device worker %d differs" % k)
        except Exception as e:  # noqa: BLE001 - reported through the list
            errors.append("device worker %d: %r" % (k, e))

    def host_worker(k):
        try:
            for _ in range(5):
                if not np.array_equal(model.calc_flat(host[k * 1000:(k + 3) * 1000]), expected_host[k * 1000:(k + 3) * 1000]):
                    errors.append("host worker %d differs" % k)
        except Exception as e:  # noqa: BLE001
            errors.append("host worker %d: %r" % (k, e))

    # larger host batches (several chunks of the staging pipeline), through three entry point families at once
    big = np.ascontiguousarray(np.tile(host, (12, 1)))
    big_expected = np.tile(expected_host, 12)
    columns = np.ascontiguousarray(big.T)
    leaf_expected = model.calc_leaf_indexes_flat(host[:5000])

    def big_host_worker(k):
        try:
            for _ in range(2):
                if k % 3 == 0 and not np.array_equal(model.calc_flat(big), big_expected):
                    errors.append("big flat worker %d differs" % k)
                if k % 3 == 1 and not np.array_equal(model.calc_flat_transposed(columns), big_expected):
                    errors.append("big transposed worker %d differs" % k)
                if k % 3 == 2 and not np.array_equal(model.calc_leaf_indexes_flat(host[:5000]), leaf_expected):
                    errors.append("leaf index worker %d differs" % k)
        except Exception as e:  # noqa: BLE001
            errors.append("big host worker %d: %r" % (k, e))

    threads = [threading.Thread(target=device_worker, args=(k,)) for k in range(4)]
    threads += [threading.Thread(target=host_worker, args=(k,)) for k in range(4)]
    threads += [threading.Thread(target=big_host_worker, args=(k,)) for k in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert errors == []


def test_perftest_tool(golden_dir, tmp_path, capsys):
    import json

    from catboost_amd import perftest

    path = os.path.join(golden_dir, "features_num_cat__dataset_adult.cbm")
    assert perftest.main(["-m", path, "--docs", "20000", "--block-size", "4096", "--repetitions", "2"]) == 0
    report = json.loads(capsys.readouterr().out)
    assert report["docs"] == 20000 and report["block_size"] == 4096 and report["trees"] == 100
    assert report["host_flat_docs_per_sec"] > 0 and report["device_docs_per_sec"] > report["host_flat_docs_per_sec"]
    assert perftest.main(["-m", str(path), "--docs", "4096", "--block-size", "256", "--repetitions", "2", "--graph"]) == 0
    assert json.loads(capsys.readouterr().out)["graph_replay_docs_per_sec"] > 0
    assert perftest.main(["-m", str(path), "--docs", "16384", "--block-size", "1024", "--repetitions", "2", "-T", "4"]) == 0
    report = json.loads(capsys.readouterr().out)
    assert report["threads"] == 4 and report["host_flat_threads_docs_per_sec"] > 0
    # a pool of flat rows: the rust fixture's three documents (one string categorical column)
    pool = tmp_path / "pool.tsv"
    pool.write_text("".join("%g\t%g\t%s\t%g\n" % (f[0], f[1], c[0], f[2]) for f, c in zip(rm.RUST_FLOATS, rm.RUST_CATS)))
    assert perftest.main(["-m", os.path.join(golden_dir, "rust_tmp_model.cbm"), "-f", str(pool), "--repetitions", "1"]) == 0
    assert json.loads(capsys.readouterr().out)["docs"] == 3


def test_plain_c_client_of_the_c_abi(golden_dir):
    """A C program linked against libcatboostmodel.so the way users of the reference library are."""
    import subprocess

    exe = os.path.join(os.path.dirname(__file__), "bin", "c_abi_client")
    if not os.path.exists(exe):
        pytest.skip("tests/bin/c_abi_client is not built (run __graft_entry__.build())")
    out = subprocess.check_output([exe, os.path.join(golden_dir, "numeric_only_model.cbm"), "0.1", "0.3", "0.2"],
                                  timeout=120)
    assert abs(float(out.decode().split()[0]) - rm.NUMERIC_ONLY_EXPECTED[0]) < 1e-15


def test_client_of_the_reference_wrapper_header(golden_dir):
    """A C++ program written against the reference's own wrapped_calcer.h and c_api.h
    (catboost/libs/model_interface), compiled unchanged and linked against this library: every
    way that wrapper calls the model gives the goldens of the reference's own tests
    (catboost/rust-package/src/model.rs:475-520, catboost/libs/model_interface/ut)."""
    import subprocess

    exe = os.path.join(os.path.dirname(__file__), "bin", "wrapped_calcer_client")
    if not os.path.exists(exe):
        pytest.skip("tests/bin/wrapped_calcer_client is not built (run __graft_entry__.build() where the reference is)")

    def run(model, floats, cats):
        text = "".join(" ".join("%r" % float(v) for v in f) + " | " + " ".join(c) + "\n" for f, c in zip(floats, cats))
        out = subprocess.check_output([exe, os.path.join(golden_dir, model)], input=text.encode(), timeout=120)
        lines = {}
        for line in out.decode().splitlines():
            name, _, rest = line.partition(" ")
            lines[name] = rest
        return lines

    got = run("rust_tmp_model.cbm", rm.RUST_FLOATS, rm.RUST_CATS)
    assert got["counts"].split()[1:] == ["3", "1", "0", "0"]
    assert int(got["evaluators"]) >= 1
    assert got["short_document"] == "refused" and got["missing_key"] == "[]"
    for name in ("single", "batch", "hashed", "from_memory", "after_error"):
        _close(np.array([float(v) for v in got[name].split()]), rm.RUST_EXPECTED)

    got = run("numeric_only_model.cbm", rm.NUMERIC_ONLY_ROWS, [[] for _ in rm.NUMERIC_ONLY_ROWS])
    assert got["counts"].split()[2] == "0"
    for name in ("single", "batch", "hashed", "flat_single", "flat", "flat_transposed", "from_memory", "after_error"):
        _close(np.array([float(v) for v in got[name].split()]), rm.NUMERIC_ONLY_EXPECTED)

    # a model with CTR features through the same wrapper
    got = run("features_num_cat__dataset_adult.cbm", rm.RUST_ADULT_FLOATS, rm.RUST_ADULT_CATS)
    for name in ("single", "batch", "hashed", "from_memory"):
        _close(np.array([float(v) for v in got[name].split()]), rm.RUST_ADULT_EXPECTED)


# ----------------------------------------------------------------------------- error paths ----

def test_error_paths(golden_dir):
    g = cb.ModelCalcer(os.path.join(golden_dir, "numeric_only_model.cbm"))
    with pytest.raises(cb.CatBoostError, match="results. size is insufficient"):
        g.calc_flat(rm.NUMERIC_ONLY_ROWS, result_size=3)
    with pytest.raises(cb.CatBoostError, match="insufficient"):
        g.calc_flat(rm.NUMERIC_ONLY_ROWS[:, :2])
    with pytest.raises(cb.CatBoostError):
        g.enable_gpu_evaluation(99)
    with pytest.raises(cb.CatBoostError, match="Incorrect model file descriptor"):
        cb.ModelCalcer(os.path.join(golden_dir, "not_a_model.cbm"))
    with pytest.raises(cb.CatBoostError, match="not supported"):
        cb.ModelCalcer(os.path.join(golden_dir, "jvm_model_with_text_features.cbm"))
    # the handle still works after failed calls
    _close(g.calc_flat(rm.NUMERIC_ONLY_ROWS), rm.NUMERIC_ONLY_EXPECTED)


# --------------------------------------------------- full workload size, properties ----

def test_c2_full_size_properties():
    """C2 at its full 4M documents on the device path. The oracle checks a sample; the rest is
    covered by properties that hold at any size: a prediction does not depend on where its
    document sits in the batch (bit for bit on the register-resident kernels), quantize +
    evaluate equals the one-call path, and tree sub-ranges add up to the whole model."""
    import torch

    docs = 4_000_000
    model, info = syn.build_model("C2")
    ev = model.evaluator()
    x = syn.device_features(info, docs)
    out = torch.zeros(docs, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    ev.eval_data(feats, docs, out.data_ptr())
    ev.synchronize()
    # sample against the oracle
    rng = np.random.default_rng(3)
    sample = np.sort(rng.choice(docs, 4000, replace=False))
    sample_t = torch.from_numpy(sample).to("cuda:0")
    o = OracleModel(read_cbm(model.save_to_buffer()))
    np.testing.assert_array_equal(out[sample_t].cpu().numpy(), o.calc(x[sample_t].cpu().numpy()))
    # position independence: the batch reversed block-wise with a ragged tail
    keep = docs - 12345
    perm = torch.arange(keep - 1, -1, -1, device="cuda:0")
    xp = x[perm].contiguous()
    outp = torch.zeros(keep, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, xp.data_ptr(), xp.shape[1]), keep, outp.data_ptr())
    ev.synchronize()
    assert torch.equal(outp, out[perm])
    del xp, outp, perm
    # quantize into a caller-owned buffer, evaluate from it
    bins = torch.zeros(ev.quantized_bytes(docs), dtype=torch.uint8, device="cuda:0")
    out2 = torch.zeros_like(out)
    torch.cuda.synchronize()
    ev.quantize(feats, docs, bins.data_ptr())
    ev.eval_quantized(bins.data_ptr(), docs, out2.data_ptr())
    ev.synchronize()
    assert torch.equal(out, out2)
    # tree sub-ranges (register kernels for the whole tree blocks, the plain kernel for a range's ragged ends) add up to
    # the whole model (scale 1, bias 0 in this workload)
    trees = model.tree_count
    parts = torch.zeros_like(out)
    part = torch.zeros_like(out)
    torch.cuda.synchronize()
    for begin, end in ((0, 300), (300, 301), (301, trees)):
        ev.eval_quantized(bins.data_ptr(), docs, part.data_ptr(), tree_start=begin, tree_end=end)
        ev.synchronize()
        parts += part
    torch.cuda.synchronize()
    assert torch.allclose(parts, out, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("cfg,trees", [("C2", 210), ("C3", 75), ("C1", 200)])
def test_tree_ranges_stay_on_the_register_kernels_and_equal_the_oracle(cfg, trees):
    """CalcTreesBlockedImpl (cpu/evaluator_impl.cpp:257-414) runs any [treeStart, treeEnd) through its one loop
    and ApplyScaleAndBias adds the bias only when the range starts at tree 0 (scale_and_bias.cpp:13-24). Here
    the whole tree blocks of a range go through the register-resident kernel and the few trees before and after
    them through the kernel that follows the model's tables, all adding in tree order: equal to the oracle bit
    for bit, for the device and the host entry points."""
    import torch

    model, info = syn.build_model(cfg, trees=trees)
    model.set_scale_and_bias(0.5, [0.25 * (k + 1) for k in range(info["dim"])])
    ev = model.evaluator()
    oracle = OracleModel(read_cbm(model.save_to_buffer()))
    docs, dim = 3001, info["dim"]
    x = syn.device_features(info, docs)
    host = x.cpu().numpy()
    bins = torch.zeros(ev.quantized_bytes(docs), dtype=torch.uint8, device="cuda:0")
    out = torch.zeros(docs * dim, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    ev.quantize(ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]), docs, bins.data_ptr())
    ranges = [(0, trees), (0, 16), (0, 17), (3, 17), (5, 9), (16, 48), (1, trees), (15, trees - 1), (33, 64),
              (31, 33), (7, 7), (0, 0), (trees, trees), (trees - 3, trees), (64, trees)]
    for begin, end in ranges:
        out.fill_(-3.0)
        torch.cuda.synchronize()
        ev.eval_quantized(bins.data_ptr(), docs, out.data_ptr(), tree_start=begin, tree_end=end)
        ev.synchronize()
        expected = oracle.calc(host, tree_start=begin, tree_end=end, threads=8)
        np.testing.assert_array_equal(out.cpu().numpy(), expected, err_msg="trees [%d, %d)" % (begin, end))
    np.testing.assert_array_equal(model.calc_flat(host[:700], tree_start=19, tree_end=trees - 20),
                                  oracle.calc(host[:700], tree_start=19, tree_end=trees - 20))


def test_c5_full_size_properties():
    """C5 at its full 10M documents (41 GB of features): a sample of the outputs against the oracle, the same
    documents at other positions of the batch give the same bits, and tree ranges add up to the whole model."""
    import torch

    model, info = syn.build_model("C5")
    ev = model.evaluator()
    oracle = OracleModel(read_cbm(model.save_to_buffer()))
    docs = info["docs"]
    x = syn.device_features(info, docs)
    out = torch.zeros(docs, dtype=torch.float64, device="cuda:0")
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    torch.cuda.synchronize()
    ev.eval_data(feats, docs, out.data_ptr())
    torch.cuda.synchronize()
    sample = torch.randperm(docs, device="cuda:0")[:3000].sort().values
    _close(out[sample].cpu().numpy(), oracle.calc(x[sample].cpu().numpy(), threads=8))
    # position independence: the last 70 001 documents moved to the front of a smaller batch
    tail = 70_001
    moved = x[docs - tail:].contiguous()
    out_moved = torch.zeros(tail, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, moved.data_ptr(), moved.shape[1]), tail, out_moved.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(out_moved, out[docs - tail:])
    # additivity over tree ranges on a slice of the batch (scale 1, bias 0 in this workload)
    part_docs = 200_000
    total = torch.zeros(part_docs, dtype=torch.float64, device="cuda:0")
    part = torch.zeros(part_docs, dtype=torch.float64, device="cuda:0")
    for begin, end in ((0, 1700), (1700, 1701), (1701, model.tree_count)):
        torch.cuda.synchronize()
        ev.eval_data(feats, part_docs, part.data_ptr(), tree_start=begin, tree_end=end)
        torch.cuda.synchronize()
        total += part
    assert torch.allclose(total, out[:part_docs], rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("name,base_docs,copies", [("C2", 1_000_000, 23), ("C4", 1_000_000, 15), ("C3", 500_000, 110)])
def test_batches_beyond_four_gibibytes(name, base_docs, copies):
    """Batches whose features, bins or results pass 4 GiB (C2: 18 GB of features, 4.6 GB of bins; C3: 4.4 GB
    of results): a base batch repeated `copies` times plus a ragged tail must give the base batch's
    predictions at every repetition, bit for bit - any 32-bit overflow in a kernel's addressing would
    break that."""
    import torch

    model, info = syn.build_model(name)
    ev = model.evaluator()
    dim = info["dim"]
    base = syn.device_features(info, base_docs)
    tail = 777
    docs = base_docs * copies + tail
    x = torch.empty((docs, base.shape[1]), dtype=torch.float32, device="cuda:0")
    for c in range(copies):
        x[c * base_docs:(c + 1) * base_docs] = base
    x[copies * base_docs:] = base[:tail]
    expected = torch.zeros(base_docs * dim, dtype=torch.float64, device="cuda:0")
    out = torch.zeros(docs * dim, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, base.data_ptr(), base.shape[1]), base_docs, expected.data_ptr())
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]), docs, out.data_ptr())
    ev.synchronize()
    assert ev.quantized_bytes(docs) > (1 << 32) or name == "C3"
    # a batch whose results pass what a launch of the register kernels addresses (C3) goes in slices through
    # the same kernels: every repetition equals the base batch bit for bit
    first = out[:base_docs * dim]
    assert torch.equal(first, expected)
    for c in range(1, copies):
        assert torch.equal(out[c * base_docs * dim:(c + 1) * base_docs * dim], first), "repetition %d" % c
    assert torch.equal(out[copies * base_docs * dim:], first[:tail * dim])
    # a tree sub-range
    half = model.tree_count // 2
    part = torch.zeros_like(out)
    part_base = torch.zeros_like(expected)
    torch.cuda.synchronize()
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, base.data_ptr(), base.shape[1]), base_docs, part_base.data_ptr(),
                 tree_start=half, tree_end=model.tree_count)
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]), docs, part.data_ptr(),
                 tree_start=half, tree_end=model.tree_count)
    ev.synchronize()
    assert torch.equal(part[(copies - 1) * base_docs * dim:copies * base_docs * dim], part_base)
    assert torch.equal(part[:base_docs * dim], part_base)
