"""Seeded sweep over random model shapes on the GPU: the library against the oracle, through the C ABI.

Each seed draws a model (oblivious, the same converted to non-symmetric, or one with CTR features of every
kind), a document count around the block sizes, and the switches that pick between kernels of equal
results; bins and leaf indexes must be equal, predictions within 1e-9 rel / 1e-12 abs. The default run
takes a few seconds; CATBOOST_AMD_SWEEP_SEEDS=first:count widens it (tens of thousands of seeds fit in
minutes).
"""
import os

import numpy as np
import pytest

import catboost_amd as cb
from oracle import model_builder as mb
from oracle.oracle import OracleModel
from tests import cbm_writer, ctr_models
from tests import refmodels as rm
from tests.test_oracle import _random_flat_data, _random_oblivious

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-9, 1e-12


def _seeds():
    first, count = (int(x) for x in os.environ.get("CATBOOST_AMD_SWEEP_SEEDS", "500000:240").split(":"))
    return range(first, first + count)


def _check(tag, g, o, x):
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x), err_msg=tag)
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x), err_msg=tag)
    expected = o.calc(x)
    np.testing.assert_allclose(g.calc_flat(x), expected, rtol=RTOL, atol=ATOL, err_msg=tag)
    np.testing.assert_allclose(g.calc_flat_transposed(np.ascontiguousarray(x.T)), expected, rtol=RTOL, atol=ATOL,
                               err_msg=tag)
    if o.tree_count >= 2:
        a, b = sorted(int(v) for v in np.random.default_rng(len(tag)).integers(0, o.tree_count + 1, size=2))
        np.testing.assert_allclose(g.calc_flat(x, tree_start=a, tree_end=b), o.calc(x, tree_start=a, tree_end=b),
                                   rtol=RTOL, atol=ATOL, err_msg=tag)


def _tree_model_case(seed, rng, asymmetric):
    dim = int(rng.choice([1, 1, 1, 2, 3, 5, 10, 20]))
    n_float = int(rng.choice([1, 2, 7, 30, 100, 130, 200, 209, 224, 250, 400, 700, 1100]))
    n_cat = int(rng.choice([0, 0, 1, 2, 5]))
    trees = int(rng.choice([1, 2, 17, 40, 150, 400]))
    max_depth = int(rng.choice([1, 3, 6, 8, 10, 12]))
    many = bool(rng.integers(0, 2))
    docs = int(rng.choice([1, 2, 63, 64, 65, 255, 256, 257, 1000, 3333, 9000]))
    trees = min(trees, max(1, 40000 // n_float))
    tag = "seed %d dim %d floats %d cats %d trees %d depth<=%d many borders %s docs %d non-symmetric %s" % (
        seed, dim, n_float, n_cat, trees, max_depth, many, docs, asymmetric)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth,
                                          dim=dim, many_borders=many, scale=float(rng.choice([1.0, 0.5, -2.0])),
                                          bias=rng.normal(size=dim) if rng.integers(0, 2) else None)
    if asymmetric:
        model = mb.convert_oblivious_to_asymmetric(model)
    x = _random_flat_data(rng, model, cat_values, docs)
    g = cb.ModelCalcer()
    g.load_from_dict(model)
    g.enable_gpu_evaluation(0)
    _check(tag, g, OracleModel(model), x)


def _ctr_model_case(seed, rng, monkeypatch):
    kwargs = dict(n_float=int(rng.choice([2, 3, 4, 8])), n_cat=int(rng.choice([1, 2, 4, 8, 20, 70])),
                  n_bases=int(rng.choice([1, 3, 8, 20, 40])), n_trees=int(rng.choice([1, 10, 60])),
                  max_depth=int(rng.choice([1, 4, 8])), wide_float=bool(rng.integers(0, 2)),
                  dim=int(rng.choice([1, 1, 3])))
    docs = int(rng.choice([1, 64, 257, 2000]))
    tile = str(int(rng.integers(0, 2)))
    monkeypatch.setenv("CATBOOST_AMD_CTR_TILE", tile)
    tag = "seed %d ctr model %s docs %d tile kernel %s" % (seed, kwargs, docs, tile)
    model, known = ctr_models.random_ctr_model(seed, **kwargs)
    floats, cats = ctr_models.random_documents(model, known, docs, seed + 7)
    g = cb.ModelCalcer(buffer=cbm_writer.write_cbm(model))
    g.enable_gpu_evaluation(0)
    o = OracleModel(model)
    _check(tag, g, o, rm.flat_rows(model, floats, cats))
    np.testing.assert_array_equal(g.quantize_hashed(floats, cats), o.binarize(floats, cats, layout="split"), err_msg=tag)
    np.testing.assert_allclose(g.calc_hashed(floats, cats), o.calc(floats, cats, layout="split"), rtol=RTOL, atol=ATOL,
                               err_msg=tag)


def test_random_model_shapes(monkeypatch, capsys):
    seeds = _seeds()
    for seed in seeds:
        if (seed - seeds[0]) % 2000 == 1999:
            with capsys.disabled():  # a long run shows that it is alive
                print("sweep: %d of %d seeds" % (seed - seeds[0] + 1, len(seeds)), flush=True)
        rng = np.random.default_rng(seed)
        kind = seed % 3
        monkeypatch.setenv("CATBOOST_AMD_REG_SIX", str(int(rng.integers(0, 2))))
        # fused or two launches, a tree's levels ordered or as in the model, small batches sliced or in one pass
        monkeypatch.setenv("CATBOOST_AMD_FUSED", str(int(rng.integers(0, 2))))
        monkeypatch.setenv("CATBOOST_AMD_LEVEL_ORDER", str(int(rng.integers(0, 2))))
        monkeypatch.setenv("CATBOOST_AMD_SMALL_BATCH", str(int(rng.integers(0, 2))))
        monkeypatch.setenv("CATBOOST_AMD_REG_SPLIT", str(int(rng.integers(0, 2))))
        monkeypatch.setenv("CATBOOST_AMD_ROW_TILE", str(int(rng.integers(0, 2))))
        # the shape of the non-symmetric LDS kernel: chosen by the model, or one of the five
        monkeypatch.setenv("CATBOOST_AMD_NS_WAVES", str(int(rng.choice([0, 4, 6, 8, 12, 16]))))
        if kind == 2:
            _ctr_model_case(seed, rng, monkeypatch)
        else:
            _tree_model_case(seed, rng, asymmetric=kind == 1)
