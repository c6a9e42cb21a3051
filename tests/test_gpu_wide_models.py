"""One-dimensional oblivious models with more buckets than the register kernels take: the tile kernels with a
tree's row in registers or broadcast from a lane (the 256-document tile fits LDS, up to ~630 buckets), and
above that the half-tile kernels, one tree or two trees per wave; against the oracle through the C ABI.

The two kernels add the trees of a document in different orders (partial sums per wave, and per lane group
in the two-tree kernel), so predictions are compared within 1e-9 rel / 1e-12 abs; the bins must be equal.
"""
import numpy as np
import pytest

import catboost_amd as cb
from oracle.oracle import OracleModel
from tests.test_oracle import _random_flat_data, _random_oblivious

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-9, 1e-12


def _evaluator(model, monkeypatch, pair):
    monkeypatch.setenv("CATBOOST_AMD_PAIR_TILE", pair)
    g = cb.ModelCalcer()
    g.load_from_dict(model)
    g.enable_gpu_evaluation(0)
    return g


@pytest.mark.parametrize("pair", ["1", "0"])
@pytest.mark.parametrize("seed,n_float,n_cat,trees,max_depth,docs", [
    (1, 900, 0, 601, 8, 1000),    # odd tree count: the last tree has no partner
    (2, 900, 12, 600, 8, 129),    # one-hot levels: the xor form, in some pairs only
    (3, 800, 40, 450, 6, 1),      # 64 leaves per tree, a single document
    (4, 1000, 3, 1400, 3, 5000),  # shallow trees in the 64-leaf kernel
])
def test_wide_models_against_the_oracle(monkeypatch, pair, seed, n_float, n_cat, trees, max_depth, docs):
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth,
                                          scale=float(rng.choice([1.0, -0.5])), bias=rng.normal(size=1))
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = _evaluator(model, monkeypatch, pair)
    assert g.bucket_count > 632, "the model must not fit the 256-document tile"
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    assert kernels["evaluate"] == ("EvalObliviousPairTileKernel" if pair == "1" else "EvalObliviousHalfTileKernel")
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    # tree ranges of odd and even lengths, from even and odd first trees, down to one pair, one tree and none;
    # the bias only with tree 0
    for begin, end in ((0, 1), (1, 2), (0, 2), (7, 9), (0, trees - 1), (1, trees), (3, 3), (trees // 2, trees),
                       (5, 8), (trees - 1, trees)):
        if end <= trees and begin <= end:
            np.testing.assert_allclose(g.calc_flat(x, tree_start=begin, tree_end=end),
                                       o.calc(x, tree_start=begin, tree_end=end), rtol=RTOL, atol=ATOL,
                                       err_msg="trees %d..%d" % (begin, end))


@pytest.mark.parametrize("n_float,trees,docs,kernel", [
    (800, 500, 700, "EvalObliviousPairTileKernel"),    # 717 rows of 128 bytes and the leaf regions fit LDS
    (1100, 900, 300, "EvalObliviousQuadTileKernel"),   # 1045 rows do not: rows of 64 bytes, four trees per wave
])
def test_wide_models_with_bins_above_127(monkeypatch, n_float, trees, docs, kernel):
    """A feature with 300 borders: its bucket of more than 127 values takes two rows of the tile, min(bin, 127)
    and max(bin - 127, 0), and the kernels with two or four trees per wave compare 7 bits as before."""
    rng = np.random.default_rng(11)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=4, trees=trees, max_depth=8, many_borders=True)
    assert max(len(f["borders"]) for f in model["float_features"]) > 127
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = _evaluator(model, monkeypatch, "1")
    assert g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)["evaluate"] == kernel
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(g.calc_flat(x, tree_start=3, tree_end=trees - 2), o.calc(x, tree_start=3, tree_end=trees - 2),
                               rtol=RTOL, atol=ATOL)


def test_two_kernels_agree_on_a_large_batch(monkeypatch):
    """66 000 documents (a ragged last block) through both kernels of one model."""
    rng = np.random.default_rng(12)
    model, cat_values = _random_oblivious(rng, n_float=950, n_cat=8, trees=301, max_depth=8)
    x = _random_flat_data(rng, model, cat_values, 66_000)
    two = _evaluator(model, monkeypatch, "1").calc_flat(x)
    one = _evaluator(model, monkeypatch, "0").calc_flat(x)
    np.testing.assert_allclose(two, one, rtol=RTOL, atol=ATOL)
    sample = np.random.default_rng(0).choice(66_000, size=2000, replace=False)
    np.testing.assert_allclose(two[sample], OracleModel(model).calc(x[sample]), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("rows_in_registers", ["1", "0"])
@pytest.mark.parametrize("seed,n_float,n_cat,trees,max_depth,docs", [
    (21, 230, 0, 301, 8, 1000),   # two workgroups of eight waves share a CU
    (22, 400, 6, 200, 8, 513),    # sixteen waves; one-hot levels in some trees
    (23, 560, 0, 500, 8, 255),    # 552 buckets: the tile leaves room for eight regions only
    (24, 300, 20, 333, 6, 1),     # 64 leaves per tree, a single document
    (25, 560, 2, 400, 3, 4097),   # shallow trees in the 64-leaf kernel
    (41, 300, 2, 300, 8, 777),    # (seeds from 41: a feature of 300 borders, whose large bucket takes two rows)
    (43, 500, 0, 800, 8, 64),
])
def test_tile_models_against_the_oracle(monkeypatch, rows_in_registers, seed, n_float, n_cat, trees, max_depth, docs):
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth,
                                          many_borders=seed >= 41, scale=float(rng.choice([1.0, -0.5])),
                                          bias=rng.normal(size=1))
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    monkeypatch.setenv("CATBOOST_AMD_ROW_TILE", rows_in_registers)
    g = cb.ModelCalcer()
    g.load_from_dict(model)
    g.enable_gpu_evaluation(0)
    assert 224 < g.bucket_count <= 632, "the model must take a tile kernel"
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    assert kernels["evaluate"] == ("EvalObliviousRowTileKernel" if rows_in_registers == "1" else "EvalObliviousTileKernel")
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    for begin, end in ((0, 1), (1, 2), (0, 17), (7, 9), (0, trees - 1), (1, trees), (3, 3), (trees // 2, trees),
                       (trees - 1, trees)):
        if end <= trees and begin <= end:
            np.testing.assert_allclose(g.calc_flat(x, tree_start=begin, tree_end=end),
                                       o.calc(x, tree_start=begin, tree_end=end), rtol=RTOL, atol=ATOL,
                                       err_msg="trees %d..%d" % (begin, end))


@pytest.mark.parametrize("seed,dim,n_float,n_cat,trees,max_depth,docs,registers", [
    (31, 2, 300, 0, 300, 8, 1000, "1"),   # two dimensions: one slice
    (32, 3, 280, 6, 300, 6, 513, "1"),    # 64 leaves and three dimensions: one slice of four; one-hot levels
    (33, 10, 420, 0, 400, 6, 255, "1"),   # five slices
    (34, 5, 300, 2, 200, 8, 4097, "1"),   # 256 leaves, three slices
    (35, 3, 30, 2, 50, 8, 700, "0"),      # a small tile: two workgroups of eight waves per CU
    (36, 13, 520, 0, 450, 5, 129, "1"),   # 494 buckets: room for eight leaf regions only
    (42, 3, 350, 3, 200, 6, 900, "1"),    # (seeds from 41: a feature of 300 borders, whose large bucket takes two rows)
])
def test_tile_models_of_several_dimensions(monkeypatch, seed, dim, n_float, n_cat, trees, max_depth, docs, registers):
    """Models of several dimensions on the tile kernel with a tree's row in registers: a workgroup sums two
    dimensions at a time over the same tile, slice after slice (four when that is the whole model)."""
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth, dim=dim,
                                          many_borders=seed >= 41, scale=float(rng.choice([1.0, -0.5])),
                                          bias=rng.normal(size=dim))
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    monkeypatch.setenv("CATBOOST_AMD_REG_KERNEL", registers)
    g = cb.ModelCalcer()
    g.load_from_dict(model)
    g.enable_gpu_evaluation(0)
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    assert kernels["evaluate"] == "EvalObliviousRowTileKernel", kernels
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    for begin, end in ((0, 1), (1, 2), (0, 17), (0, trees - 1), (1, trees), (3, 3), (trees // 2, trees)):
        np.testing.assert_allclose(g.calc_flat(x, tree_start=begin, tree_end=end),
                                   o.calc(x, tree_start=begin, tree_end=end), rtol=RTOL, atol=ATOL,
                                   err_msg="trees %d..%d" % (begin, end))


@pytest.mark.parametrize("dim", [1, 3])
@pytest.mark.parametrize("row_tile", ["1", "0"])
def test_trees_without_splits_on_the_tile_kernels(monkeypatch, row_tile, dim):
    """A model whose trees have no splits has no buckets; its documents keep one all-zero bucket, which is the
    row that the padding levels of the tile kernels read. Every document gets the sum of the trees' only leaves."""
    monkeypatch.setenv("CATBOOST_AMD_REG_KERNEL", "0")
    monkeypatch.setenv("CATBOOST_AMD_ROW_TILE", row_tile)
    leaves = [([], [0.25 + k for k in range(dim)]), ([], [0.5 - k for k in range(dim)]), ([], [2.0] * dim)]
    g = cb.ModelCalcer()
    g.build_oblivious([dict(index=0, flat_index=0)], [], dim, leaves, bias=[1.0] * dim)
    g.enable_gpu_evaluation(0)
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, 700)
    assert kernels["evaluate"] == ("EvalObliviousRowTileKernel" if row_tile == "1" else "EvalObliviousTileKernel")
    x = np.random.default_rng(0).normal(size=(700, 1)).astype(np.float32)
    expected = np.array([1.0 + sum(leaf[1][k] for leaf in leaves) for k in range(dim)])
    np.testing.assert_allclose(g.calc_flat(x).reshape(700, dim), np.tile(expected, (700, 1)), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(g.calc_flat(x, tree_start=1, tree_end=3).reshape(700, dim),
                               np.tile(expected - 1.0 - np.array([leaves[0][1][k] for k in range(dim)]), (700, 1)),
                               rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed,n_float,n_cat,trees,max_depth,many,docs", [
    (51, 40, 0, 60, 12, False, 1000),   # twelve levels: four in the second half; two workgroups of eight waves per CU
    (52, 30, 5, 25, 16, False, 513),    # sixteen levels, one-hot levels in either half
    (53, 300, 3, 40, 11, True, 255),    # a feature of 300 borders: two rows of the tile for its large bucket
    (54, 20, 4, 80, 10, False, 4097),   # depth 10 with one-hot splits, which the register kernels do not take
    (55, 500, 0, 30, 14, False, 64),    # a tile of which one fits a CU: sixteen waves
])
def test_deep_trees_on_the_tile_kernel(seed, n_float, n_cat, trees, max_depth, many, docs):
    """One-dimensional models of depth 9 to 16 outside the register kernels: the tile kernel that walks a tree's
    levels in two halves and gathers the leaf values from the model's table. Bins and leaf indexes equal the
    oracle's, predictions within the tolerance (partial sums per wave)."""
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth,
                                          many_borders=many, scale=float(rng.choice([1.0, -0.5])),
                                          bias=rng.normal(size=1))
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = cb.ModelCalcer()
    g.load_from_dict(model)
    g.enable_gpu_evaluation(0)
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    assert kernels["evaluate"] == "EvalObliviousDeepTileKernel", kernels
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    for begin, end in ((0, 1), (1, 2), (0, 17), (0, trees - 1), (1, trees), (3, 3), (trees // 2, trees)):
        np.testing.assert_allclose(g.calc_flat(x, tree_start=begin, tree_end=end),
                                   o.calc(x, tree_start=begin, tree_end=end), rtol=RTOL, atol=ATOL,
                                   err_msg="trees %d..%d" % (begin, end))


@pytest.mark.parametrize("quad", ["1", "0"])
@pytest.mark.parametrize("seed,n_float,n_cat,trees,max_depth,many,docs", [
    (61, 1300, 0, 901, 8, False, 700),    # 1241 buckets; a last tree without partners
    (62, 1500, 6, 602, 8, False, 129),    # one-hot levels; two trees left over
    (63, 1700, 10, 1503, 6, False, 65),   # 64 leaves per tree, 1541 buckets; three trees left over
    (64, 1250, 3, 700, 8, True, 1),       # a feature of 300 borders: two rows for its large bucket; a single document
    (65, 1900, 4, 1500, 8, False, 300),   # 1766 buckets: LDS for four waves' leaf regions only
])
def test_very_wide_models_against_the_oracle(monkeypatch, quad, seed, n_float, n_cat, trees, max_depth, many, docs):
    """More rows than the half tile holds: a tile of 64 documents with four trees per wave, or (switched off) the
    half-tile kernel with one tree per wave while its tile fits, else the plain kernel."""
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth,
                                          many_borders=many, scale=float(rng.choice([1.0, -0.5])),
                                          bias=rng.normal(size=1))
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = _evaluator(model, monkeypatch, quad)
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    if quad == "1":
        assert kernels["evaluate"] == "EvalObliviousQuadTileKernel", kernels
    else:
        assert kernels["evaluate"] in ("EvalObliviousHalfTileKernel", "EvalObliviousKernel"), kernels
    np.testing.assert_array_equal(g.quantize_flat(x), o.binarize(x))
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    for begin, end in ((0, 1), (1, 2), (0, 3), (2, 9), (0, trees - 1), (1, trees), (3, 3), (trees // 2, trees),
                       (5, 8), (trees - 3, trees)):
        np.testing.assert_allclose(g.calc_flat(x, tree_start=begin, tree_end=end),
                                   o.calc(x, tree_start=begin, tree_end=end), rtol=RTOL, atol=ATOL,
                                   err_msg="trees %d..%d" % (begin, end))


@pytest.mark.parametrize("seed,dim,n_float,n_cat,trees,max_depth,docs", [
    (61, 3, 40, 0, 60, 12, 1000),    # twelve levels, three dimensions: two slices of two
    (62, 2, 30, 5, 25, 16, 513),     # sixteen levels, one-hot levels in either half, one slice
    (63, 10, 300, 3, 30, 11, 255),   # five slices over a tile of 300 rows
    (64, 5, 20, 4, 40, 9, 4097),     # depth 9 with one-hot splits and several dimensions
])
def test_deep_trees_of_several_dimensions_on_the_tile_kernel(seed, dim, n_float, n_cat, trees, max_depth, docs):
    """Models of depth 9 to 16 with several dimensions: the deep-tile kernel sums two dimensions per walk of the
    trees (the plain kernel took these before). Leaf indexes equal the oracle's, predictions within the tolerance."""
    rng = np.random.default_rng(seed)
    model, cat_values = _random_oblivious(rng, n_float=n_float, n_cat=n_cat, trees=trees, max_depth=max_depth, dim=dim,
                                          scale=float(rng.choice([1.0, -0.5])), bias=rng.normal(size=dim))
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = cb.ModelCalcer()
    g.load_from_dict(model)
    g.enable_gpu_evaluation(0)
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    assert kernels["evaluate"] == "EvalObliviousDeepTileKernel", kernels
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    for begin, end in ((0, 1), (1, 2), (0, 17), (0, trees - 1), (1, trees), (3, 3), (trees // 2, trees)):
        np.testing.assert_allclose(g.calc_flat(x, tree_start=begin, tree_end=end),
                                   o.calc(x, tree_start=begin, tree_end=end), rtol=RTOL, atol=ATOL,
                                   err_msg="trees %d..%d" % (begin, end))


def _model_with_a_large_one_hot_bucket(rng, n_float, trees, max_depth, cardinality, dim=1):
    """Oblivious model over n_float float features and one categorical feature of `cardinality` values, every one
    of which some one-hot split tests: the feature's bucket then holds that many values (bins up to `cardinality`)."""
    from oracle import model_builder as mb
    from oracle.oracle import integer_cat_feature_hash

    ffs = [mb.float_feature(i, i) for i in range(n_float)]
    cfs = [mb.cat_feature(0, n_float)]
    cands = {i: np.unique(rng.normal(size=int(rng.integers(1, 6))).astype(np.float32)) for i in range(n_float)}
    values = [integer_cat_feature_hash(v) for v in range(cardinality)]
    tree_list = []
    for t in range(trees):
        depth = int(rng.integers(1, max_depth + 1))
        splits = []
        for d in range(depth):
            if rng.random() < 0.3:
                splits.append(("onehot", 0, int(values[int(rng.integers(0, cardinality))])))
            else:
                f = int(rng.integers(0, n_float))
                splits.append(("float", f, float(rng.choice(cands[f]))))
        tree_list.append((splits, rng.normal(size=(1 << depth) * dim)))
    for v in values:
        tree_list.append(([("onehot", 0, int(v))], rng.normal(size=2 * dim)))
    return mb.build_oblivious(ffs, cfs, dim, tree_list, scale=0.5, bias=rng.normal(size=dim)), {0: values}


@pytest.mark.parametrize("seed,n_float,trees,max_depth,cardinality,dim,kernel", [
    (71, 300, 200, 8, 200, 1, "EvalObliviousRowTileKernel"),    # values below and above 127 of one bucket
    (72, 300, 700, 6, 254, 3, "EvalObliviousRowTileKernel"),    # the largest bucket a feature can have, three dimensions
    (73, 900, 900, 8, 130, 1, "EvalObliviousPairTileKernel"),   # two trees per wave on half a tile
    (74, 60, 40, 12, 180, 1, "EvalObliviousDeepTileKernel"),    # in either half of a deep tree's levels
])
def test_one_hot_bucket_of_more_than_127_values_on_the_tile_kernels(seed, n_float, trees, max_depth, cardinality, dim, kernel):
    """A one-hot bucket of more than 127 values takes two rows of the tile (the bins up to 127, and bin - 127 from
    128 on), so that "bin == value" stays a 7-bit compare: such models ran on the half-tile or the plain kernel
    before. Bins and leaf indexes equal the oracle's, predictions within the tolerance."""
    rng = np.random.default_rng(seed)
    model, cat_values = _model_with_a_large_one_hot_bucket(rng, n_float, trees, max_depth, cardinality, dim)
    docs = 3000
    x = _random_flat_data(rng, model, cat_values, docs)
    o = OracleModel(model)
    g = cb.ModelCalcer()
    g.load_from_dict(model)
    g.enable_gpu_evaluation(0)
    kernels = g.evaluator().describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)
    assert kernels["evaluate"] == kernel, kernels
    bins = o.binarize(x)
    assert bins.max() > 127
    np.testing.assert_array_equal(g.quantize_flat(x), bins)
    np.testing.assert_array_equal(g.calc_leaf_indexes_flat(x), o.leaf_indexes(x))
    np.testing.assert_allclose(g.calc_flat(x), o.calc(x), rtol=RTOL, atol=ATOL)
    total = len(model["tree_sizes"])
    for begin, end in ((0, 1), (1, 2), (0, 17), (3, 3), (total // 2, total)):
        np.testing.assert_allclose(g.calc_flat(x, tree_start=begin, tree_end=end),
                                   o.calc(x, tree_start=begin, tree_end=end), rtol=RTOL, atol=ATOL,
                                   err_msg="trees %d..%d" % (begin, end))
