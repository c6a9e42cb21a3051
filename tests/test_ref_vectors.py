"""Vectors produced by the reference's own standalone evaluator (see
tests/golden/make_ref_vectors.py): the oracle must reproduce them bit for bit, the HIP evaluator
within the prediction tolerance. The models include a 300-border (two-bucket) feature, depth 0-10
trees, scale/bias, and documents with NaN, +-inf and values exactly on borders."""
import os

import numpy as np
import pytest

from oracle.cbm_reader import read_cbm
from oracle.oracle import OracleModel


def _cases(golden_dir):
    data = np.load(os.path.join(golden_dir, "ref_standalone_vectors.npz"), allow_pickle=False)
    i = 0
    while "model_%d" % i in data:
        yield data["model_%d" % i].tobytes(), data["docs_%d" % i], data["expected_%d" % i]
        i += 1


def test_oracle_reproduces_reference_standalone_evaluator(golden_dir):
    n = 0
    for cbm, docs, expected in _cases(golden_dir):
        o = OracleModel(read_cbm(cbm))
        np.testing.assert_array_equal(o.calc(docs), expected)
        bf, _ = o.bruteforce(docs)
        np.testing.assert_allclose(bf, expected, rtol=1e-13, atol=1e-13)
        n += 1
    assert n == 3


@pytest.mark.both_batch_modes
@pytest.mark.gpu
def test_hip_evaluator_reproduces_reference_standalone_evaluator(golden_dir):
    import catboost_amd as cb

    for cbm, docs, expected in _cases(golden_dir):
        m = cb.ModelCalcer(buffer=cbm)
        np.testing.assert_allclose(m.calc_flat(docs), expected, rtol=1e-9, atol=1e-12)
        o = OracleModel(read_cbm(cbm))
        np.testing.assert_array_equal(m.quantize_flat(docs), o.binarize(docs))
        np.testing.assert_array_equal(m.calc_leaf_indexes_flat(docs), o.leaf_indexes(docs))
