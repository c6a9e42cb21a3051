"""Small batches on the register-resident kernels: slices of the trees on workgroups of their own. Needs an MI355X.

The reference special-cases single documents (c_api.cpp:383-384, cpu/evaluator_impl.cpp:417-460); here a
batch too small to fill the chip is spread by cutting the trees into slices whose raw sums a second kernel
adds in slice order. Bar: 1e-9 relative / 1e-12 absolute against the oracle, the same bits on every call,
and the bit-exact single pass again from the size on where slicing stops.
"""
import numpy as np
import pytest

import catboost_amd as cb
from catboost_amd import synthetic as syn
from oracle.cbm_reader import read_cbm
from oracle.oracle import OracleModel

pytestmark = [pytest.mark.gpu, pytest.mark.small_batch]


@pytest.mark.parametrize("cfg,trees", [("C2", 1000), ("C1", 200), ("C3", 300), ("C2", 37)])
def test_small_batches_through_tree_slices(cfg, trees):
    import torch

    model, info = syn.build_model(cfg, trees=trees)
    model.set_scale_and_bias(0.25, [0.5 + k for k in range(info["dim"])])
    model.enable_gpu_evaluation(0)
    ev = model.evaluator()
    oracle = OracleModel(read_cbm(model.save_to_buffer()))
    dim = info["dim"]
    x = syn.device_features(info, 530_000)  # more than 256 workgroups of eight 256-document blocks
    host = x.cpu().numpy()
    for docs in (1, 256, 4096, 65_536):
        part = x[:docs].contiguous()
        feats = ev.features(cb.LAYOUT_FLAT_ROWS, part.data_ptr(), part.shape[1])
        a = torch.full((docs * dim,), -1.0, dtype=torch.float64, device="cuda:0")
        b = torch.full((docs * dim,), -2.0, dtype=torch.float64, device="cuda:0")
        torch.cuda.synchronize()
        ev.eval_data(feats, docs, a.data_ptr())
        ev.eval_data(feats, docs, b.data_ptr())
        torch.cuda.synchronize()
        assert torch.equal(a, b), "two calls differ"
        expected = oracle.calc(host[:docs], threads=8)
        np.testing.assert_allclose(a.cpu().numpy(), expected, rtol=1e-9, atol=1e-12)
        # the host entry point takes the same path
        np.testing.assert_array_equal(model.calc_flat(host[:min(docs, 5000)]), a.cpu().numpy()[:min(docs, 5000) * dim])
    # a batch that fills the chip goes the single pass again: the CPU evaluator's bits (one-dimensional models)
    docs = host.shape[0]
    out = torch.zeros(docs * dim, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]), docs, out.data_ptr())
    torch.cuda.synchronize()
    expected = oracle.calc(host, threads=8)
    if dim == 1:
        np.testing.assert_array_equal(out.cpu().numpy(), expected)
    else:
        np.testing.assert_allclose(out.cpu().numpy(), expected, rtol=1e-9, atol=1e-12)


def test_small_batch_slicing_switched_off_through_the_api():
    """CbHipSetSmallBatchSlicing / CbHipEvaluatorSetSmallBatchSlicing: with the slices off a small batch is summed in
    one pass in tree order, the CPU evaluator's bits, through the model handle's host calls and the evaluator's
    device calls; switched on again the slices are back."""
    import torch

    model, info = syn.build_model("C2", trees=200)
    model.enable_gpu_evaluation(0)
    oracle = OracleModel(read_cbm(model.save_to_buffer()))
    x = syn.device_features(info, 3000)
    host = x.cpu().numpy()
    expected = oracle.calc(host, threads=8)
    ev = model.evaluator()
    assert "slices" in ev.describe_kernels(cb.LAYOUT_FLAT_ROWS, 3000)["evaluate"]
    sliced = model.calc_flat(host)
    np.testing.assert_allclose(sliced, expected, rtol=1e-9, atol=1e-12)
    model.set_small_batch_slicing(False)
    assert "slices" not in str(ev.describe_kernels(cb.LAYOUT_FLAT_ROWS, 3000))   # (this model: the fused kernel at any size)
    np.testing.assert_array_equal(model.calc_flat(host), expected)
    out = torch.zeros(3000, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    ev.eval_data(ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1]), 3000, out.data_ptr())
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), expected)
    # the setting survives a new evaluator of the handle (a feature layout rebuilds it)
    model.set_feature_layout(None, None, None)
    np.testing.assert_array_equal(model.calc_flat(host), expected)
    ev = model.evaluator()
    ev.set_small_batch_slicing(True)
    assert "slices" in ev.describe_kernels(cb.LAYOUT_FLAT_ROWS, 3000)["evaluate"]
    np.testing.assert_array_equal(model.calc_flat(host), sliced)
