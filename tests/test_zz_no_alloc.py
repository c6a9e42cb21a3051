"""CbHipEvalDataNoAlloc, the entry point that allocates nothing, against CbHipEvalData. Needs an MI355X.

Both run the same binarize and evaluate kernels; one keeps the bins in the evaluator's scratch buffer,
the other in the library's fixed device array. Bar: bit for bit, and against the oracle within
1e-9 relative / 1e-12 absolute. Two calls in a row, the second with fewer documents, so that what the
first call left in the array sits behind (and under) the second call's bins.
"""
import numpy as np
import pytest

import catboost_amd as cb
from catboost_amd import synthetic as syn
from oracle.cbm_reader import read_cbm
from oracle.oracle import OracleModel

pytestmark = pytest.mark.gpu

NO_ALLOC_BYTES = 32 << 20


def _run_both(ev, feats, docs, dim, tree_range=(0, None)):
    import torch

    a = torch.full((docs * dim,), -7.0, dtype=torch.float64, device="cuda:0")
    b = torch.full((docs * dim,), -9.0, dtype=torch.float64, device="cuda:0")
    torch.cuda.synchronize()
    ev.eval_data_no_alloc(feats, docs, a.data_ptr(), tree_start=tree_range[0], tree_end=tree_range[1])
    ev.synchronize()
    ev.eval_data(feats, docs, b.data_ptr(), tree_start=tree_range[0], tree_end=tree_range[1])
    torch.cuda.synchronize()
    return a, b


@pytest.mark.parametrize("cfg,trees,fused", [("C2", 60, "0"), ("C2", 60, "1"), ("C3", 40, "1"), ("C4", 30, "1"), ("C5", 20, "1")])
def test_no_alloc_entry_point_equals_eval_data(cfg, trees, fused, monkeypatch):
    import torch

    # C2 has a fused kernel (no bins in memory at all); CATBOOST_AMD_FUSED=0 keeps it on the two launches
    # whose bins sit in the fixed array, as the other models' do
    monkeypatch.setenv("CATBOOST_AMD_FUSED", fused)
    model, info = syn.build_model(cfg, trees=trees)
    model.enable_gpu_evaluation(0)
    ev = model.evaluator()
    oracle = OracleModel(read_cbm(model.save_to_buffer()))
    dim = info["dim"]
    first_docs = 7001
    assert ev.quantized_bytes(first_docs) <= NO_ALLOC_BYTES
    x = syn.device_features(info, first_docs)
    for docs in (first_docs, 1300):  # the second call is smaller: the first call's bins stay behind it
        part = x[:docs].contiguous()
        feats = ev.features(cb.LAYOUT_FLAT_ROWS, part.data_ptr(), part.shape[1])
        got, expected = _run_both(ev, feats, docs, dim)
        assert torch.equal(got, expected), (cfg, docs)
        np.testing.assert_allclose(got.cpu().numpy(), oracle.calc(part.cpu().numpy(), threads=8), rtol=1e-9, atol=1e-12)
    # a tree sub-range goes the same way
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    got, expected = _run_both(ev, feats, 900, dim, tree_range=(3, trees - 2))
    assert torch.equal(got, expected)


def test_no_alloc_entry_point_refuses_batches_beyond_its_buffer(monkeypatch):
    import torch

    monkeypatch.setenv("CATBOOST_AMD_FUSED", "0")
    model, info = syn.build_model("C2", trees=5)
    model.enable_gpu_evaluation(0)
    ev = model.evaluator()
    per_block = ev.quantized_bytes(256)
    max_docs = NO_ALLOC_BYTES // per_block * 256
    assert ev.quantized_bytes(max_docs) <= NO_ALLOC_BYTES < ev.quantized_bytes(max_docs + 1)
    x = syn.device_features(info, max_docs)
    out = torch.zeros(max_docs + 1, dtype=torch.float64, device="cuda:0")
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    with pytest.raises(cb.CatBoostError, match="at most %d documents" % max_docs):
        ev.eval_data_no_alloc(feats, max_docs + 1, out.data_ptr())
    # the largest batch that fits runs and equals the allocating entry point
    got, expected = _run_both(ev, feats, max_docs, 1)
    assert torch.equal(got, expected)


@pytest.mark.small_batch
def test_no_alloc_entry_point_under_the_default_switches():
    """With the library's default handling of small batches: a fused model's batch that is too large for the fixed
    buffer and smaller than the size from which CbHipEvalData itself launches the fused kernel (it must not be
    refused: the fused kernel needs no buffer), and a model of more than 64 trees whose small batches
    CbHipEvalData cuts into slices of the trees while the entry point that allocates nothing makes the single
    pass in tree order: both agree with the oracle, the single pass bit for bit."""
    import torch

    model, info = syn.build_model("C2", trees=96)
    model.enable_gpu_evaluation(0)
    ev = model.evaluator()
    oracle = OracleModel(read_cbm(model.save_to_buffer()))
    assert "fused" in ev.describe_kernels(cb.LAYOUT_FLAT_ROWS, 1 << 20)
    per_block = ev.quantized_bytes(256)
    max_docs = NO_ALLOC_BYTES // per_block * 256
    docs = max_docs + 777
    assert "fused" not in ev.describe_kernels(cb.LAYOUT_FLAT_ROWS, docs)      # CbHipEvalData: two launches at this size
    x = syn.device_features(info, docs)
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, x.data_ptr(), x.shape[1])
    got, expected = _run_both(ev, feats, docs, 1)
    sample = np.sort(np.random.default_rng(5).choice(docs, 3000, replace=False))
    want = oracle.calc(x[torch.from_numpy(sample).to("cuda:0")].cpu().numpy(), threads=8)
    np.testing.assert_array_equal(got.cpu().numpy()[sample], want)               # fused kernel: tree order
    np.testing.assert_allclose(expected.cpu().numpy()[sample], want, rtol=1e-9, atol=1e-12)
    # a small batch: slices in CbHipEvalData, one pass here
    small = 3000
    assert "slices" in ev.describe_kernels(cb.LAYOUT_FLAT_ROWS, small).get("evaluate", "")
    part = x[:small].contiguous()
    feats = ev.features(cb.LAYOUT_FLAT_ROWS, part.data_ptr(), part.shape[1])
    got, expected = _run_both(ev, feats, small, 1)
    want = oracle.calc(part.cpu().numpy(), threads=8)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    np.testing.assert_allclose(expected.cpu().numpy(), want, rtol=1e-9, atol=1e-12)
