"""Seeded synthetic models and documents of the five evaluation workloads.

  C1  oblivious RMSE regressor: 200 trees, depth 6, 50 float features, 128 candidate borders per
      feature at N(0,1) quantiles, no NaN, 1M docs N(0,1).
  C2  oblivious regressor: 1000 trees, depth 8, 200 float features (half N(0,1), half
      log-normal(0,1)) with 254 candidate borders at empirical quantiles, 5 % NaN per feature,
      NanMode=Min (HasNans, AsFalse), 4M docs.
  C3  oblivious MultiClass, 10 classes: 2000 trees, depth 6, 100 float features uniform(-3,3)
      with 64 borders, 2M docs.
  C4  non-symmetric regressor: 500 trees, depth <= 10, a node at depth < 10 is a leaf with
      probability 0.15; 300 float features with 254 borders, 2 % NaN (HasNans, AsFalse), 4M docs.
  C5  oblivious binary-logloss model with one-hot splits: 5000 trees, depth 8, 1000 float
      features (254 borders) + 16 categorical features of cardinality 2..10 whose integer ids are
      hashed with the cat-feature hash; a split first picks one of the 1016 features uniformly,
      then a border / category uniformly (so about 1.6 % of the splits are one-hot); 10M docs.

  C2B C2 over 20 features instead of 200, so that about 200 borders of every feature are used: bins
      above 127 (the 8-bit compare of the mixed kernels). Not one of the baseline workloads.

  C2W C2 over 400 features and 2M docs: more buckets than the register-resident kernels hold, the LDS tile
      kernel's case. Not one of the baseline workloads.

  C2N C2 over 90 features: few enough buckets for the 96-register kernel shape (four waves per SIMD), which the
      CATBOOST_AMD_REG_MIN_BUCKETS switch can trade for the 200-register shape (two waves per SIMD) on the
      same model. Not one of the baseline workloads.

Every split is (feature, border) drawn uniformly; models go through the builder, so only the
borders that some split uses survive. Leaf values are N(0, sigma).
"""
import numpy as np
from scipy.stats import norm

from . import SPLIT_DTYPE, ModelCalcer, integer_cat_feature_hash

CONFIGS = {
    "C1": dict(kind="oblivious", trees=200, depth=6, floats=50, borders=128, dim=1, leaf_sigma=0.01, docs=1_000_000,
               dist="normal", nan_rate=0.0),
    "C2": dict(kind="oblivious", trees=1000, depth=8, floats=200, borders=254, dim=1, leaf_sigma=0.005,
               docs=4_000_000, dist="normal_lognormal", nan_rate=0.05),
    "C2B": dict(kind="oblivious", trees=1000, depth=8, floats=20, borders=254, dim=1, leaf_sigma=0.005,
                docs=4_000_000, dist="normal_lognormal", nan_rate=0.05),
    "C2W": dict(kind="oblivious", trees=1000, depth=8, floats=400, borders=254, dim=1, leaf_sigma=0.005,
                docs=2_000_000, dist="normal_lognormal", nan_rate=0.05),
    "C2N": dict(kind="oblivious", trees=1000, depth=8, floats=90, borders=254, dim=1, leaf_sigma=0.005,
                docs=4_000_000, dist="normal_lognormal", nan_rate=0.05),
    "C3": dict(kind="oblivious", trees=2000, depth=6, floats=100, borders=64, dim=10, leaf_sigma=0.01,
               docs=2_000_000, dist="uniform3", nan_rate=0.0),
    "C4": dict(kind="nonsymmetric", trees=500, depth=10, floats=300, borders=254, dim=1, leaf_sigma=0.01,
               docs=4_000_000, dist="normal", nan_rate=0.02, leaf_prob=0.15),
    "C5": dict(kind="oblivious", trees=5000, depth=8, floats=1000, borders=254, dim=1, leaf_sigma=0.01,
               docs=10_000_000, dist="normal", nan_rate=0.0, cats=16),
}


def _candidate_borders(cfg, rng):
    """Per float feature: sorted unique fp32 candidate borders."""
    nf, nb = cfg["floats"], cfg["borders"]
    q = (np.arange(nb) + 1.0) / (nb + 1.0)
    out = []
    for f in range(nf):
        if cfg["dist"] == "normal":
            b = norm.ppf(q)
        elif cfg["dist"] == "uniform3":
            b = -3.0 + 6.0 * q
        else:  # empirical quantiles of a seeded sample of the feature's own distribution
            sample = rng.standard_normal(20000)
            if f >= nf // 2:
                sample = np.exp(sample)
            b = np.quantile(sample, q)
        out.append(np.unique(b.astype(np.float32)))
    return out


def _features(cfg):
    nan = cfg["nan_rate"] > 0
    floats = [dict(index=i, flat_index=i, has_nans=nan, nan_treatment=1 if nan else 0) for i in range(cfg["floats"])]
    cats = [dict(index=i, flat_index=cfg["floats"] + i, used=True) for i in range(cfg.get("cats", 0))]
    return floats, cats


def _cat_cardinalities(cfg, rng):
    if "cat_cardinality" in cfg:   # every categorical feature with that many values (up to 254 fit a one-hot bucket)
        return np.full(cfg.get("cats", 0), cfg["cat_cardinality"], dtype=np.int64)
    return rng.integers(2, 11, size=cfg.get("cats", 0))


def _draw_splits(cfg, rng, count, cands, cat_hashes):
    """`count` random splits as a SPLIT_DTYPE array."""
    nf, nc = cfg["floats"], cfg.get("cats", 0)
    out = np.zeros(count, dtype=SPLIT_DTYPE)
    feat = rng.integers(0, nf + nc, size=count)
    u = rng.random(size=count)
    sizes = np.array([len(c) for c in cands] + [len(h) for h in cat_hashes])
    pick = np.minimum((u * sizes[feat]).astype(np.int64), sizes[feat] - 1)
    is_cat = feat >= nf
    out["Type"] = np.where(is_cat, 2, 0)
    out["FeatureIndex"] = np.where(is_cat, feat - nf, feat)
    # gather borders / values
    offs = np.concatenate([[0], np.cumsum(sizes)])
    flat_borders = np.concatenate([c.astype(np.float32) for c in cands] + [np.zeros(len(h), np.float32) for h in cat_hashes])
    flat_values = np.concatenate([np.zeros(len(c), np.int32) for c in cands] + [np.asarray(h, np.int32) for h in cat_hashes])
    at = offs[feat] + pick
    out["Border"] = np.where(is_cat, 0.0, flat_borders[at])
    out["Value"] = np.where(is_cat, flat_values[at], 0)
    return out


def build_model(name, seed=0, trees=None):
    """Builds config `name` through the library's model builder; returns (ModelCalcer, info)."""
    cfg = dict(CONFIGS[name])
    if trees is not None:
        cfg["trees"] = trees
    rng = np.random.default_rng([seed, sum(ord(c) for c in name)])
    cands = _candidate_borders(cfg, rng)
    card = _cat_cardinalities(cfg, rng)
    cat_hashes = [[integer_cat_feature_hash(v) for v in range(int(c))] for c in card]
    floats, cats = _features(cfg)
    dim = cfg["dim"]
    model = ModelCalcer()
    if cfg["kind"] == "oblivious":
        depths = np.full(cfg["trees"], cfg["depth"], dtype=np.int32)
        splits = _draw_splits(cfg, rng, int(depths.sum()), cands, cat_hashes)
        leaves = rng.normal(0.0, cfg["leaf_sigma"], size=int((1 << cfg["depth"]) * dim * cfg["trees"]))
        model.build_oblivious_packed(floats, cats, dim, depths, splits, leaves)
    else:
        # pre-order node arrays; a node at depth < max is a leaf with probability leaf_prob
        offsets, is_split, left, right, depth_of = [0], [], [], [], []
        for _ in range(cfg["trees"]):
            base = len(is_split)
            stack = [(0, -1, 0)]  # (depth, parent position, which child)
            while stack:
                depth, parent, side = stack.pop()
                pos = len(is_split)
                if parent >= 0:
                    (left if side == 0 else right)[parent] = pos - base
                leaf = depth >= cfg["depth"] or rng.random() < cfg["leaf_prob"]
                is_split.append(0 if leaf else 1)
                left.append(0)
                right.append(0)
                depth_of.append(depth)
                if not leaf:
                    stack.append((depth + 1, pos, 1))
                    stack.append((depth + 1, pos, 0))
            offsets.append(len(is_split))
        n = len(is_split)
        is_split = np.asarray(is_split, np.int32)
        splits = _draw_splits(cfg, rng, n, cands, cat_hashes)
        value_off = np.cumsum(1 - is_split) * dim - dim
        value_off[is_split == 1] = 0
        values = rng.normal(0.0, cfg["leaf_sigma"], size=int((1 - is_split).sum()) * dim)
        model.build_non_symmetric_packed(floats, cats, dim, offsets, is_split, splits, left, right, value_off, values)
    info = dict(cfg, name=name, seed=seed, cat_cardinalities=[int(c) for c in card], cat_hashes=cat_hashes,
                flat_size=cfg["floats"] + cfg.get("cats", 0))
    return model, info


def host_features(info, doc_count, seed=1):
    """Flat row-major fp32 documents [doc_count, flat_size] on the host (numpy)."""
    rng = np.random.default_rng([seed, 77])
    nf = info["floats"]
    x = rng.standard_normal((doc_count, info["flat_size"]), dtype=np.float32)
    if info["dist"] == "uniform3":
        x[:, :nf] = rng.uniform(-3.0, 3.0, size=(doc_count, nf)).astype(np.float32)
    elif info["dist"] == "normal_lognormal":
        x[:, nf // 2:nf] = np.exp(x[:, nf // 2:nf])
    if info["nan_rate"] > 0:
        x[:, :nf][rng.random((doc_count, nf)) < info["nan_rate"]] = np.nan
    for c, hashes in enumerate(info["cat_hashes"]):
        ids = rng.integers(0, len(hashes), size=doc_count)
        x[:, nf + c] = np.asarray(hashes, np.int32)[ids].view(np.float32)
    return x


def device_features(info, doc_count, seed=1, device="cuda:0"):
    """Same distributions generated directly in device memory with torch (returns a tensor)."""
    import torch

    gen = torch.Generator(device=device)
    gen.manual_seed(1000 + seed)
    nf, width = info["floats"], info["flat_size"]
    x = torch.empty((doc_count, width), dtype=torch.float32, device=device)
    # generated in row chunks to bound temporaries
    step = max(1, (1 << 28) // max(width, 1))
    for b in range(0, doc_count, step):
        e = min(doc_count, b + step)
        part = x[b:e]
        if info["dist"] == "uniform3":
            part[:, :nf].uniform_(-3.0, 3.0, generator=gen)
        else:
            part[:, :nf].normal_(0.0, 1.0, generator=gen)
            if info["dist"] == "normal_lognormal":
                part[:, nf // 2:nf].exp_()
        if info["nan_rate"] > 0:
            mask = torch.rand((e - b, nf), device=device, generator=gen) < info["nan_rate"]
            part[:, :nf].masked_fill_(mask, float("nan"))
        for c, hashes in enumerate(info["cat_hashes"]):
            table = torch.tensor(hashes, dtype=torch.int32, device=device)
            ids = torch.randint(0, len(hashes), (e - b,), device=device, generator=gen)
            part[:, nf + c] = table[ids].view(torch.float32)
    return x
