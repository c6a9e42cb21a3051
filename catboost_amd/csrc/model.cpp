#include "model.h"

#include <algorithm>
#include <cmath>
#include <limits>
#include <numeric>
#include <tuple>

namespace cbamd {

// TModelSplit ordering, catboost/libs/model/split.h:69-87 with the per-kind orderings of
// online_ctr.h:49-51 (float: feature, border) and :84-86 (one-hot: cat feature, value).
bool TModelSplit::operator<(const TModelSplit& o) const {
    if (Type != o.Type) {
        return static_cast<int>(Type) < static_cast<int>(o.Type);
    }
    if (Type == ESplitType::FloatFeature || Type == ESplitType::OnlineCtr) {
        return std::tie(FeatureIndex, Border) < std::tie(o.FeatureIndex, o.Border);
    }
    return std::tie(FeatureIndex, Value) < std::tie(o.FeatureIndex, o.Value);
}

bool TModelSplit::operator==(const TModelSplit& o) const {
    if (Type != o.Type) {
        return false;
    }
    if (Type == ESplitType::FloatFeature || Type == ESplitType::OnlineCtr) {
        return FeatureIndex == o.FeatureIndex && Border == o.Border;
    }
    return FeatureIndex == o.FeatureIndex && Value == o.Value;
}

size_t TModelTrees::GetFlatFeatureVectorExpectedSize() const {
    int result = 0;
    if (!CatFeatures.empty()) {
        result = std::max(result, CatFeatures.back().FlatIndex + 1);
    }
    if (!FloatFeatures.empty()) {
        result = std::max(result, FloatFeatures.back().FlatIndex + 1);
    }
    return static_cast<size_t>(result);
}

bool TModelTrees::IsZeroBias() const {  // scale_and_bias.h:37-44
    for (double b : Bias) {
        if (b != 0.0) {
            return false;
        }
    }
    return true;
}

bool TModelTrees::IsIdentityScaleAndBias() const {  // scale_and_bias.h:46-48
    return Scale == 1.0 && IsZeroBias();
}

void TModelTrees::SetScaleAndBias(double scale, const std::vector<double>& biasIn) {
    CBAMD_ENSURE(std::isfinite(scale), "Invalid scale " + std::to_string(scale));
    std::vector<double> bias = biasIn;
    for (size_t i = 0; i < bias.size(); ++i) {
        CBAMD_ENSURE(std::isfinite(bias[i]), "Invalid bias[" + std::to_string(i) + "] : " + std::to_string(bias[i]));
    }
    if (bias.empty()) {
        bias.resize(ApproxDimension, 0.0);
    }
    CBAMD_ENSURE(
        static_cast<size_t>(ApproxDimension) == bias.size(),
        "Inappropraite dimension of bias, should be " + std::to_string(ApproxDimension) + " found " + std::to_string(bias.size()));
    Scale = scale;
    Bias = bias;
}

void TModelTrees::AddBinTree(const std::vector<int>& binSplits) {
    TreeSplits.insert(TreeSplits.end(), binSplits.begin(), binSplits.end());
    if (TreeStartOffsets.empty()) {
        TreeStartOffsets.push_back(0);
    } else {
        TreeStartOffsets.push_back(TreeStartOffsets.back() + TreeSizes.back());
    }
    TreeSizes.push_back(static_cast<int>(binSplits.size()));
}

void TModelTrees::UpdateRuntimeData() {
    CBAMD_ENSURE(ApproxDimension >= 1, "approx dimension must be positive");
    if (Bias.empty()) {
        Bias.assign(ApproxDimension, 0.0);
    }
    CBAMD_ENSURE(Bias.size() == static_cast<size_t>(ApproxDimension), "Inappropraite dimension of bias");
    CBAMD_ENSURE(TreeSizes.size() == TreeStartOffsets.size(), "tree sizes and tree start offsets differ in length");

    // CalcForApplyData, model.cpp:431-449
    UsedFloatFeaturesCount = 0;
    UsedCatFeaturesCount = 0;
    MinimalSufficientFloatFeaturesVectorSize = 0;
    MinimalSufficientCatFeaturesVectorSize = 0;
    for (const auto& f : FloatFeatures) {
        if (f.UsedInModel()) {
            ++UsedFloatFeaturesCount;
            MinimalSufficientFloatFeaturesVectorSize = static_cast<size_t>(f.Index) + 1;
        }
    }
    for (const auto& c : CatFeatures) {
        if (c.UsedInModel) {
            ++UsedCatFeaturesCount;
            MinimalSufficientCatFeaturesVectorSize = static_cast<size_t>(c.Index) + 1;
        }
    }

    // CalcBinFeatures, model.cpp:471-577: one binary feature per border / one-hot value; a
    // feature with n borders occupies ceil(n / 254) consecutive buckets.
    struct TFeatureSplitId {
        uint32_t FeatureIdx;
        uint32_t SplitIdx;
    };
    std::vector<TFeatureSplitId> splitIds;
    BinFeatures.clear();
    uint32_t buckets = 0;
    for (const auto& f : FloatFeatures) {
        if (!f.UsedInModel()) {
            continue;
        }
        for (size_t borderId = 0; borderId < f.Borders.size(); ++borderId) {
            BinFeatures.push_back(TModelSplit::Float(f.Index, f.Borders[borderId]));
            splitIds.push_back({buckets + static_cast<uint32_t>(borderId / kMaxValuesPerBin),
                                static_cast<uint32_t>(borderId % kMaxValuesPerBin) + 1});
        }
        buckets += static_cast<uint32_t>((f.Borders.size() + kMaxValuesPerBin - 1) / kMaxValuesPerBin);
    }
    for (const auto& oh : OneHotFeatures) {
        for (size_t valueId = 0; valueId < oh.Values.size(); ++valueId) {
            BinFeatures.push_back(TModelSplit::OneHot(oh.CatFeatureIndex, oh.Values[valueId]));
            splitIds.push_back({buckets + static_cast<uint32_t>(valueId / kMaxValuesPerBin),
                                static_cast<uint32_t>(valueId % kMaxValuesPerBin) + 1});
        }
        buckets += static_cast<uint32_t>((oh.Values.size() + kMaxValuesPerBin - 1) / kMaxValuesPerBin);
    }
    CtrFirstBucket = buckets;
    for (size_t i = 0; i < CtrFeatures.size(); ++i) {
        const auto& borders = CtrFeatures[i].Borders;
        for (size_t borderId = 0; borderId < borders.size(); ++borderId) {
            BinFeatures.push_back(TModelSplit::Ctr(static_cast<int>(i), borders[borderId]));
            splitIds.push_back({buckets + static_cast<uint32_t>(borderId / kMaxValuesPerBin),
                                static_cast<uint32_t>(borderId % kMaxValuesPerBin) + 1});
        }
        buckets += static_cast<uint32_t>((borders.size() + kMaxValuesPerBin - 1) / kMaxValuesPerBin);
    }
    EffectiveBinFeaturesBucketCount = buckets;

    RepackedBins.clear();
    RepackedBins.reserve(TreeSplits.size());
    if (splitIds.empty() && !TreeSplits.empty()) {
        // trees without any condition; only non-symmetric models may look like this
        for (int s : TreeSplits) {
            CBAMD_ENSURE(s == 0, "expected 0 as empty nodes marker");
        }
        CBAMD_ENSURE(!IsOblivious(),
                     "Expected asymmetric trees: Split ids present and are zeroes, but there is no actual splits in model");
        RepackedBins.resize(TreeSplits.size());
    } else {
        for (int s : TreeSplits) {
            CBAMD_ENSURE(s >= 0 && static_cast<size_t>(s) < splitIds.size(), "tree split index out of range");
            const auto& id = splitIds[s];
            CBAMD_ENSURE(id.FeatureIdx <= 0xffff, "Too many features in model, ask catboost team for support");
            TRepackedBin rb;
            rb.FeatureIndex = static_cast<uint16_t>(id.FeatureIdx);
            if (BinFeatures[s].Type != ESplitType::OneHotFeature) {
                rb.SplitIdx = static_cast<uint8_t>(id.SplitIdx);
            } else {
                rb.XorMask = static_cast<uint8_t>((~id.SplitIdx) & 0xff);
                rb.SplitIdx = 0xff;
            }
            RepackedBins.push_back(rb);
        }
    }

    // CalcFirstLeafOffsets, model.cpp:586-624
    TreeFirstLeafOffsets.assign(TreeSizes.size(), 0);
    if (IsOblivious()) {
        size_t cur = 0;
        for (size_t t = 0; t < TreeSizes.size(); ++t) {
            CBAMD_ENSURE(TreeSizes[t] >= 0 && TreeSizes[t] < 31, "unsupported tree depth");
            CBAMD_ENSURE(TreeStartOffsets[t] >= 0 &&
                             static_cast<size_t>(TreeStartOffsets[t]) + TreeSizes[t] <= TreeSplits.size(),
                         "tree splits out of range");
            TreeFirstLeafOffsets[t] = cur;
            cur += (static_cast<size_t>(1) << TreeSizes[t]) * ApproxDimension;
        }
        CBAMD_ENSURE(cur <= LeafValues.size(), "leaf values vector is shorter than the trees need");
    } else {
        CBAMD_ENSURE(NonSymmetricStepNodes.size() == NonSymmetricNodeIdToLeafId.size() &&
                         NonSymmetricStepNodes.size() == TreeSplits.size(),
                     "non-symmetric node tables differ in length");
        for (size_t t = 0; t < TreeSizes.size(); ++t) {
            CBAMD_ENSURE(TreeStartOffsets[t] >= 0 && TreeSizes[t] > 0 &&
                             static_cast<size_t>(TreeStartOffsets[t]) + static_cast<size_t>(TreeSizes[t]) <=
                                 NonSymmetricStepNodes.size(),
                         "tree nodes out of range");
            const int begin = TreeStartOffsets[t];
            const int end = begin + TreeSizes[t];
            uint32_t minLeaf = std::numeric_limits<uint32_t>::max();
            for (int n = begin; n < end; ++n) {
                const auto& node = NonSymmetricStepNodes[n];
                // every step must stay inside its tree
                CBAMD_ENSURE(n + node.LeftSubtreeDiff < end && n + node.RightSubtreeDiff < end,
                             "non-symmetric step leaves its tree");
                if (node.LeftSubtreeDiff == 0 || node.RightSubtreeDiff == 0) {
                    const uint32_t leaf = NonSymmetricNodeIdToLeafId[n];
                    CBAMD_ENSURE(leaf % ApproxDimension == 0, "Expect that leaf values are aligned.");
                    CBAMD_ENSURE(static_cast<size_t>(leaf) + ApproxDimension <= LeafValues.size(),
                                 "leaf value index out of range");
                    minLeaf = std::min(minLeaf, leaf);
                }
            }
            CBAMD_ENSURE(minLeaf != std::numeric_limits<uint32_t>::max(), "tree has no terminal node");
            TreeFirstLeafOffsets[t] = minLeaf;
        }
    }
}

void TModelTrees::ConvertObliviousToAsymmetric() {
    if (!IsOblivious()) {
        return;
    }
    std::vector<int> treeSplits, treeSizes, treeStartOffsets;
    std::vector<TNonSymmetricTreeStepNode> stepNodes;
    std::vector<uint32_t> nodeIdToLeafId;
    size_t leafStartOffset = 0;
    for (size_t treeId = 0; treeId < TreeSizes.size(); ++treeId) {
        size_t treeSize = 0;
        treeStartOffsets.push_back(static_cast<int>(treeSplits.size()));
        for (int depth = 0; depth < TreeSizes[treeId]; ++depth) {
            const int split = TreeSplits[TreeStartOffsets[treeId] + TreeSizes[treeId] - 1 - depth];
            for (size_t cloneId = 0; cloneId < (static_cast<size_t>(1) << depth); ++cloneId) {
                treeSplits.push_back(split);
                nodeIdToLeafId.push_back(std::numeric_limits<uint32_t>::max());
                stepNodes.push_back({static_cast<uint16_t>(treeSize + 1), static_cast<uint16_t>(treeSize + 2)});
                ++treeSize;
            }
        }
        for (size_t cloneId = 0; cloneId < (static_cast<size_t>(1) << TreeSizes[treeId]); ++cloneId) {
            treeSplits.push_back(0);
            nodeIdToLeafId.push_back(static_cast<uint32_t>((leafStartOffset + cloneId) * ApproxDimension));
            stepNodes.push_back({0, 0});
            ++treeSize;
        }
        leafStartOffset += static_cast<size_t>(1) << TreeSizes[treeId];
        treeSizes.push_back(static_cast<int>(treeSize));
    }
    TreeSplits = std::move(treeSplits);
    TreeSizes = std::move(treeSizes);
    TreeStartOffsets = std::move(treeStartOffsets);
    NonSymmetricStepNodes = std::move(stepNodes);
    NonSymmetricNodeIdToLeafId = std::move(nodeIdToLeafId);
    UpdateRuntimeData();
}

void TFullModel::EnsureSupported() const {
    for (const auto& part : ModelPartIds) {
        CBAMD_ENSURE(part == "static_provider_v1",
                     "Model part '" + std::string(part.c_str()) + "' (text or embedding data) is not supported by the HIP evaluator");
    }
    // every CTR of the model needs its table of learned statistics (ICtrProvider::HasNeededCtrs,
    // static_ctr_provider.cpp:133-140) and refers to features the model has
    for (const auto& feature : Trees.CtrFeatures) {
        const TCtrValueTable* table = FindCtrTable(feature.Ctr.Base);
        CBAMD_ENSURE(table != nullptr, "Model has a CTR feature without its table of learned statistics");
        CBAMD_ENSURE(table->IndexHashRaw.size() % 12 == 0 && table->IndexHashRaw.size() >= 12 &&
                         ((table->IndexHashRaw.size() / 12) & (table->IndexHashRaw.size() / 12 - 1)) == 0,
                     "Dense hash view must have 2^k buckets");
    }
    CBAMD_ENSURE(Trees.TextFeatureCount == 0 && Trees.EstimatedFeatureCount == 0,
                 "Model contains text features, HIP evaluation impossible");
    CBAMD_ENSURE(Trees.EmbeddingFeatureCount == 0, "Model contains embedding features, HIP evaluation impossible");
}

namespace {

int RemapOne(bool defined, const std::vector<uint32_t>& list, int position, const char* what) {
    if (!defined) {
        return position;
    }
    CBAMD_ENSURE(position >= 0 && static_cast<size_t>(position) < list.size(),
                 "feature layout: " + what + " has no entry for position " + std::to_string(position));
    CBAMD_ENSURE(list[position] <= 0x7fffffffu, "feature layout: position is too large");
    return static_cast<int>(list[position]);
}

}  // namespace

TFeaturePosition TFeatureLayout::Remap(const TFloatFeature& feature) const {
    TFeaturePosition p;
    p.Index = RemapOne(HasFloatFeatureIndexes, FloatFeatureIndexes, feature.Index, "FloatFeatureIndexes");
    p.FlatIndex = RemapOne(HasFlatIndexes, FlatIndexes, feature.FlatIndex, "FlatIndexes");
    return p;
}

TFeaturePosition TFeatureLayout::Remap(const TCatFeature& feature) const {
    TFeaturePosition p;
    p.Index = RemapOne(HasCatFeatureIndexes, CatFeatureIndexes, feature.Index, "CatFeatureIndexes");
    p.FlatIndex = RemapOne(HasFlatIndexes, FlatIndexes, feature.FlatIndex, "FlatIndexes");
    return p;
}

const TCtrValueTable* TFullModel::FindCtrTable(const TModelCtrBase& base) const {
    for (const auto& table : CtrTables) {
        if (table.ModelCtrBase == base) {
            return &table;
        }
    }
    return nullptr;
}

std::vector<std::string> TFullModel::GetUsedFeaturesNames() const {
    std::vector<std::pair<int, std::string>> items;
    for (const auto& f : Trees.FloatFeatures) {
        items.emplace_back(f.FlatIndex, f.FeatureId.empty() ? std::to_string(f.FlatIndex) : f.FeatureId);
    }
    for (const auto& c : Trees.CatFeatures) {
        items.emplace_back(c.FlatIndex, c.FeatureId.empty() ? std::to_string(c.FlatIndex) : c.FeatureId);
    }
    std::stable_sort(items.begin(), items.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    std::vector<std::string> result;
    for (auto& it : items) {
        result.push_back(std::move(it.second));
    }
    return result;
}

}  // namespace cbamd
