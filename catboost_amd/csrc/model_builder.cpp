#include "model_builder.h"

#include <algorithm>
#include <limits>

namespace cbamd {

TCommonModelBuilderHelper::TCommonModelBuilderHelper(std::vector<TFloatFeature> allFloatFeatures,
                                                     std::vector<TCatFeature> allCategoricalFeatures,
                                                     int approxDimension)
    : ApproxDimension(approxDimension)
    , FloatFeatures(std::move(allFloatFeatures))
    , CatFeatures(std::move(allCategoricalFeatures))
{
    CBAMD_ENSURE(approxDimension >= 1, "approx dimension must be positive");
    // model_build_helper.cpp:24-49: features must come sorted by flat index
    CBAMD_ENSURE(std::is_sorted(FloatFeatures.begin(), FloatFeatures.end(),
                                [](const TFloatFeature& a, const TFloatFeature& b) { return a.FlatIndex < b.FlatIndex; }),
                 "Float features should be sorted");
    CBAMD_ENSURE(std::is_sorted(CatFeatures.begin(), CatFeatures.end(),
                                [](const TCatFeature& a, const TCatFeature& b) { return a.FlatIndex < b.FlatIndex; }),
                 "Cat features should be sorted");
    for (size_t i = 0; i < FloatFeatures.size(); ++i) {
        FloatFeaturesInternalIndexesMap[FloatFeatures[i].Index] = i;
    }
    for (size_t i = 0; i < CatFeatures.size(); ++i) {
        CatFeaturesInternalIndexesMap[CatFeatures[i].Index] = i;
    }
}

void TCommonModelBuilderHelper::ProcessSplitsSet(const std::set<TModelSplit>& splits, TModelTrees* trees) {
    // model_build_helper.cpp:100-126 + TModelTrees::ProcessSplitsSet, model.cpp:181-236
    trees->ApproxDimension = ApproxDimension;
    for (auto& f : FloatFeatures) {
        f.Borders.clear();
    }
    for (auto& c : CatFeatures) {
        c.UsedInModel = false;
    }
    trees->OneHotFeatures.clear();
    for (const auto& split : splits) {
        if (split.Type == ESplitType::FloatFeature) {
            auto it = FloatFeaturesInternalIndexesMap.find(split.FeatureIndex);
            CBAMD_ENSURE(it != FloatFeaturesInternalIndexesMap.end(), "split on an unknown float feature");
            FloatFeatures[it->second].Borders.push_back(split.Border);
        } else {
            CBAMD_ENSURE(split.Type == ESplitType::OneHotFeature, "unsupported split type");
            auto it = CatFeaturesInternalIndexesMap.find(split.FeatureIndex);
            CBAMD_ENSURE(it != CatFeaturesInternalIndexesMap.end(), "split on an unknown categorical feature");
            CatFeatures[it->second].UsedInModel = true;
            if (trees->OneHotFeatures.empty() || trees->OneHotFeatures.back().CatFeatureIndex != split.FeatureIndex) {
                trees->OneHotFeatures.emplace_back();
                trees->OneHotFeatures.back().CatFeatureIndex = split.FeatureIndex;
            }
            trees->OneHotFeatures.back().Values.push_back(split.Value);
        }
    }
    trees->FloatFeatures = FloatFeatures;
    trees->CatFeatures = CatFeatures;
    BinFeatureIndexes.clear();
    for (const auto& split : splits) {
        const int idx = static_cast<int>(BinFeatureIndexes.size());
        BinFeatureIndexes[split] = idx;
    }
}

void TObliviousTreeBuilder::AddTree(const std::vector<TModelSplit>& modelSplits, const double* leafValues,
                                    size_t leafValuesCount) {
    CBAMD_ENSURE(modelSplits.size() < 31, "tree is too deep");
    CBAMD_ENSURE((static_cast<size_t>(1) << modelSplits.size()) * ApproxDimension == leafValuesCount,
                 "leaf values count does not match tree depth and approx dimension");
    LeafValues.insert(LeafValues.end(), leafValues, leafValues + leafValuesCount);
    Trees.push_back(modelSplits);
}

void TObliviousTreeBuilder::Build(TModelTrees* result) {
    *result = TModelTrees();
    std::set<TModelSplit> splitSet;
    for (const auto& tree : Trees) {
        for (const auto& s : tree) {
            splitSet.insert(s);
        }
    }
    ProcessSplitsSet(splitSet, result);
    result->LeafValues = std::move(LeafValues);
    for (const auto& tree : Trees) {
        std::vector<int> bins;
        bins.reserve(tree.size());
        for (const auto& s : tree) {
            bins.push_back(BinFeatureIndexes.at(s));
        }
        result->AddBinTree(bins);
    }
    result->UpdateRuntimeData();
}

void TNonSymmetricTreeModelBuilder::AddTree(const TNonSymmetricTreeNode& head) {
    const size_t prev = FlatSplitsVector.size();
    TreeStartOffsets.push_back(static_cast<int>(prev));
    AddTreeNode(head);
    TreeSizes.push_back(static_cast<int>(FlatSplitsVector.size() - prev));
}

uint32_t TNonSymmetricTreeModelBuilder::AddTreeNode(const TNonSymmetricTreeNode& node) {
    // pre-order flattening; a split node with exactly one leaf child keeps that child's value on
    // itself and steps 0 towards it (model_build_helper.cpp:249-288)
    const uint32_t nodeId = static_cast<uint32_t>(FlatNonSymmetricStepNodes.size());
    if (node.IsSplit) {
        CBAMD_ENSURE(node.Left && node.Right, "split node must have both children");
        ModelSplitSet.insert(node.SplitCondition);
        FlatSplitsVector.emplace_back(true, node.SplitCondition);
        FlatNonSymmetricStepNodes.emplace_back();
        auto checkedDiff = [](uint32_t diff) {
            CBAMD_ENSURE(diff < 0xffff, "non-symmetric tree is too large for 16-bit node steps");
            return static_cast<uint16_t>(diff);
        };
        if (node.Left->IsSplit == node.Right->IsSplit) {
            FlatNodeValueIndexes.push_back(std::numeric_limits<uint32_t>::max());
            const uint32_t leftId = AddTreeNode(*node.Left);
            const uint32_t rightId = AddTreeNode(*node.Right);
            FlatNonSymmetricStepNodes[nodeId] = {checkedDiff(leftId - nodeId), checkedDiff(rightId - nodeId)};
        } else if (node.Right->IsSplit) {
            InsertNodeValue(*node.Left);
            const uint32_t rightId = AddTreeNode(*node.Right);
            FlatNonSymmetricStepNodes[nodeId] = {0, checkedDiff(rightId - nodeId)};
        } else {
            InsertNodeValue(*node.Right);
            const uint32_t leftId = AddTreeNode(*node.Left);
            FlatNonSymmetricStepNodes[nodeId] = {checkedDiff(leftId - nodeId), 0};
        }
    } else {
        FlatSplitsVector.emplace_back(false, TModelSplit());
        FlatNonSymmetricStepNodes.push_back({0, 0});
        InsertNodeValue(node);
    }
    return nodeId;
}

void TNonSymmetricTreeModelBuilder::InsertNodeValue(const TNonSymmetricTreeNode& node) {
    FlatNodeValueIndexes.push_back(static_cast<uint32_t>(FlatValueVector.size()));
    CBAMD_ENSURE(static_cast<int>(node.Value.size()) == ApproxDimension,
                 "Different model approx dimension and value dimensions");
    FlatValueVector.insert(FlatValueVector.end(), node.Value.begin(), node.Value.end());
}

void TNonSymmetricTreeModelBuilder::Build(TModelTrees* result) {
    *result = TModelTrees();
    ProcessSplitsSet(ModelSplitSet, result);
    result->NonSymmetricStepNodes = std::move(FlatNonSymmetricStepNodes);
    result->NonSymmetricNodeIdToLeafId = std::move(FlatNodeValueIndexes);
    result->LeafValues = std::move(FlatValueVector);
    for (const auto& s : FlatSplitsVector) {
        result->TreeSplits.push_back(s.first ? BinFeatureIndexes.at(s.second) : 0);
    }
    result->TreeSizes = std::move(TreeSizes);
    result->TreeStartOffsets = std::move(TreeStartOffsets);
    result->UpdateRuntimeData();
}

}  // namespace cbamd
