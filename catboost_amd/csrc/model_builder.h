// Model builders with the semantics of TObliviousTreeBuilder / TNonSymmetricTreeModelBuilder
// (catboost/libs/model/model_build_helper.h, model_build_helper.cpp:100-304).
#pragma once

#include "model.h"

#include <map>
#include <memory>
#include <set>

namespace cbamd {

class TCommonModelBuilderHelper {
public:
    TCommonModelBuilderHelper(std::vector<TFloatFeature> allFloatFeatures,
                              std::vector<TCatFeature> allCategoricalFeatures,
                              int approxDimension);

protected:
    // Clears all borders, re-adds only the borders that occur in `splits` (in sorted order),
    // rebuilds the one-hot features, marks used cat features and numbers the binary features.
    void ProcessSplitsSet(const std::set<TModelSplit>& splits, TModelTrees* trees);

    int ApproxDimension;
    std::vector<TFloatFeature> FloatFeatures;
    std::vector<TCatFeature> CatFeatures;
    std::map<int, size_t> FloatFeaturesInternalIndexesMap;
    std::map<int, size_t> CatFeaturesInternalIndexesMap;
    std::map<TModelSplit, int> BinFeatureIndexes;
};

class TObliviousTreeBuilder : public TCommonModelBuilderHelper {
public:
    using TCommonModelBuilderHelper::TCommonModelBuilderHelper;

    // leaf values laid out [leaf * approxDimension + dimension]
    void AddTree(const std::vector<TModelSplit>& modelSplits, const double* leafValues, size_t leafValuesCount);
    void Build(TModelTrees* result);

private:
    std::vector<std::vector<TModelSplit>> Trees;
    std::vector<double> LeafValues;
};

struct TNonSymmetricTreeNode {
    bool IsSplit = false;
    TModelSplit SplitCondition;
    std::unique_ptr<TNonSymmetricTreeNode> Left;
    std::unique_ptr<TNonSymmetricTreeNode> Right;
    std::vector<double> Value;  // approxDimension values for a leaf
};

class TNonSymmetricTreeModelBuilder : public TCommonModelBuilderHelper {
public:
    using TCommonModelBuilderHelper::TCommonModelBuilderHelper;

    void AddTree(const TNonSymmetricTreeNode& head);
    void Build(TModelTrees* result);

private:
    uint32_t AddTreeNode(const TNonSymmetricTreeNode& node);
    void InsertNodeValue(const TNonSymmetricTreeNode& node);

    std::vector<int> TreeSizes;
    std::vector<int> TreeStartOffsets;
    std::vector<std::pair<bool, TModelSplit>> FlatSplitsVector;
    std::vector<double> FlatValueVector;
    std::vector<TNonSymmetricTreeStepNode> FlatNonSymmetricStepNodes;
    std::vector<uint32_t> FlatNodeValueIndexes;
    std::set<TModelSplit> ModelSplitSet;
};

}  // namespace cbamd
