// Host-side model of a CatBoost tree ensemble: the tables of TModelTrees plus the runtime
// tables the evaluator needs. Mirrors catboost/libs/model/model.h:64-187 and features.h:16-160.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace cbamd {

// Raised for every condition the reference reports through CB_ENSURE
// (catboost/libs/helpers/exception.h:15); the C ABI turns it into `false` + GetErrorString().
class TModelError : public std::runtime_error {
public:
    explicit TModelError(const std::string& what) : std::runtime_error(what) {}
};

#define CBAMD_ENSURE(cond, msg)                                   \
    do {                                                          \
        if (!(cond)) {                                            \
            throw ::cbamd::TModelError(std::string() + msg);      \
        }                                                         \
    } while (0)

constexpr uint32_t kMaxValuesPerBin = 254;  // MAX_VALUES_PER_BIN, model.h:72

enum class ENanValueTreatment : int8_t { AsIs = 0, AsFalse = 1, AsTrue = 2 };  // features.h:51-55

struct TFloatFeature {  // features.h:50-94
    bool HasNans = false;
    int Index = -1;
    int FlatIndex = -1;
    std::vector<float> Borders;
    std::string FeatureId;
    ENanValueTreatment NanValueTreatment = ENanValueTreatment::AsIs;
    bool UsedInModel() const { return !Borders.empty(); }
};

struct TCatFeature {  // features.h:104-140
    int Index = -1;
    int FlatIndex = -1;
    std::string FeatureId;
    bool UsedInModel = true;
};

struct TOneHotFeature {  // features.h:142-160
    int CatFeatureIndex = -1;
    std::vector<int> Values;
    std::vector<std::string> StringValues;
};

enum class ECtrType : int8_t {  // flatbuffers/ctr_data.fbs:5-12
    Borders = 0,
    Buckets = 1,
    BinarizedTargetMeanValue = 2,
    FloatTargetMeanValue = 3,
    Counter = 4,
    FeatureFreq = 5
};

struct TFloatSplit {  // online_ctr.h:32-64
    int FloatFeature = 0;
    float Split = 0.f;
    bool operator==(const TFloatSplit& o) const { return FloatFeature == o.FloatFeature && Split == o.Split; }
    bool operator<(const TFloatSplit& o) const {
        return FloatFeature != o.FloatFeature ? FloatFeature < o.FloatFeature : Split < o.Split;
    }
};

struct TOneHotSplit {  // online_ctr.h:66-98
    int CatFeatureIdx = 0;
    int Value = 0;
    bool operator==(const TOneHotSplit& o) const { return CatFeatureIdx == o.CatFeatureIdx && Value == o.Value; }
    bool operator<(const TOneHotSplit& o) const {
        return CatFeatureIdx != o.CatFeatureIdx ? CatFeatureIdx < o.CatFeatureIdx : Value < o.Value;
    }
};

// The features a CTR is computed over (online_ctr.h:108-170).
struct TFeatureCombination {
    std::vector<int> CatFeatures;
    std::vector<TFloatSplit> BinFeatures;
    std::vector<TOneHotSplit> OneHotFeatures;
    bool operator==(const TFeatureCombination& o) const {
        return CatFeatures == o.CatFeatures && BinFeatures == o.BinFeatures && OneHotFeatures == o.OneHotFeatures;
    }
};

struct TModelCtrBase {  // online_ctr.h:178-258: identifies a table of learned statistics
    TFeatureCombination Projection;
    ECtrType CtrType = ECtrType::Borders;
    int TargetBorderClassifierIdx = 0;
    bool operator==(const TModelCtrBase& o) const {
        return Projection == o.Projection && CtrType == o.CtrType &&
               TargetBorderClassifierIdx == o.TargetBorderClassifierIdx;
    }
};

struct TModelCtr {  // online_ctr.h:260-316
    TModelCtrBase Base;
    int TargetBorderIdx = 0;
    float PriorNum = 0.f;
    float PriorDenom = 1.f;
    float Shift = 0.f;
    float Scale = 1.f;
    float Calc(float countInClass, float totalCount) const {  // online_ctr.h:290-293
        const float ctr = (countInClass + PriorNum) / (totalCount + PriorDenom);
        return (ctr + Shift) * Scale;
    }
};

struct TCtrFeature {  // features.h:306-323
    TModelCtr Ctr;
    std::vector<float> Borders;
};

// One table of learned statistics (ctr_value_table.h:17-109): an open-addressing index
// hash -> row (12-byte buckets {u64 hash, u32 row}, helpers/dense_hash_view.h:12-66) and the rows.
struct TCtrValueTable {
    TModelCtrBase ModelCtrBase;
    std::vector<uint8_t> IndexHashRaw;
    std::vector<uint8_t> CTRBlob;
    int CounterDenominator = 0;
    int TargetClassesCount = 0;
};

struct TRepackedBin {  // model.h:64-70
    uint16_t FeatureIndex = 0;
    uint8_t XorMask = 0;
    uint8_t SplitIdx = 0;
};

struct TNonSymmetricTreeStepNode {  // model.h:78-95
    uint16_t LeftSubtreeDiff = 0xffff;
    uint16_t RightSubtreeDiff = 0xffff;
};

enum class ESplitType : int { FloatFeature = 0, EstimatedFeature = 1, OneHotFeature = 2, OnlineCtr = 3 };  // split.h:20-25

// TModelSplit restricted to the kinds this evaluator supports (split.h:27-100).
struct TModelSplit {
    ESplitType Type = ESplitType::FloatFeature;
    int FeatureIndex = 0;  // float feature index / cat feature index / position in CtrFeatures
    float Border = 0.f;
    int Value = 0;

    static TModelSplit Float(int feature, float border) {
        TModelSplit s;
        s.Type = ESplitType::FloatFeature;
        s.FeatureIndex = feature;
        s.Border = border;
        return s;
    }
    static TModelSplit OneHot(int catFeature, int value) {
        TModelSplit s;
        s.Type = ESplitType::OneHotFeature;
        s.FeatureIndex = catFeature;
        s.Value = value;
        return s;
    }
    static TModelSplit Ctr(int ctrFeature, float border) {
        TModelSplit s;
        s.Type = ESplitType::OnlineCtr;
        s.FeatureIndex = ctrFeature;
        s.Border = border;
        return s;
    }
    bool operator<(const TModelSplit& o) const;
    bool operator==(const TModelSplit& o) const;
};

struct TModelTrees {
    // ---- serialized state (flatbuffers/model.fbs:22-46)
    int ApproxDimension = 1;
    std::vector<int> TreeSplits;
    std::vector<int> TreeSizes;
    std::vector<int> TreeStartOffsets;
    std::vector<TCatFeature> CatFeatures;
    std::vector<TFloatFeature> FloatFeatures;
    std::vector<TOneHotFeature> OneHotFeatures;
    std::vector<TCtrFeature> CtrFeatures;
    std::vector<double> LeafValues;
    std::vector<double> LeafWeights;
    std::vector<TNonSymmetricTreeStepNode> NonSymmetricStepNodes;
    std::vector<uint32_t> NonSymmetricNodeIdToLeafId;
    double Scale = 1.0;
    std::vector<double> Bias;  // ApproxDimension values
    // feature kinds this evaluator refuses; only their presence is recorded
    size_t TextFeatureCount = 0;
    size_t EstimatedFeatureCount = 0;
    size_t EmbeddingFeatureCount = 0;

    // ---- runtime state (TRuntimeData / TForApplyData, model.h:146-187)
    std::vector<TModelSplit> BinFeatures;
    uint32_t EffectiveBinFeaturesBucketCount = 0;
    uint32_t CtrFirstBucket = 0;  // buckets of float and one-hot features come first, CTR buckets after them
    std::vector<TRepackedBin> RepackedBins;
    std::vector<size_t> TreeFirstLeafOffsets;
    size_t UsedFloatFeaturesCount = 0;
    size_t UsedCatFeaturesCount = 0;
    size_t MinimalSufficientFloatFeaturesVectorSize = 0;
    size_t MinimalSufficientCatFeaturesVectorSize = 0;

    bool IsOblivious() const {  // model.h:271-273
        return NonSymmetricStepNodes.empty() && NonSymmetricNodeIdToLeafId.empty();
    }
    size_t GetTreeCount() const { return TreeSizes.size(); }
    size_t GetNumFloatFeatures() const {  // model.h:494-500
        return FloatFeatures.empty() ? 0 : static_cast<size_t>(FloatFeatures.back().Index) + 1;
    }
    size_t GetNumCatFeatures() const {  // model.h:502-508
        return CatFeatures.empty() ? 0 : static_cast<size_t>(CatFeatures.back().Index) + 1;
    }
    size_t GetFlatFeatureVectorExpectedSize() const;  // model.h:534-541
    bool IsIdentityScaleAndBias() const;
    bool IsZeroBias() const;

    // UpdateRuntimeData = CalcForApplyData + CalcBinFeatures (model.cpp:425-429, 471-624).
    void UpdateRuntimeData();
    // model.cpp:634-674
    void ConvertObliviousToAsymmetric();
    void SetScaleAndBias(double scale, const std::vector<double>& bias);  // model.cpp:700-709
    // Adds the tree-start offsets that the low-level AddBinTree API derives (model.cpp:238-254).
    void AddBinTree(const std::vector<int>& binSplits);
};

struct TFeaturePosition {  // features.h:16-48
    int Index = -1;
    int FlatIndex = -1;
};

// Where the model's features sit in a caller's data when that differs from the positions stored in
// the model (NCB::NModelEvaluation::TFeatureLayout, evaluation_interface.h:17-69): a feature at model
// position p is read at FloatFeatureIndexes[p] / CatFeatureIndexes[p] (separate float and categorical
// arrays) or FlatIndexes[p] (flat vectors). A list that is not defined leaves its positions as they are.
struct TFeatureLayout {
    bool HasFloatFeatureIndexes = false;
    bool HasCatFeatureIndexes = false;
    bool HasFlatIndexes = false;
    std::vector<uint32_t> FloatFeatureIndexes;
    std::vector<uint32_t> CatFeatureIndexes;
    std::vector<uint32_t> FlatIndexes;

    bool Defined() const { return HasFloatFeatureIndexes || HasCatFeatureIndexes || HasFlatIndexes; }
    // GetRemappedPosition; a position outside a defined list is an error (TVector::at there)
    TFeaturePosition Remap(const TFloatFeature& feature) const;
    TFeaturePosition Remap(const TCatFeature& feature) const;
};

struct TFullModel {
    TModelTrees Trees;
    std::map<std::string, std::string> ModelInfo;
    std::vector<std::string> ModelPartIds;
    // the tables of the static CTR provider (model part "static_provider_v1", static_ctr_provider.h:14-88)
    std::vector<TCtrValueTable> CtrTables;
    const TCtrValueTable* FindCtrTable(const TModelCtrBase& base) const;

    // .cbm (de)serialisation, model.cpp:1113-1228
    void Load(const void* data, size_t size);
    void LoadFromFile(const std::string& path);
    // the "json" model format (model_export/json_model_helpers.cpp:583-608)
    void LoadFromJson(const void* data, size_t size);
    void LoadFromJsonFile(const std::string& path);
    std::string Save() const;
    void SaveToFile(const std::string& path) const;

    // Throws unless every feature kind in the model is one the HIP evaluator handles.
    void EnsureSupported() const;
    std::vector<std::string> GetUsedFeaturesNames() const;  // model.cpp:1300-1343
};

}  // namespace cbamd
