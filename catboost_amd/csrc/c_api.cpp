// The exported C ABI: the reference's model_calcer surface (include/c_api.h) and the
// evaluator-level seam (include/cb_hip_evaluator.h), both in front of THipEvaluator.
// Error handling follows catboost/libs/model_interface/c_api.cpp:33-37, 263-291: every entry
// point catches, stores the message in a thread-local and returns false / NULL.
#include "../../include/c_api.h"
#include "../../include/cb_hip_evaluator.h"

#include "cat_hash.h"
#include "fast_exp.h"
#include "hip_evaluator.h"
#include "model.h"
#include "model_builder.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

using namespace cbamd;

namespace {

thread_local std::string LastError;

struct TModelHandle {
    TFullModel Model;
    std::unique_ptr<THipEvaluator> Evaluator;
    std::mutex EvaluatorLock;
    int DeviceId = 0;
    EApiPredictionType PredictionType = APT_RAW_FORMULA_VAL;
    TFeatureLayout Layout;  // IModelEvaluator::SetFeatureLayout, evaluation_interface.h:82
    bool SmallBatchSlicing = true;  // CbHipSetSmallBatchSlicing

    void ResetEvaluator() {
        std::lock_guard<std::mutex> g(EvaluatorLock);
        Evaluator.reset();
    }
    // lazily binds the model to its device (TFullModel::GetCurrentEvaluator, model.h:682-689)
    THipEvaluator& GetEvaluator() {
        std::lock_guard<std::mutex> g(EvaluatorLock);
        if (!Evaluator) {
            Model.EnsureSupported();
            Evaluator.reset(new THipEvaluator(Model.Trees, DeviceId, &Model.CtrTables, &Layout));
            if (!SmallBatchSlicing) {
                Evaluator->SetSmallBatchSlicing(false);
            }
        }
        return *Evaluator;
    }
};

TModelHandle* H(void* h) {
    CBAMD_ENSURE(h != nullptr, "model handle is null");
    return static_cast<TModelHandle*>(h);
}

template <typename F>
bool Guard(F&& f) {
    try {
        f();
        return true;
    } catch (const std::exception& e) {
        LastError = e.what();
    } catch (...) {
        LastError = "unknown error";
    }
    return false;
}

size_t PredictionDims(const TModelHandle& h) {  // evaluation_interface.h:86-99
    return h.PredictionType == APT_CLASS ? 1 : static_cast<size_t>(h.Model.Trees.ApproxDimension);
}

void CheckResultSize(const TModelHandle& h, size_t docCount, size_t resultSize) {
    // TEvalResultProcessor, eval_processing.cpp:18-23
    const size_t dims = PredictionDims(h);
    CBAMD_ENSURE(resultSize == docCount * dims,
                 "`results` size is insufficient: Results.size() = " + std::to_string(resultSize) +
                     ", resultApproxDimension = " + std::to_string(dims) +
                     ", docCount * resultApproxDimension = " + std::to_string(docCount * dims));
    if (h.Model.Trees.ApproxDimension > 1 && (h.PredictionType == APT_CLASS || h.PredictionType == APT_PROBABILITY)) {
        CBAMD_ENSURE(h.Model.Trees.IsIdentityScaleAndBias(),
                     "Non-identity {Scale,Bias} for normalizing a multiclass model is not supported");
    }
}

// Turns raw formula values into the requested prediction type on the host, block by block like
// TEvalResultProcessor::PostprocessBlock (eval_processing.h:174-240; blocks of min(128, docCount)
// documents, cpu/formula_evaluator.cpp:27), with the reference's exponent (fast_exp.h).
void PostProcess(EApiPredictionType type, size_t dim, size_t docCount, const double* raw, double* out) {
    const size_t block = std::min<size_t>(128, docCount);
    for (size_t begin = 0; begin < docCount; begin += block) {
        const size_t n = std::min(block, docCount - begin);
        const double* r = raw + begin * dim;
        if (type == APT_CLASS) {
            double* o = out + begin;
            for (size_t i = 0; i < n; ++i) {
                // one dimension: the raw value against the border 0 (the CPU evaluator never passes a
                // probability border); otherwise the first largest dimension
                o[i] = dim == 1 ? static_cast<double>(r[i] > 0.0)
                                : static_cast<double>(std::max_element(r + i * dim, r + (i + 1) * dim) - (r + i * dim));
            }
            continue;
        }
        double* o = out + begin * dim;
        std::copy(r, r + n * dim, o);
        const auto sigmoid = [](double* v, size_t count) {  // CalcSigmoid, eval_processing.h:92-99
            for (size_t i = 0; i < count; ++i) {
                v[i] = -v[i];
            }
            FastExpInplace(v, count);
            for (size_t i = 0; i < count; ++i) {
                v[i] = 1. / (1. + v[i]);
            }
        };
        if (dim == 1) {
            switch (type) {
                case APT_PROBABILITY:
                    sigmoid(o, n);
                    break;
                case APT_EXPONENT:
                    FastExpInplace(o, n);
                    break;
                default:
                    CBAMD_ENSURE(false, "unsupported prediction type");
            }
            continue;
        }
        switch (type) {
            case APT_RMSE_WITH_UNCERTAINTY:  // CalcSquaredExponentInplace on the second value of a document
                for (size_t i = 1; i < n * dim; i += dim) {
                    o[i] *= 2.0f;
                    FastExpInplace(o + i, 1);
                }
                break;
            case APT_PROBABILITY:  // CalcSoftmax per document, eval_processing.h:15-27
                for (size_t i = 0; i < n; ++i) {
                    double* v = o + i * dim;
                    const double top = *std::max_element(v, v + dim);
                    for (size_t k = 0; k < dim; ++k) {
                        v[k] = v[k] - top;
                    }
                    FastExpInplace(v, dim);
                    double sum = 0;
                    for (size_t k = 0; k < dim; ++k) {
                        sum += v[k];
                    }
                    for (size_t k = 0; k < dim; ++k) {
                        v[k] /= sum;
                    }
                }
                break;
            case APT_MULTI_PROBABILITY:
                sigmoid(o, n * dim);
                break;
            default:
                // the reference's switch has no other case for several dimensions and leaves the raw
                // values in place (a debug-only assert)
                break;
        }
    }
}

// Runs `calc(double* result, int predictionType)`: the evaluator applies the handle's prediction type on
// the device before it copies the results back.
template <typename F>
void CalcWithPredictionType(TModelHandle& h, size_t docCount, double* result, size_t resultSize, F&& calc) {
    CheckResultSize(h, docCount, resultSize);
    calc(result, static_cast<int>(h.PredictionType));
}

void CalcFlatImpl(void* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd, const float** floatFeatures,
                  size_t floatFeaturesSize, double* result, size_t resultSize) {
    TModelHandle& h = *H(modelHandle);
    CalcWithPredictionType(h, docCount, result, resultSize, [&](double* out, int predictionType) {
        h.GetEvaluator().CalcHostRows(floatFeatures, floatFeaturesSize, /*flat*/ true, nullptr, 0, docCount, treeStart,
                                      treeEnd, out, predictionType);
    });
}

void CalcHashedImpl(void* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd, const float** floatFeatures,
                    size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize, double* result,
                    size_t resultSize) {
    TModelHandle& h = *H(modelHandle);
    static_assert(sizeof(int) == sizeof(int32_t), "int must be 32 bits");
    CalcWithPredictionType(h, docCount, result, resultSize, [&](double* out, int predictionType) {
        h.GetEvaluator().CalcHostRows(floatFeaturesSize ? floatFeatures : nullptr, floatFeaturesSize, /*flat*/ false,
                                      catFeaturesSize ? reinterpret_cast<const int32_t* const*>(catFeatures) : nullptr,
                                      catFeaturesSize, docCount, treeStart, treeEnd, out, predictionType);
    });
}

// hashes string categories into an int matrix (cpu/formula_evaluator.cpp:396-398)
struct THashedCats {
    std::vector<int32_t> Data;
    std::vector<const int32_t*> Rows;
    THashedCats(const char* const* const* catFeatures, size_t docCount, size_t catFeaturesSize) {
        Data.resize(docCount * catFeaturesSize);
        Rows.resize(docCount);
        for (size_t d = 0; d < docCount; ++d) {
            Rows[d] = Data.data() + d * catFeaturesSize;
            for (size_t c = 0; c < catFeaturesSize; ++c) {
                const char* s = catFeatures[d][c];
                CBAMD_ENSURE(s != nullptr, "categorical feature value is null");
                Data[d * catFeaturesSize + c] = CalcCatFeatureHashInt(s, std::strlen(s));
            }
        }
    }
};

void CalcStringCatsImpl(void* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd,
                        const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures,
                        size_t catFeaturesSize, double* result, size_t resultSize) {
    CBAMD_ENSURE(catFeaturesSize == 0 || catFeatures != nullptr, "categorical features pointer is null");
    THashedCats hashed(catFeatures, docCount, catFeaturesSize);
    CalcHashedImpl(modelHandle, docCount, treeStart, treeEnd, floatFeatures, floatFeaturesSize,
                   reinterpret_cast<const int**>(hashed.Rows.data()), catFeaturesSize, result, resultSize);
}

void EnsureNoTextOrEmbeddings(size_t textFeaturesSize, size_t embeddingFeaturesSize) {
    CBAMD_ENSURE(textFeaturesSize == 0, "text features are not supported by the HIP evaluator");
    CBAMD_ENSURE(embeddingFeaturesSize == 0, "embedding features are not supported by the HIP evaluator");
}

void SpecificClass(void* modelHandle, int classId, const std::vector<double>& raw, double* result, size_t resultSize) {
    const size_t dim = static_cast<size_t>(H(modelHandle)->Model.Trees.ApproxDimension);
    CBAMD_ENSURE(classId >= 0 && static_cast<size_t>(classId) < dim, "class id is out of range");
    CBAMD_ENSURE(resultSize * dim <= raw.size(), "result size is larger than the document count");
    for (size_t d = 0; d < resultSize; ++d) {
        result[d] = raw[d * dim + classId];
    }
}

bool ReturnIndices(const std::vector<size_t>& values, size_t** indices, size_t* count) {
    return Guard([&] {
        *count = values.size();
        if (values.empty()) {
            *indices = nullptr;
            return;
        }
        *indices = static_cast<size_t*>(std::malloc(sizeof(size_t) * values.size()));
        if (!*indices) {
            throw std::bad_alloc();
        }
        std::copy(values.begin(), values.end(), *indices);
    });
}

void ArraysToTrees(const CbHipModelArrays& a, bool withTrees, TModelTrees* trees) {
    CBAMD_ENSURE(a.ApproxDimension >= 1, "approx dimension must be positive");
    trees->ApproxDimension = a.ApproxDimension;
    CBAMD_ENSURE(a.FloatFeatureCount >= 0 && a.CatFeatureCount >= 0 && a.OneHotFeatureCount >= 0, "negative feature count");
    for (int i = 0; i < a.FloatFeatureCount; ++i) {
        TFloatFeature f;
        f.Index = a.FloatFeatureIndex[i];
        f.FlatIndex = a.FloatFeatureFlatIndex[i];
        f.HasNans = a.FloatFeatureHasNans ? a.FloatFeatureHasNans[i] != 0 : false;
        const int nan = a.FloatFeatureNanTreatment ? a.FloatFeatureNanTreatment[i] : 0;
        CBAMD_ENSURE(nan >= 0 && nan <= 2, "unknown NaN value treatment");
        f.NanValueTreatment = static_cast<ENanValueTreatment>(nan);
        if (withTrees && a.FloatFeatureBorderOffsets) {
            const int b0 = a.FloatFeatureBorderOffsets[i], b1 = a.FloatFeatureBorderOffsets[i + 1];
            CBAMD_ENSURE(b0 >= 0 && b1 >= b0, "float feature border offsets must not decrease");
            f.Borders.assign(a.FloatFeatureBorders + b0, a.FloatFeatureBorders + b1);
        }
        trees->FloatFeatures.push_back(std::move(f));
    }
    for (int i = 0; i < a.CatFeatureCount; ++i) {
        TCatFeature c;
        c.Index = a.CatFeatureIndex[i];
        c.FlatIndex = a.CatFeatureFlatIndex[i];
        c.UsedInModel = a.CatFeatureUsed ? a.CatFeatureUsed[i] != 0 : true;
        trees->CatFeatures.push_back(std::move(c));
    }
    if (a.Bias) {
        trees->Bias.assign(a.Bias, a.Bias + a.ApproxDimension);
    } else {
        trees->Bias.assign(a.ApproxDimension, 0.0);
    }
    trees->Scale = a.Scale;
    if (!withTrees) {
        return;
    }
    for (int i = 0; i < a.OneHotFeatureCount; ++i) {
        TOneHotFeature oh;
        oh.CatFeatureIndex = a.OneHotCatFeatureIndex[i];
        const int v0 = a.OneHotValueOffsets[i], v1 = a.OneHotValueOffsets[i + 1];
        CBAMD_ENSURE(v0 >= 0 && v1 >= v0, "one-hot value offsets must not decrease");
        oh.Values.assign(a.OneHotValues + v0, a.OneHotValues + v1);
        trees->OneHotFeatures.push_back(std::move(oh));
    }
    CBAMD_ENSURE(a.TreeCount >= 0 && a.TreeSplitsCount >= 0 && a.StepNodeCount >= 0, "negative table size");
    trees->TreeSizes.assign(a.TreeSizes, a.TreeSizes + a.TreeCount);
    trees->TreeStartOffsets.assign(a.TreeStartOffsets, a.TreeStartOffsets + a.TreeCount);
    trees->TreeSplits.assign(a.TreeSplits, a.TreeSplits + a.TreeSplitsCount);
    trees->LeafValues.assign(a.LeafValues, a.LeafValues + a.LeafValuesCount);
    trees->NonSymmetricStepNodes.resize(a.StepNodeCount);
    for (int i = 0; i < a.StepNodeCount; ++i) {
        trees->NonSymmetricStepNodes[i] = {a.StepNodes[2 * i], a.StepNodes[2 * i + 1]};
    }
    if (a.StepNodeCount) {
        trees->NonSymmetricNodeIdToLeafId.assign(a.NodeIdToLeafId, a.NodeIdToLeafId + a.StepNodeCount);
    }
    trees->SetScaleAndBias(trees->Scale, trees->Bias);
    trees->UpdateRuntimeData();
}

TModelSplit ToSplit(const CbHipModelSplit& s) {
    if (s.Type == static_cast<int>(ESplitType::FloatFeature)) {
        return TModelSplit::Float(s.FeatureIndex, s.Border);
    }
    CBAMD_ENSURE(s.Type == static_cast<int>(ESplitType::OneHotFeature), "unsupported split type");
    return TModelSplit::OneHot(s.FeatureIndex, s.Value);
}

TFeatureBatch ToBatch(const CbHipFeatures* f) {
    CBAMD_ENSURE(f != nullptr, "features descriptor is null");
    TFeatureBatch b;
    CBAMD_ENSURE(f->Layout >= 0 && f->Layout <= 2, "unknown feature layout");
    b.Layout = static_cast<TFeatureBatch::ELayout>(f->Layout);
    b.Floats = f->Floats;
    b.Stride = f->Stride;
    b.Cats = f->Cats;
    b.CatStride = f->CatStride;
    return b;
}

THipEvaluator* E(CbHipEvaluatorHandle* e) {
    CBAMD_ENSURE(e != nullptr, "evaluator handle is null");
    return static_cast<THipEvaluator*>(e);
}

}  // namespace

extern "C" {

// ------------------------------------------------------------------------- data wrapper ----

DataWrapperHandle* DataWrapperCreate(size_t) {
    LastError = "DataWrapper is not supported by the HIP evaluator";
    return nullptr;
}
void DataWrapperDelete(DataWrapperHandle*) {}
void AddFloatFeatures(DataWrapperHandle*, const float**, size_t) {}
void AddCatFeatures(DataWrapperHandle*, const char***, size_t) {}
void AddTextFeatures(DataWrapperHandle*, const char***, size_t) {}
void AddEmbeddingFeatures(DataWrapperHandle*, const float***, size_t*, size_t) {}
DataProviderHandle* BuildDataProvider(DataWrapperHandle*) {
    LastError = "DataWrapper is not supported by the HIP evaluator";
    return nullptr;
}

// --------------------------------------------------------------------------- life cycle ----

ModelCalcerHandle* ModelCalcerCreate(void) {
    try {
        auto* h = new TModelHandle;
        h->Model.Trees.UpdateRuntimeData();
        return h;
    } catch (const std::exception& e) {
        LastError = e.what();
    }
    return nullptr;
}

void ModelCalcerDelete(ModelCalcerHandle* modelHandle) {
    delete static_cast<TModelHandle*>(modelHandle);
}

const char* GetErrorString(void) {
    return LastError.c_str();
}

bool LoadFullModelFromFile(ModelCalcerHandle* modelHandle, const char* filename) {
    return Guard([&] {
        CBAMD_ENSURE(filename != nullptr, "file name is null");
        TFullModel model;
        model.LoadFromFile(filename);
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model = std::move(model);
    });
}

bool LoadFullModelFromBuffer(ModelCalcerHandle* modelHandle, const void* binaryBuffer, size_t binaryBufferSize) {
    return Guard([&] {
        CBAMD_ENSURE(binaryBuffer != nullptr, "model buffer is null");
        TFullModel model;
        model.Load(binaryBuffer, binaryBufferSize);
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model = std::move(model);
    });
}

bool CbHipLoadFullModelFromJsonFile(void* modelHandle, const char* filename) {
    return Guard([&] {
        CBAMD_ENSURE(filename != nullptr, "file name is null");
        TFullModel model;
        model.LoadFromJsonFile(filename);
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model = std::move(model);
    });
}

bool CbHipLoadFullModelFromJsonBuffer(void* modelHandle, const void* jsonText, size_t jsonTextSize) {
    return Guard([&] {
        CBAMD_ENSURE(jsonText != nullptr, "model buffer is null");
        TFullModel model;
        model.LoadFromJson(jsonText, jsonTextSize);
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model = std::move(model);
    });
}

bool LoadFullModelZeroCopy(ModelCalcerHandle* modelHandle, const void* binaryBuffer, size_t binaryBufferSize) {
    return LoadFullModelFromBuffer(modelHandle, binaryBuffer, binaryBufferSize);
}

bool EnableGPUEvaluation(ModelCalcerHandle* modelHandle, int deviceId) {
    return Guard([&] {
        TModelHandle* h = H(modelHandle);
        CBAMD_ENSURE(deviceId >= 0 && deviceId < GetHipDeviceCount(), "HIP device " + std::to_string(deviceId) + " does not exist");
        if (deviceId != h->DeviceId) {
            h->ResetEvaluator();
            h->DeviceId = deviceId;
        }
        h->GetEvaluator();
    });
}

bool GetSupportedEvaluatorTypes(ModelCalcerHandle*, enum ECatBoostApiFormulaEvaluatorType** formulaEvaluatorTypes,
                                size_t* formulaEvaluatorTypesCount) {
    return Guard([&] {
        *formulaEvaluatorTypes = static_cast<ECatBoostApiFormulaEvaluatorType*>(std::malloc(sizeof(ECatBoostApiFormulaEvaluatorType)));
        if (!*formulaEvaluatorTypes) {
            throw std::bad_alloc();
        }
        (*formulaEvaluatorTypes)[0] = CBA_FET_GPU;
        *formulaEvaluatorTypesCount = 1;
    });
}

bool SetPredictionType(ModelCalcerHandle* modelHandle, enum EApiPredictionType predictionType) {
    return Guard([&] {
        CBAMD_ENSURE(predictionType >= APT_RAW_FORMULA_VAL && predictionType <= APT_MULTI_PROBABILITY, "Unexpected prediction type");
        H(modelHandle)->PredictionType = predictionType;
    });
}

bool SetPredictionTypeString(ModelCalcerHandle* modelHandle, const char* predictionTypeStr) {
    return Guard([&] {
        CBAMD_ENSURE(predictionTypeStr != nullptr, "prediction type string is null");
        static const char* kNames[] = {"RawFormulaVal", "Exponent", "RMSEWithUncertainty", "Probability", "Class", "MultiProbability"};
        for (int i = 0; i < 6; ++i) {
            if (std::strcmp(predictionTypeStr, kNames[i]) == 0) {
                H(modelHandle)->PredictionType = static_cast<EApiPredictionType>(i);
                return;
            }
        }
        CBAMD_ENSURE(false, std::string("Unknown prediction type: ") + predictionTypeStr);
    });
}

// -------------------------------------------------------------------------- predictions ----

bool CalcModelPredictionFlatStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd,
                                   const float** floatFeatures, size_t floatFeaturesSize, double* result,
                                   size_t resultSize) {
    return Guard([&] {
        CalcFlatImpl(modelHandle, docCount, treeStart, treeEnd, floatFeatures, floatFeaturesSize, result, resultSize);
    });
}

bool CalcModelPredictionFlat(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                             size_t floatFeaturesSize, double* result, size_t resultSize) {
    return CalcModelPredictionFlatStaged(modelHandle, docCount, 0, GetTreeCount(modelHandle), floatFeatures,
                                         floatFeaturesSize, result, resultSize);
}

bool CalcModelPredictionFlatTransposedStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart,
                                             size_t treeEnd, const float** floatFeatures, size_t floatFeaturesSize,
                                             double* result, size_t resultSize) {
    return Guard([&] {
        TModelHandle& h = *H(modelHandle);
        CalcWithPredictionType(h, docCount, result, resultSize, [&](double* out, int predictionType) {
            h.GetEvaluator().CalcHostColumns(floatFeatures, floatFeaturesSize, docCount, treeStart, treeEnd, out,
                                             predictionType);
        });
    });
}

bool CalcModelPredictionFlatTransposed(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                                       size_t floatFeaturesSize, double* result, size_t resultSize) {
    return CalcModelPredictionFlatTransposedStaged(modelHandle, docCount, 0, GetTreeCount(modelHandle), floatFeatures,
                                                   floatFeaturesSize, result, resultSize);
}

bool CalcModelPredictionStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd,
                               const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures,
                               size_t catFeaturesSize, double* result, size_t resultSize) {
    return Guard([&] {
        CalcStringCatsImpl(modelHandle, docCount, treeStart, treeEnd, floatFeatures, floatFeaturesSize, catFeatures,
                           catFeaturesSize, result, resultSize);
    });
}

bool CalcModelPrediction(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                         size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, double* result,
                         size_t resultSize) {
    return CalcModelPredictionStaged(modelHandle, docCount, 0, GetTreeCount(modelHandle), floatFeatures,
                                     floatFeaturesSize, catFeatures, catFeaturesSize, result, resultSize);
}

bool CalcModelPredictionSingleStaged(ModelCalcerHandle* modelHandle, size_t treeStart, size_t treeEnd,
                                     const float* floatFeatures, size_t floatFeaturesSize, const char** catFeatures,
                                     size_t catFeaturesSize, double* result, size_t resultSize) {
    return Guard([&] {
        const float* rows[1] = {floatFeatures};
        const char** catRows[1] = {catFeatures};
        CalcStringCatsImpl(modelHandle, 1, treeStart, treeEnd, rows, floatFeaturesSize, catRows, catFeaturesSize, result,
                           resultSize);
    });
}

bool CalcModelPredictionSingle(ModelCalcerHandle* modelHandle, const float* floatFeatures, size_t floatFeaturesSize,
                               const char** catFeatures, size_t catFeaturesSize, double* result, size_t resultSize) {
    return CalcModelPredictionSingleStaged(modelHandle, 0, GetTreeCount(modelHandle), floatFeatures, floatFeaturesSize,
                                           catFeatures, catFeaturesSize, result, resultSize);
}

bool CalcModelPredictionWithHashedCatFeatures(ModelCalcerHandle* modelHandle, size_t docCount,
                                              const float** floatFeatures, size_t floatFeaturesSize,
                                              const int** catFeatures, size_t catFeaturesSize, double* result,
                                              size_t resultSize) {
    return Guard([&] {
        CalcHashedImpl(modelHandle, docCount, 0, H(modelHandle)->Model.Trees.GetTreeCount(), floatFeatures,
                       floatFeaturesSize, catFeatures, catFeaturesSize, result, resultSize);
    });
}

bool CalcModelPredictionTextStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd,
                                   const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures,
                                   size_t catFeaturesSize, const char***, size_t textFeaturesSize, double* result,
                                   size_t resultSize) {
    return Guard([&] {
        EnsureNoTextOrEmbeddings(textFeaturesSize, 0);
        CalcStringCatsImpl(modelHandle, docCount, treeStart, treeEnd, floatFeatures, floatFeaturesSize, catFeatures,
                           catFeaturesSize, result, resultSize);
    });
}

bool CalcModelPredictionText(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                             size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize,
                             const char*** textFeatures, size_t textFeaturesSize, double* result, size_t resultSize) {
    return CalcModelPredictionTextStaged(modelHandle, docCount, 0, GetTreeCount(modelHandle), floatFeatures,
                                         floatFeaturesSize, catFeatures, catFeaturesSize, textFeatures,
                                         textFeaturesSize, result, resultSize);
}

bool CalcModelPredictionTextAndEmbeddingsStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart,
                                                size_t treeEnd, const float** floatFeatures, size_t floatFeaturesSize,
                                                const char*** catFeatures, size_t catFeaturesSize, const char***,
                                                size_t textFeaturesSize, const float***, size_t*,
                                                size_t embeddingFeaturesSize, double* result, size_t resultSize) {
    return Guard([&] {
        EnsureNoTextOrEmbeddings(textFeaturesSize, embeddingFeaturesSize);
        CalcStringCatsImpl(modelHandle, docCount, treeStart, treeEnd, floatFeatures, floatFeaturesSize, catFeatures,
                           catFeaturesSize, result, resultSize);
    });
}

bool CalcModelPredictionTextAndEmbeddings(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                                          size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize,
                                          const char*** textFeatures, size_t textFeaturesSize,
                                          const float*** embeddingFeatures, size_t* embeddingDimensions,
                                          size_t embeddingFeaturesSize, double* result, size_t resultSize) {
    return CalcModelPredictionTextAndEmbeddingsStaged(modelHandle, docCount, 0, GetTreeCount(modelHandle), floatFeatures,
                                                      floatFeaturesSize, catFeatures, catFeaturesSize, textFeatures,
                                                      textFeaturesSize, embeddingFeatures, embeddingDimensions,
                                                      embeddingFeaturesSize, result, resultSize);
}

bool CalcModelPredictionWithHashedCatFeaturesAndTextFeatures(ModelCalcerHandle* modelHandle, size_t docCount,
                                                             const float** floatFeatures, size_t floatFeaturesSize,
                                                             const int** catFeatures, size_t catFeaturesSize,
                                                             const char***, size_t textFeaturesSize, double* result,
                                                             size_t resultSize) {
    return Guard([&] {
        EnsureNoTextOrEmbeddings(textFeaturesSize, 0);
        CalcHashedImpl(modelHandle, docCount, 0, H(modelHandle)->Model.Trees.GetTreeCount(), floatFeatures,
                       floatFeaturesSize, catFeatures, catFeaturesSize, result, resultSize);
    });
}

bool CalcModelPredictionWithHashedCatFeaturesAndTextAndEmbeddingFeatures(
    ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize,
    const int** catFeatures, size_t catFeaturesSize, const char***, size_t textFeaturesSize, const float***, size_t*,
    size_t embeddingFeaturesSize, double* result, size_t resultSize) {
    return Guard([&] {
        EnsureNoTextOrEmbeddings(textFeaturesSize, embeddingFeaturesSize);
        CalcHashedImpl(modelHandle, docCount, 0, H(modelHandle)->Model.Trees.GetTreeCount(), floatFeatures,
                       floatFeaturesSize, catFeatures, catFeaturesSize, result, resultSize);
    });
}

// ----------------------------------------------------------------------- specific class ----

#define CBAMD_SPECIFIC_CLASS(docs, call)                                                        \
    return Guard([&] {                                                                          \
        const size_t dim = static_cast<size_t>(H(modelHandle)->Model.Trees.ApproxDimension);    \
        std::vector<double> raw((docs) * dim);                                                  \
        if (!(call)) {                                                                          \
            throw TModelError(LastError);                                                       \
        }                                                                                       \
        SpecificClass(modelHandle, classId, raw, result, resultSize);                           \
    })

bool PredictSpecificClassFlat(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                              size_t floatFeaturesSize, int classId, double* result, size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(docCount, CalcModelPredictionFlat(modelHandle, docCount, floatFeatures, floatFeaturesSize,
                                                           raw.data(), raw.size()));
}

bool PredictSpecificClass(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                          size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, int classId,
                          double* result, size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(docCount, CalcModelPrediction(modelHandle, docCount, floatFeatures, floatFeaturesSize,
                                                       catFeatures, catFeaturesSize, raw.data(), raw.size()));
}

bool PredictSpecificClassText(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                              size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize,
                              const char*** textFeatures, size_t textFeaturesSize, int classId, double* result,
                              size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(docCount, CalcModelPredictionText(modelHandle, docCount, floatFeatures, floatFeaturesSize,
                                                           catFeatures, catFeaturesSize, textFeatures, textFeaturesSize,
                                                           raw.data(), raw.size()));
}

bool PredictSpecificClassTextAndEmbeddings(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures,
                                           size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize,
                                           const char*** textFeatures, size_t textFeaturesSize,
                                           const float*** embeddingFeatures, size_t* embeddingDimensions,
                                           size_t embeddingFeaturesSize, int classId, double* result,
                                           size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(docCount, CalcModelPredictionTextAndEmbeddings(
                                       modelHandle, docCount, floatFeatures, floatFeaturesSize, catFeatures,
                                       catFeaturesSize, textFeatures, textFeaturesSize, embeddingFeatures,
                                       embeddingDimensions, embeddingFeaturesSize, raw.data(), raw.size()));
}

bool PredictSpecificClassSingle(ModelCalcerHandle* modelHandle, const float* floatFeatures, size_t floatFeaturesSize,
                                const char** catFeatures, size_t catFeaturesSize, int classId, double* result,
                                size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(size_t(1), CalcModelPredictionSingle(modelHandle, floatFeatures, floatFeaturesSize, catFeatures,
                                                              catFeaturesSize, raw.data(), raw.size()));
}

bool PredictSpecificClassWithHashedCatFeatures(ModelCalcerHandle* modelHandle, size_t docCount,
                                               const float** floatFeatures, size_t floatFeaturesSize,
                                               const int** catFeatures, size_t catFeaturesSize, int classId,
                                               double* result, size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(docCount, CalcModelPredictionWithHashedCatFeatures(modelHandle, docCount, floatFeatures,
                                                                            floatFeaturesSize, catFeatures,
                                                                            catFeaturesSize, raw.data(), raw.size()));
}

bool PredictSpecificClassWithHashedCatFeaturesAndTextFeatures(ModelCalcerHandle* modelHandle, size_t docCount,
                                                              const float** floatFeatures, size_t floatFeaturesSize,
                                                              const int** catFeatures, size_t catFeaturesSize,
                                                              const char*** textFeatures, size_t textFeaturesSize,
                                                              int classId, double* result, size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(docCount, CalcModelPredictionWithHashedCatFeaturesAndTextFeatures(
                                       modelHandle, docCount, floatFeatures, floatFeaturesSize, catFeatures,
                                       catFeaturesSize, textFeatures, textFeaturesSize, raw.data(), raw.size()));
}

bool PredictSpecificClassWithHashedCatFeaturesAndTextAndEmbeddingFeatures(
    ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize,
    const int** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize,
    const float*** embeddingFeatures, size_t* embeddingDimensions, size_t embeddingFeaturesSize, int classId,
    double* result, size_t resultSize) {
    CBAMD_SPECIFIC_CLASS(docCount, CalcModelPredictionWithHashedCatFeaturesAndTextAndEmbeddingFeatures(
                                       modelHandle, docCount, floatFeatures, floatFeaturesSize, catFeatures,
                                       catFeaturesSize, textFeatures, textFeaturesSize, embeddingFeatures,
                                       embeddingDimensions, embeddingFeaturesSize, raw.data(), raw.size()));
}

// ------------------------------------------------------------------------------- hashes ----

int GetStringCatFeatureHash(const char* data, size_t size) {
    return CalcCatFeatureHashInt(data, size);
}

int GetIntegerCatFeatureHash(long long val) {
    char buf[32];
    const int n = std::snprintf(buf, sizeof(buf), "%lld", val);
    return CalcCatFeatureHashInt(buf, static_cast<size_t>(n));
}

// -------------------------------------------------------------------- model description ----

size_t GetFloatFeaturesCount(ModelCalcerHandle* modelHandle) {
    return static_cast<TModelHandle*>(modelHandle)->Model.Trees.GetNumFloatFeatures();
}
size_t GetCatFeaturesCount(ModelCalcerHandle* modelHandle) {
    return static_cast<TModelHandle*>(modelHandle)->Model.Trees.GetNumCatFeatures();
}
size_t GetTextFeaturesCount(ModelCalcerHandle*) { return 0; }
size_t GetEmbeddingFeaturesCount(ModelCalcerHandle*) { return 0; }
size_t GetTreeCount(ModelCalcerHandle* modelHandle) {
    return static_cast<TModelHandle*>(modelHandle)->Model.Trees.GetTreeCount();
}
size_t GetDimensionsCount(ModelCalcerHandle* modelHandle) {
    return static_cast<size_t>(static_cast<TModelHandle*>(modelHandle)->Model.Trees.ApproxDimension);
}
size_t GetPredictionDimensionsCount(ModelCalcerHandle* modelHandle) {
    return PredictionDims(*static_cast<TModelHandle*>(modelHandle));
}

bool GetFloatFeatureIndices(ModelCalcerHandle* modelHandle, size_t** indices, size_t* count) {
    std::vector<size_t> v;
    for (const auto& f : static_cast<TModelHandle*>(modelHandle)->Model.Trees.FloatFeatures) {
        v.push_back(static_cast<size_t>(f.FlatIndex));
    }
    return ReturnIndices(v, indices, count);
}
bool GetCatFeatureIndices(ModelCalcerHandle* modelHandle, size_t** indices, size_t* count) {
    std::vector<size_t> v;
    for (const auto& c : static_cast<TModelHandle*>(modelHandle)->Model.Trees.CatFeatures) {
        v.push_back(static_cast<size_t>(c.FlatIndex));
    }
    return ReturnIndices(v, indices, count);
}
bool GetTextFeatureIndices(ModelCalcerHandle*, size_t** indices, size_t* count) {
    return ReturnIndices({}, indices, count);
}
bool GetEmbeddingFeatureIndices(ModelCalcerHandle*, size_t** indices, size_t* count) {
    return ReturnIndices({}, indices, count);
}

bool CheckModelMetadataHasKey(ModelCalcerHandle* modelHandle, const char* keyPtr, size_t keySize) {
    const auto& info = static_cast<TModelHandle*>(modelHandle)->Model.ModelInfo;
    return info.count(std::string(keyPtr, keySize)) != 0;
}
size_t GetModelInfoValueSize(ModelCalcerHandle* modelHandle, const char* keyPtr, size_t keySize) {
    const auto& info = static_cast<TModelHandle*>(modelHandle)->Model.ModelInfo;
    auto it = info.find(std::string(keyPtr, keySize));
    return it == info.end() ? 0 : it->second.size();
}
const char* GetModelInfoValue(ModelCalcerHandle* modelHandle, const char* keyPtr, size_t keySize) {
    const auto& info = static_cast<TModelHandle*>(modelHandle)->Model.ModelInfo;
    auto it = info.find(std::string(keyPtr, keySize));
    return it == info.end() ? nullptr : it->second.c_str();
}

bool GetModelUsedFeaturesNames(ModelCalcerHandle* modelHandle, char*** featureNames, size_t* featureCount) {
    return Guard([&] {
        const auto names = H(modelHandle)->Model.GetUsedFeaturesNames();
        *featureNames = static_cast<char**>(std::malloc(sizeof(char*) * std::max<size_t>(names.size(), 1)));
        if (!*featureNames) {
            throw std::bad_alloc();
        }
        *featureCount = names.size();
        for (size_t i = 0; i < names.size(); ++i) {
            (*featureNames)[i] = static_cast<char*>(std::malloc(names[i].size() + 1));
            if (!(*featureNames)[i]) {
                for (size_t j = 0; j < i; ++j) {
                    std::free((*featureNames)[j]);
                }
                std::free(*featureNames);
                throw std::bad_alloc();
            }
            std::memcpy((*featureNames)[i], names[i].c_str(), names[i].size() + 1);
        }
    });
}

// ------------------------------------------------------------------ evaluator-level ABI ----

CbHipEvaluatorHandle* CbHipEvaluatorCreate(const CbHipModelArrays* model, int deviceId) {
    try {
        CBAMD_ENSURE(model != nullptr, "model arrays are null");
        TModelTrees trees;
        ArraysToTrees(*model, true, &trees);
        return new THipEvaluator(trees, deviceId);
    } catch (const std::exception& e) {
        LastError = e.what();
    }
    return nullptr;
}

void CbHipEvaluatorDelete(CbHipEvaluatorHandle* evaluator) {
    delete static_cast<THipEvaluator*>(evaluator);
}

size_t CbHipTreeCount(CbHipEvaluatorHandle* evaluator) {
    return static_cast<THipEvaluator*>(evaluator)->GetTreeCount();
}
int32_t CbHipApproxDimension(CbHipEvaluatorHandle* evaluator) {
    return static_cast<THipEvaluator*>(evaluator)->GetApproxDimension();
}
uint32_t CbHipBucketCount(CbHipEvaluatorHandle* evaluator) {
    return static_cast<THipEvaluator*>(evaluator)->GetBucketCount();
}
size_t CbHipQuantizedBytes(CbHipEvaluatorHandle* evaluator, size_t docCount) {
    return static_cast<THipEvaluator*>(evaluator)->QuantizedBytes(docCount);
}

bool CbHipQuantize(CbHipEvaluatorHandle* evaluator, const CbHipFeatures* deviceFeatures, size_t docCount,
                   void* deviceBins, void* hipStream) {
    return Guard([&] {
        E(evaluator)->QuantizeDevice(ToBatch(deviceFeatures), docCount, static_cast<uint8_t*>(deviceBins), hipStream);
    });
}

bool CbHipEvalQuantized(CbHipEvaluatorHandle* evaluator, const void* deviceBins, size_t docCount, size_t treeStart,
                        size_t treeEnd, double* deviceResults, void* hipStream) {
    return Guard([&] {
        E(evaluator)->EvalQuantizedDevice(static_cast<const uint8_t*>(deviceBins), docCount, treeStart, treeEnd,
                                          deviceResults, hipStream);
    });
}

bool CbHipEvalData(CbHipEvaluatorHandle* evaluator, const CbHipFeatures* deviceFeatures, size_t docCount,
                   size_t treeStart, size_t treeEnd, double* deviceResults, void* hipStream) {
    return Guard([&] {
        E(evaluator)->CalcDevice(ToBatch(deviceFeatures), docCount, treeStart, treeEnd, deviceResults, hipStream);
    });
}

bool CbHipEvalDataNoAlloc(CbHipEvaluatorHandle* evaluator, const CbHipFeatures* deviceFeatures, size_t docCount,
                          size_t treeStart, size_t treeEnd, double* deviceResults, void* hipStream) {
    return Guard([&] {
        E(evaluator)->CalcDeviceNoAlloc(ToBatch(deviceFeatures), docCount, treeStart, treeEnd, deviceResults, hipStream);
    });
}

bool CbHipLeafIndexesQuantized(CbHipEvaluatorHandle* evaluator, const void* deviceBins, size_t docCount,
                               size_t treeStart, size_t treeEnd, uint32_t* deviceIndexes, void* hipStream) {
    return Guard([&] {
        E(evaluator)->LeafIndexesQuantizedDevice(static_cast<const uint8_t*>(deviceBins), docCount, treeStart, treeEnd,
                                                 deviceIndexes, hipStream);
    });
}

bool CbHipExportQuantized(CbHipEvaluatorHandle* evaluator, const void* deviceBins, size_t docCount,
                          uint8_t* deviceReferenceLayout, void* hipStream) {
    return Guard([&] {
        E(evaluator)->ExportQuantizedDevice(static_cast<const uint8_t*>(deviceBins), docCount, deviceReferenceLayout,
                                            hipStream);
    });
}

bool CbHipApplyPredictionTypeDevice(CbHipEvaluatorHandle* evaluator, int predictionType, size_t docCount,
                                    const double* deviceRaw, double* deviceResult, void* hipStream) {
    return Guard([&] {
        E(evaluator)->ApplyPredictionTypeDevice(predictionType, 0, docCount, docCount, deviceRaw, deviceResult, hipStream);
    });
}

bool CbHipSynchronize(CbHipEvaluatorHandle* evaluator, void* hipStream) {
    return Guard([&] { E(evaluator)->Synchronize(hipStream); });
}

bool CbHipLastKernelTimes(CbHipEvaluatorHandle* evaluator, float* binarizeMs, float* evalMs) {
    return Guard([&] {
        const TKernelTimes t = E(evaluator)->LastKernelTimes();
        if (binarizeMs) {
            *binarizeMs = t.BinarizeMs;
        }
        if (evalMs) {
            *evalMs = t.EvalMs;
        }
    });
}

bool CbHipDescribeKernels(CbHipEvaluatorHandle* evaluator, int layout, size_t docCount, char* buffer, size_t bufferSize) {
    return Guard([&] {
        CBAMD_ENSURE(buffer != nullptr && bufferSize > 0, "description buffer is null");
        const std::string text = E(evaluator)->DescribeKernels(layout, docCount);
        CBAMD_ENSURE(text.size() < bufferSize, "description buffer is too small");
        std::memcpy(buffer, text.c_str(), text.size() + 1);
    });
}

bool CbHipEvaluatorSetSmallBatchSlicing(CbHipEvaluatorHandle* evaluator, bool enabled) {
    return Guard([&] { E(evaluator)->SetSmallBatchSlicing(enabled); });
}

bool CbHipSetSmallBatchSlicing(void* modelHandle, bool enabled) {
    return Guard([&] {
        TModelHandle* h = H(modelHandle);
        std::lock_guard<std::mutex> g(h->EvaluatorLock);
        h->SmallBatchSlicing = enabled;
        if (h->Evaluator) {
            h->Evaluator->SetSmallBatchSlicing(enabled);
        }
    });
}

CbHipEvaluatorHandle* CbHipGetEvaluator(void* modelHandle) {
    try {
        return &H(modelHandle)->GetEvaluator();
    } catch (const std::exception& e) {
        LastError = e.what();
    }
    return nullptr;
}

bool CbHipSetFeatureLayout(void* modelHandle, const uint32_t* floatFeatureIndexes, size_t floatFeatureIndexesSize,
                           const uint32_t* catFeatureIndexes, size_t catFeatureIndexesSize, const uint32_t* flatIndexes,
                           size_t flatIndexesSize) {
    return Guard([&] {
        TModelHandle* h = H(modelHandle);
        TFeatureLayout layout;
        if (floatFeatureIndexes != nullptr) {
            layout.HasFloatFeatureIndexes = true;
            layout.FloatFeatureIndexes.assign(floatFeatureIndexes, floatFeatureIndexes + floatFeatureIndexesSize);
        }
        if (catFeatureIndexes != nullptr) {
            layout.HasCatFeatureIndexes = true;
            layout.CatFeatureIndexes.assign(catFeatureIndexes, catFeatureIndexes + catFeatureIndexesSize);
        }
        if (flatIndexes != nullptr) {
            layout.HasFlatIndexes = true;
            layout.FlatIndexes.assign(flatIndexes, flatIndexes + flatIndexesSize);
        }
        // every position the evaluator would read must have an entry; checked now, not at the next call
        for (const auto& f : h->Model.Trees.FloatFeatures) {
            if (f.UsedInModel()) {
                layout.Remap(f);
            }
        }
        for (const auto& c : h->Model.Trees.CatFeatures) {
            if (c.UsedInModel) {
                layout.Remap(c);
            }
        }
        h->ResetEvaluator();
        h->Layout = std::move(layout);
    });
}

bool CbHipLoadModelFromArrays(void* modelHandle, const CbHipModelArrays* model) {
    return Guard([&] {
        CBAMD_ENSURE(model != nullptr, "model arrays are null");
        TFullModel m;
        ArraysToTrees(*model, true, &m.Trees);
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model = std::move(m);
    });
}

bool CbHipBuildObliviousModel(void* modelHandle, const CbHipModelArrays* features, int32_t treeCount,
                              const int32_t* treeDepths, const CbHipModelSplit* splits, const double* leafValues) {
    return Guard([&] {
        CBAMD_ENSURE(features != nullptr, "feature description is null");
        TModelTrees proto;
        ArraysToTrees(*features, false, &proto);
        TObliviousTreeBuilder builder(proto.FloatFeatures, proto.CatFeatures, proto.ApproxDimension);
        size_t splitPos = 0, leafPos = 0;
        for (int t = 0; t < treeCount; ++t) {
            CBAMD_ENSURE(treeDepths[t] >= 0 && treeDepths[t] < 31, "unsupported tree depth");
            std::vector<TModelSplit> treeSplits;
            for (int d = 0; d < treeDepths[t]; ++d) {
                treeSplits.push_back(ToSplit(splits[splitPos++]));
            }
            const size_t leafCount = (static_cast<size_t>(1) << treeDepths[t]) * proto.ApproxDimension;
            builder.AddTree(treeSplits, leafValues + leafPos, leafCount);
            leafPos += leafCount;
        }
        TFullModel m;
        builder.Build(&m.Trees);
        m.Trees.SetScaleAndBias(proto.Scale, proto.Bias);
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model = std::move(m);
    });
}

bool CbHipBuildNonSymmetricModel(void* modelHandle, const CbHipModelArrays* features, int32_t treeCount,
                                 const int32_t* treeNodeOffsets, const int32_t* nodeIsSplit,
                                 const CbHipModelSplit* nodeSplits, const int32_t* nodeLeft, const int32_t* nodeRight,
                                 const int64_t* nodeValueOffset, const double* nodeValues) {
    return Guard([&] {
        CBAMD_ENSURE(features != nullptr, "feature description is null");
        TModelTrees proto;
        ArraysToTrees(*features, false, &proto);
        TNonSymmetricTreeModelBuilder builder(proto.FloatFeatures, proto.CatFeatures, proto.ApproxDimension);
        const int dim = proto.ApproxDimension;
        for (int t = 0; t < treeCount; ++t) {
            const int begin = treeNodeOffsets[t], end = treeNodeOffsets[t + 1];
            CBAMD_ENSURE(begin >= 0 && end > begin, "tree without nodes");
            // children always come after their parent, so nodes are materialised back to front
            std::vector<std::unique_ptr<TNonSymmetricTreeNode>> nodes(end - begin);
            for (int i = end - 1; i >= begin; --i) {
                auto node = std::make_unique<TNonSymmetricTreeNode>();
                if (nodeIsSplit[i]) {
                    node->IsSplit = true;
                    node->SplitCondition = ToSplit(nodeSplits[i]);
                    const int l = nodeLeft[i], r = nodeRight[i];
                    CBAMD_ENSURE(l > i - begin && l < end - begin && r > i - begin && r < end - begin && l != r,
                                 "child index must follow its parent inside the tree");
                    CBAMD_ENSURE(nodes[l] && nodes[r], "tree node has two parents");
                    node->Left = std::move(nodes[l]);
                    node->Right = std::move(nodes[r]);
                } else {
                    node->Value.assign(nodeValues + nodeValueOffset[i], nodeValues + nodeValueOffset[i] + dim);
                }
                nodes[i - begin] = std::move(node);
            }
            builder.AddTree(*nodes[0]);
        }
        TFullModel m;
        builder.Build(&m.Trees);
        m.Trees.SetScaleAndBias(proto.Scale, proto.Bias);
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model = std::move(m);
    });
}

bool CbHipSaveModelToFile(void* modelHandle, const char* filename) {
    return Guard([&] {
        CBAMD_ENSURE(filename != nullptr, "file name is null");
        H(modelHandle)->Model.SaveToFile(filename);
    });
}

bool CbHipSaveModelToBuffer(void* modelHandle, void** buffer, size_t* size) {
    return Guard([&] {
        const std::string data = H(modelHandle)->Model.Save();
        *buffer = std::malloc(data.size());
        if (!*buffer) {
            throw std::bad_alloc();
        }
        std::memcpy(*buffer, data.data(), data.size());
        *size = data.size();
    });
}

bool CbHipConvertObliviousToAsymmetric(void* modelHandle) {
    return Guard([&] {
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model.Trees.ConvertObliviousToAsymmetric();
    });
}

bool CbHipSetScaleAndBias(void* modelHandle, double scale, const double* bias, size_t biasSize) {
    return Guard([&] {
        TModelHandle* h = H(modelHandle);
        h->ResetEvaluator();
        h->Model.Trees.SetScaleAndBias(scale, std::vector<double>(bias, bias + biasSize));
    });
}

bool CbHipSetModelInfo(void* modelHandle, const char* key, const char* value) {
    return Guard([&] {
        CBAMD_ENSURE(key != nullptr && value != nullptr, "null key or value");
        H(modelHandle)->Model.ModelInfo[key] = value;
    });
}

bool CbHipCalcFlatContiguous(void* modelHandle, const float* features, size_t docCount, size_t stride,
                             size_t treeStart, size_t treeEnd, double* result, size_t resultSize) {
    return Guard([&] {
        std::vector<const float*> rows(docCount);
        for (size_t d = 0; d < docCount; ++d) {
            rows[d] = features + d * stride;
        }
        CalcFlatImpl(modelHandle, docCount, treeStart, treeEnd, rows.data(), stride, result, resultSize);
    });
}

bool CbHipCalcLeafIndexesFlat(void* modelHandle, size_t docCount, const float** floatFeatures,
                              size_t floatFeaturesSize, size_t treeStart, size_t treeEnd, uint32_t* indexes,
                              size_t indexesSize) {
    return Guard([&] {
        TModelHandle& h = *H(modelHandle);
        CBAMD_ENSURE(treeStart <= treeEnd, "tree range is out of bounds");
        CBAMD_ENSURE(indexesSize == docCount * (treeEnd - treeStart),
                     "`treeLeafIndexes` size is insufficient: " + std::to_string(indexesSize) + " expected " +
                         std::to_string(docCount * (treeEnd - treeStart)));
        h.GetEvaluator().LeafIndexesHostRows(floatFeatures, floatFeaturesSize, true, nullptr, 0, docCount, treeStart,
                                             treeEnd, indexes);
    });
}

bool CbHipQuantizeFlat(void* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize,
                       uint8_t* bins, size_t binsSize) {
    return Guard([&] {
        TModelHandle& h = *H(modelHandle);
        CBAMD_ENSURE(binsSize == docCount * h.Model.Trees.EffectiveBinFeaturesBucketCount, "Not enough space to store quantized features");
        h.GetEvaluator().QuantizeHostRows(floatFeatures, floatFeaturesSize, true, nullptr, 0, docCount, bins);
    });
}

bool CbHipQuantizeWithHashedCatFeatures(void* modelHandle, size_t docCount, const float** floatFeatures,
                                        size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize,
                                        uint8_t* bins, size_t binsSize) {
    return Guard([&] {
        TModelHandle& h = *H(modelHandle);
        CBAMD_ENSURE(binsSize == docCount * h.Model.Trees.EffectiveBinFeaturesBucketCount, "Not enough space to store quantized features");
        h.GetEvaluator().QuantizeHostRows(floatFeaturesSize ? floatFeatures : nullptr, floatFeaturesSize, false,
                                          catFeaturesSize ? reinterpret_cast<const int32_t* const*>(catFeatures) : nullptr,
                                          catFeaturesSize, docCount, bins);
    });
}

uint32_t CbHipModelBucketCount(void* modelHandle) {
    return static_cast<TModelHandle*>(modelHandle)->Model.Trees.EffectiveBinFeaturesBucketCount;
}

void CbHipFastExpInplace(double* values, size_t count) {
    FastExpInplace(values, count);
}

bool CbHipApplyPredictionType(int predictionType, size_t dim, size_t docCount, const double* raw, double* result) {
    return Guard([&] {
        CBAMD_ENSURE(dim >= 1 && (docCount == 0 || (raw != nullptr && result != nullptr)), "invalid arguments");
        const auto type = static_cast<EApiPredictionType>(predictionType);
        if (type == APT_RAW_FORMULA_VAL) {
            std::copy(raw, raw + docCount * dim, result);
        } else {
            PostProcess(type, dim, docCount, raw, result);
        }
    });
}

}  // extern "C"
