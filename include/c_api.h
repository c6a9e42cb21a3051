/*
 * C ABI of the MI355X-native CatBoost model evaluator: libcatboostmodel.so.
 *
 * Every symbol, signature and enum value below is the one the reference exports from its own
 * libcatboostmodel (catboost/libs/model_interface/c_api.h, export list
 * catboost/libs/model_interface/calcer.exports), so that programs and bindings linked against the
 * reference library (wrapped_calcer.h, Rust catboost-sys, the Node addon, .NET P/Invoke,
 * ClickHouse) run unchanged on top of this one. Each declaration names the reference declaration
 * it takes the place of as c_api.h:LINE.
 *
 * Evaluation always runs on the GPU through hand-written HIP kernels; there is no CPU evaluator in
 * this library. A call that needs the GPU fails (false + GetErrorString()) when no HIP device is
 * usable. EnableGPUEvaluation selects the device up front; without it the first prediction call
 * binds the model to device 0.
 *
 * Conventions (as in the reference, catboost/libs/model_interface/c_api.cpp:33-37, 263-291):
 * functions returning bool report failure with false and a thread-local message readable through
 * GetErrorString(); arrays returned through T** are malloc'd and freed by the caller with free().
 */
#ifndef CATBOOST_AMD_C_API_H
#define CATBOOST_AMD_C_API_H

#include <stdbool.h>
#include <stddef.h>

#define CATBOOST_APPLIER_MAJOR 1 /* c_api.h:7 */
#define CATBOOST_APPLIER_MINOR 2 /* c_api.h:8 */
#define CATBOOST_APPLIER_FIX 10  /* c_api.h:9 */

#if defined(__cplusplus)
extern "C" {
#endif

#define CATBOOST_API

typedef void DataWrapperHandle;  /* c_api.h:26 */
typedef void DataProviderHandle; /* c_api.h:28 */
typedef void ModelCalcerHandle;  /* c_api.h:48 */

enum EApiPredictionType { /* c_api.h:50-57 */
    APT_RAW_FORMULA_VAL = 0,
    APT_EXPONENT = 1,
    APT_RMSE_WITH_UNCERTAINTY = 2,
    APT_PROBABILITY = 3,
    APT_CLASS = 4,
    APT_MULTI_PROBABILITY = 5,
};

enum ECatBoostApiFormulaEvaluatorType { /* c_api.h:59-62 */
    CBA_FET_CPU = 0,
    CBA_FET_GPU = 1,
};

/* ---- data wrapper (c_api.h:34-46). The evaluator takes raw feature matrices; these entry
 * points are exported for link compatibility, create nothing and BuildDataProvider returns NULL. */
CATBOOST_API DataWrapperHandle* DataWrapperCreate(size_t docsCount);
CATBOOST_API void DataWrapperDelete(DataWrapperHandle* dataWrapperHandle);
CATBOOST_API void AddFloatFeatures(DataWrapperHandle* dataWrapperHandle, const float** floatFeatures, size_t floatFeaturesSize);
CATBOOST_API void AddCatFeatures(DataWrapperHandle* dataWrapperHandle, const char*** catFeatures, size_t catFeaturesSize);
CATBOOST_API void AddTextFeatures(DataWrapperHandle* dataWrapperHandle, const char*** textFeatures, size_t textFeaturesSize);
CATBOOST_API void AddEmbeddingFeatures(DataWrapperHandle* dataWrapperHandle, const float*** embeddingFeatures, size_t* embeddingDimensions, size_t embeddingFeaturesSize);
CATBOOST_API DataProviderHandle* BuildDataProvider(DataWrapperHandle* dataWrapperHandle);

/* ---- handle life cycle and errors */
CATBOOST_API ModelCalcerHandle* ModelCalcerCreate(void);            /* c_api.h:68 */
CATBOOST_API void ModelCalcerDelete(ModelCalcerHandle* modelHandle); /* c_api.h:74 */
CATBOOST_API const char* GetErrorString(void);                      /* c_api.h:84 */

/* ---- model loading: .cbm files / buffers ("CBM1" + flatbuffer + the tables of the static CTR
 * provider). Models with text or embedding features are refused with an error. */
CATBOOST_API bool LoadFullModelFromFile(ModelCalcerHandle* modelHandle, const char* filename); /* c_api.h:92 */
CATBOOST_API bool LoadFullModelFromBuffer(ModelCalcerHandle* modelHandle, const void* binaryBuffer, size_t binaryBufferSize); /* c_api.h:103 */
/* The tables are copied to the GPU, so nothing points into the caller's buffer after return. */
CATBOOST_API bool LoadFullModelZeroCopy(ModelCalcerHandle* modelHandle, const void* binaryBuffer, size_t binaryBufferSize); /* c_api.h:116 */

/* ---- evaluator selection */
CATBOOST_API bool EnableGPUEvaluation(ModelCalcerHandle* modelHandle, int deviceId); /* c_api.h:124 */
CATBOOST_API bool GetSupportedEvaluatorTypes(ModelCalcerHandle* modelHandle, enum ECatBoostApiFormulaEvaluatorType** formulaEvaluatorTypes, size_t* formulaEvaluatorTypesCount); /* c_api.h:135 */
CATBOOST_API bool SetPredictionType(ModelCalcerHandle* modelHandle, enum EApiPredictionType predictionType); /* c_api.h:144 */
CATBOOST_API bool SetPredictionTypeString(ModelCalcerHandle* modelHandle, const char* predictionTypeStr);    /* c_api.h:149 */

/* ---- predictions. result[doc * dims + k]; resultSize must equal docCount * prediction dims.
 * Flat: floatFeatures[doc][flat feature index], categorical hashes bit-cast into their float slot. */
CATBOOST_API bool CalcModelPredictionFlat(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, double* result, size_t resultSize); /* c_api.h:165 */
CATBOOST_API bool CalcModelPredictionFlatStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd, const float** floatFeatures, size_t floatFeaturesSize, double* result, size_t resultSize); /* c_api.h:188 */
/* Transposed: floatFeatures[flat feature index][doc] */
CATBOOST_API bool CalcModelPredictionFlatTransposed(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, double* result, size_t resultSize); /* c_api.h:208 */
CATBOOST_API bool CalcModelPredictionFlatTransposedStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd, const float** floatFeatures, size_t floatFeaturesSize, double* result, size_t resultSize); /* c_api.h:230 */
/* floatFeatures[doc][float feature index], catFeatures[doc][cat feature index] as C strings */
CATBOOST_API bool CalcModelPrediction(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, double* result, size_t resultSize); /* c_api.h:252 */
CATBOOST_API bool CalcModelPredictionStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, double* result, size_t resultSize); /* c_api.h:276 */
CATBOOST_API bool CalcModelPredictionSingle(ModelCalcerHandle* modelHandle, const float* floatFeatures, size_t floatFeaturesSize, const char** catFeatures, size_t catFeaturesSize, double* result, size_t resultSize); /* c_api.h:418 */
CATBOOST_API bool CalcModelPredictionSingleStaged(ModelCalcerHandle* modelHandle, size_t treeStart, size_t treeEnd, const float* floatFeatures, size_t floatFeaturesSize, const char** catFeatures, size_t catFeaturesSize, double* result, size_t resultSize); /* c_api.h:441 */
/* catFeatures[doc][cat feature index] already hashed */
CATBOOST_API bool CalcModelPredictionWithHashedCatFeatures(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize, double* result, size_t resultSize); /* c_api.h:462 */

/* ---- text / embedding entry points (c_api.h:302-402, 469-484): models with such features cannot
 * be loaded, so these work exactly when no text / embedding feature is passed (sizes 0) and fail
 * with "not supported" otherwise. */
CATBOOST_API bool CalcModelPredictionText(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, double* result, size_t resultSize);
CATBOOST_API bool CalcModelPredictionTextStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, double* result, size_t resultSize);
CATBOOST_API bool CalcModelPredictionTextAndEmbeddings(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, const float*** embeddingFeatures, size_t* embeddingDimensions, size_t embeddingFeaturesSize, double* result, size_t resultSize);
CATBOOST_API bool CalcModelPredictionTextAndEmbeddingsStaged(ModelCalcerHandle* modelHandle, size_t docCount, size_t treeStart, size_t treeEnd, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, const float*** embeddingFeatures, size_t* embeddingDimensions, size_t embeddingFeaturesSize, double* result, size_t resultSize);
CATBOOST_API bool CalcModelPredictionWithHashedCatFeaturesAndTextFeatures(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, double* result, size_t resultSize);
CATBOOST_API bool CalcModelPredictionWithHashedCatFeaturesAndTextAndEmbeddingFeatures(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, const float*** embeddingFeatures, size_t* embeddingDimensions, size_t embeddingFeaturesSize, double* result, size_t resultSize);

/* ---- one class of a multi-dimensional model (c_api.h:492-558); resultSize == docCount */
CATBOOST_API bool PredictSpecificClassFlat(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, int classId, double* result, size_t resultSize);
CATBOOST_API bool PredictSpecificClass(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, int classId, double* result, size_t resultSize);
CATBOOST_API bool PredictSpecificClassText(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, int classId, double* result, size_t resultSize);
CATBOOST_API bool PredictSpecificClassTextAndEmbeddings(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const char*** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, const float*** embeddingFeatures, size_t* embeddingDimensions, size_t embeddingFeaturesSize, int classId, double* result, size_t resultSize);
CATBOOST_API bool PredictSpecificClassSingle(ModelCalcerHandle* modelHandle, const float* floatFeatures, size_t floatFeaturesSize, const char** catFeatures, size_t catFeaturesSize, int classId, double* result, size_t resultSize);
CATBOOST_API bool PredictSpecificClassWithHashedCatFeatures(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize, int classId, double* result, size_t resultSize);
CATBOOST_API bool PredictSpecificClassWithHashedCatFeaturesAndTextFeatures(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, int classId, double* result, size_t resultSize);
CATBOOST_API bool PredictSpecificClassWithHashedCatFeaturesAndTextAndEmbeddingFeatures(ModelCalcerHandle* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize, const char*** textFeatures, size_t textFeaturesSize, const float*** embeddingFeatures, size_t* embeddingDimensions, size_t embeddingFeaturesSize, int classId, double* result, size_t resultSize);

/* ---- categorical hashes */
CATBOOST_API int GetStringCatFeatureHash(const char* data, size_t size); /* c_api.h:566 */
CATBOOST_API int GetIntegerCatFeatureHash(long long val);               /* c_api.h:575 */

/* ---- model description (c_api.h:581-687) */
CATBOOST_API size_t GetFloatFeaturesCount(ModelCalcerHandle* modelHandle);
CATBOOST_API bool GetFloatFeatureIndices(ModelCalcerHandle* modelHandle, size_t** indices, size_t* count);
CATBOOST_API size_t GetCatFeaturesCount(ModelCalcerHandle* modelHandle);
CATBOOST_API bool GetCatFeatureIndices(ModelCalcerHandle* modelHandle, size_t** indices, size_t* count);
CATBOOST_API size_t GetTextFeaturesCount(ModelCalcerHandle* modelHandle);
CATBOOST_API bool GetTextFeatureIndices(ModelCalcerHandle* modelHandle, size_t** indices, size_t* count);
CATBOOST_API size_t GetEmbeddingFeaturesCount(ModelCalcerHandle* modelHandle);
CATBOOST_API bool GetEmbeddingFeatureIndices(ModelCalcerHandle* modelHandle, size_t** indices, size_t* count);
CATBOOST_API size_t GetTreeCount(ModelCalcerHandle* modelHandle);
CATBOOST_API size_t GetDimensionsCount(ModelCalcerHandle* modelHandle);
CATBOOST_API size_t GetPredictionDimensionsCount(ModelCalcerHandle* modelHandle);
CATBOOST_API bool CheckModelMetadataHasKey(ModelCalcerHandle* modelHandle, const char* keyPtr, size_t keySize);
CATBOOST_API size_t GetModelInfoValueSize(ModelCalcerHandle* modelHandle, const char* keyPtr, size_t keySize);
CATBOOST_API const char* GetModelInfoValue(ModelCalcerHandle* modelHandle, const char* keyPtr, size_t keySize);
CATBOOST_API bool GetModelUsedFeaturesNames(ModelCalcerHandle* modelHandle, char*** featureNames, size_t* featureCount);

#if defined(__cplusplus)
}
#endif
#endif
