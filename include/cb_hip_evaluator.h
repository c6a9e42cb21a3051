/*
 * Evaluator-level C ABI of the MI355X-native CatBoost evaluator (same libcatboostmodel.so).
 *
 * This is the seam an in-tree backend of the reference binds: an IModelEvaluator registered for
 * EFormulaEvaluatorType::GPU (catboost/libs/model/evaluation_interface.h:70-308,
 * catboost/libs/model/cuda/evaluator.cpp:419) that forwards to the calls below instead of to
 * TGPUCatboostEvaluationContext (catboost/libs/model/cuda/evaluator.cuh:80-97). Plain pointers and
 * sizes only. None of these symbols exists in the reference's export list; they carry the CbHip
 * prefix so the reference surface (c_api.h) stays intact.
 *
 * Error convention as in c_api.h: false / NULL + thread-local GetErrorString().
 */
#ifndef CB_HIP_EVALUATOR_H
#define CB_HIP_EVALUATOR_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#if defined(__cplusplus)
extern "C" {
#endif

typedef void CbHipEvaluatorHandle;

/* The tables of TModelTrees as flat arrays (catboost/libs/model/model.h:97-141 IModelTreeData,
 * catboost/libs/model/features.h:50-160). Nothing is retained after the call returns. */
typedef struct CbHipModelArrays {
    int32_t ApproxDimension;

    int32_t TreeCount;
    const int32_t* TreeSizes;        /* depth (oblivious) or node count (non-symmetric) */
    const int32_t* TreeStartOffsets;
    int32_t TreeSplitsCount;
    const int32_t* TreeSplits;       /* binary feature ids, CalcBinFeatures order (model.cpp:471-577) */

    int32_t FloatFeatureCount;       /* in model order, sorted by FlatIndex */
    const int32_t* FloatFeatureIndex;
    const int32_t* FloatFeatureFlatIndex;
    const int32_t* FloatFeatureHasNans;
    const int32_t* FloatFeatureNanTreatment; /* 0 AsIs, 1 AsFalse, 2 AsTrue (features.h:51-55) */
    const int32_t* FloatFeatureBorderOffsets; /* FloatFeatureCount + 1 */
    const float* FloatFeatureBorders;

    int32_t CatFeatureCount;
    const int32_t* CatFeatureIndex;
    const int32_t* CatFeatureFlatIndex;
    const int32_t* CatFeatureUsed;

    int32_t OneHotFeatureCount;
    const int32_t* OneHotCatFeatureIndex;
    const int32_t* OneHotValueOffsets; /* OneHotFeatureCount + 1 */
    const int32_t* OneHotValues;

    uint64_t LeafValuesCount;
    const double* LeafValues;        /* [tree][leaf * ApproxDimension + k] */

    int32_t StepNodeCount;           /* 0 for oblivious models */
    const uint16_t* StepNodes;       /* pairs (LeftSubtreeDiff, RightSubtreeDiff), model.h:78-95 */
    const uint32_t* NodeIdToLeafId;

    double Scale;
    const double* Bias;              /* ApproxDimension values */
} CbHipModelArrays;

enum ECbHipFeatureLayout {
    CBHIP_FLAT_ROWS = 0,    /* Floats[doc * Stride + FlatIndex], cat hashes bit-cast in the row */
    CBHIP_FLAT_COLUMNS = 1, /* Floats[FlatIndex * Stride + doc] */
    CBHIP_SPLIT_ROWS = 2,   /* Floats[doc * Stride + Index], Cats[doc * CatStride + Index] */
};

/* A batch of documents in DEVICE memory (TGPUDataInput, cuda/evaluator.cuh:38-51). */
typedef struct CbHipFeatures {
    int32_t Layout;
    const float* Floats;
    size_t Stride;
    const int32_t* Cats;
    size_t CatStride;
} CbHipFeatures;

/* Diagnostic switches, read from the environment whenever an evaluator is built (CbHipEvaluatorCreate, the
 * first prediction of a model handle, CbHipSetFeatureLayout), and only in a process whose environment has
 * CATBOOST_AMD_TEST_SWITCHES=1: without it none of the names below is looked at. They select between kernels
 * that return the same results and exist for tests and measurements.
 *   CATBOOST_AMD_REG_KERNEL=0        no register-resident assembly kernels (the LDS tile kernels instead)
 *   CATBOOST_AMD_REG_SIX=0           no six-bit form of the register-resident kernels and of the pair-tile kernel
 *   CATBOOST_AMD_REG_MIN_BUCKETS=n   only register-resident kernel shapes that hold n buckets or more
 *   CATBOOST_AMD_REG_SPLIT=0         a float feature with more than 127 used borders sends the model to the mixed
 *                                    (8-bit compare) kernels instead of taking two bins registers
 *   CATBOOST_AMD_SMALL_BATCH=0       the start value of CbHipSetSmallBatchSlicing is "off"
 *   CATBOOST_AMD_LEVEL_ORDER=0       register-resident kernels keep the model's order of a tree's levels
 *   CATBOOST_AMD_FUSED=0             binarize and evaluate always as two launches (no fused kernels)
 *   CATBOOST_AMD_PAIR_TILE=0         wide one-dimensional models (more buckets than an LDS tile of 256 documents
 *                                    holds): one tree per wave instead of two or four
 *   CATBOOST_AMD_ROW_TILE=0          models outside the register kernels whose 256-document tile fits LDS: the tile
 *                                    kernel that broadcasts a tree's levels from a lane instead of the one that
 *                                    keeps a tree's row in registers (depth 9 to 16: the plain kernel)
 *   CATBOOST_AMD_NS_WAVES=4|6|8|12|16 non-symmetric models walked out of LDS: only that many waves per workgroup
 *                                    (regions of 2048, 1536 or 1024 tree entries) instead of the most that hold
 *                                    the model's largest tree
 *   CATBOOST_AMD_CTR_TILE=0          the plain CTR kernel instead of the LDS tile one */

/* Model upload: validates the tables, derives buckets / repacked splits / leaf offsets and
 * copies SoA tables to device `deviceId` (takes the place of the TGpuEvaluator constructor,
 * cuda/evaluator.cpp:18-85). */
CbHipEvaluatorHandle* CbHipEvaluatorCreate(const CbHipModelArrays* model, int deviceId);
void CbHipEvaluatorDelete(CbHipEvaluatorHandle* evaluator);

size_t CbHipTreeCount(CbHipEvaluatorHandle* evaluator);
int32_t CbHipApproxDimension(CbHipEvaluatorHandle* evaluator);
uint32_t CbHipBucketCount(CbHipEvaluatorHandle* evaluator);

/* Bytes of a quantized buffer for docCount documents. */
size_t CbHipQuantizedBytes(CbHipEvaluatorHandle* evaluator, size_t docCount);

/* Binarize device-resident features into `deviceBins` (TGPUCatboostEvaluationContext::QuantizeData,
 * cuda/evaluator.cu:379-416; IModelEvaluator::Quantize). `hipStream` is a hipStream_t or NULL for
 * the evaluator's own stream; the call is asynchronous on that stream. Like CbHipEvalQuantized,
 * CbHipLeafIndexesQuantized, CbHipExportQuantized and CbHipApplyPredictionTypeDevice it only launches
 * kernels (no allocation, synchronisation or memset), so a caller may capture it into a HIP graph. */
bool CbHipQuantize(CbHipEvaluatorHandle* evaluator, const CbHipFeatures* deviceFeatures, size_t docCount,
                   void* deviceBins, void* hipStream);

/* Evaluate trees [treeStart, treeEnd) on quantized documents into deviceResults[doc * dim + k]
 * (EvalQuantizedData, cuda/evaluator.cu:344-377; IModelEvaluator::Calc(IQuantizedData*)).
 * Raw formula values: Scale * sum + Bias, bias only when treeStart == 0. Asynchronous. */
bool CbHipEvalQuantized(CbHipEvaluatorHandle* evaluator, const void* deviceBins, size_t docCount, size_t treeStart,
                        size_t treeEnd, double* deviceResults, void* hipStream);

/* Binarize + evaluate with the evaluator's own scratch bins (EvalData, cuda/evaluator.cu:418-428).
 * Synchronises the stream before returning and records the two kernel times. */
bool CbHipEvalData(CbHipEvaluatorHandle* evaluator, const CbHipFeatures* deviceFeatures, size_t docCount,
                   size_t treeStart, size_t treeEnd, double* deviceResults, void* hipStream);

/* CbHipEvalData for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. The bins of the
 * call sit in a fixed 32 MiB array that every GPU the library runs on holds until the process ends,
 * instead of the evaluator's grow-only scratch buffer; the call allocates nothing, waits for nothing
 * and records no kernel times: it only launches the binarize and evaluate kernels on `hipStream`
 * (NULL = the evaluator's own stream). Fails when CbHipQuantizedBytes(evaluator, docCount) exceeds
 * 32 MiB (the error names the largest document count for the model); a model that runs on a fused
 * kernel keeps its bins in registers there, uses no buffer and has no such limit (a batch of such a model
 * that does not fit the buffer takes the fused kernel at any size). The call never cuts the trees into
 * slices (it has no memory for partial sums): every sum is one pass in tree order, the CPU evaluator's order
 * of additions, so for small batches it may differ in the last bits from CbHipEvalData with slicing on, and
 * it has none of that call's small-batch speed-up. All calls on one GPU share the array, so calls that
 * overlap there (two streams, two threads, two evaluators) race; calls in stream order on one stream are
 * safe. */
bool CbHipEvalDataNoAlloc(CbHipEvaluatorHandle* evaluator, const CbHipFeatures* deviceFeatures, size_t docCount,
                          size_t treeStart, size_t treeEnd, double* deviceResults, void* hipStream);

/* Leaf indexes deviceIndexes[doc * (treeEnd - treeStart) + t] (IModelEvaluator::CalcLeafIndexes on
 * quantized data, evaluation_interface.h:289-294; unimplemented in cuda/evaluator.cpp:337-348). */
bool CbHipLeafIndexesQuantized(CbHipEvaluatorHandle* evaluator, const void* deviceBins, size_t docCount,
                               size_t treeStart, size_t treeEnd, uint32_t* deviceIndexes, void* hipStream);

/* Bins re-laid out as the reference's CPU quantized data: blocks of 128 documents,
 * [block][bucket][doc in block] (cpu/quantization.h:18-52, 357-365); docCount * buckets bytes. */
bool CbHipExportQuantized(CbHipEvaluatorHandle* evaluator, const void* deviceBins, size_t docCount,
                          uint8_t* deviceReferenceLayout, void* hipStream);

/* Raw formula values deviceRaw[doc * dim + k] (what CbHipEvalQuantized / CbHipEvalData write) -> the
 * prediction type `predictionType` (EApiPredictionType of c_api.h), on the device: what
 * TEvalResultProcessor::PostprocessBlock (catboost/libs/model/eval_processing.h:174-240) does after the CPU
 * evaluator and ProcessResultsImpl (cuda/evaluator.cu:262-296, Probability and Class of one dimension
 * only) after the CUDA one. deviceResult holds docCount values for APT_CLASS, docCount * dim otherwise;
 * it may be deviceRaw itself unless the type is APT_CLASS and the model has several dimensions. */
bool CbHipApplyPredictionTypeDevice(CbHipEvaluatorHandle* evaluator, int predictionType, size_t docCount,
                                    const double* deviceRaw, double* deviceResult, void* hipStream);

bool CbHipSynchronize(CbHipEvaluatorHandle* evaluator, void* hipStream);

/* hipEvent-measured duration of the binarize and evaluate kernels of the last CbHipEvalData or
 * host-level prediction call (summed over its chunks). A call that ran as one fused launch reports the
 * whole launch as evalMs and 0 as binarizeMs, whatever the entry point. */
bool CbHipLastKernelTimes(CbHipEvaluatorHandle* evaluator, float* binarizeMs, float* evalMs);

/* Which kernels a whole-model CbHipEvalData (or host entry point) call on docCount documents of `layout`
 * (ECbHipFeatureLayout) launches, as text: "fused=<kernel>" or "binarize=<kernel>;evaluate=<kernel>". For logs
 * and benchmarks; no counterpart in the reference. */
bool CbHipDescribeKernels(CbHipEvaluatorHandle* evaluator, int layout, size_t docCount, char* buffer, size_t bufferSize);

/* Batches of fewer than 256 workgroups (65 536 to 262 144 documents, by the kernel) are spread over the GPU by
 * cutting the trees into slices that run side by side; a slice adds its leaves in tree order and the slices'
 * sums are then added in slice order. The result is the same for every call and every batch size below that
 * limit, and differs in the last bits (inside 1e-9 relative) from the single pass in tree order that larger
 * batches, CbHipEvalQuantized and the CPU evaluator make (cpu/evaluator_impl.cpp:362-460; single document:
 * c_api.cpp:383-384). enabled = false turns the slices off for later calls: every sum is then one pass in tree
 * order whatever the batch size, at the price of the small-batch speed-up (C2 model, 4096 documents: 0.13
 * instead of 0.04 ms per call). No counterpart in the reference. The first form acts on a bare evaluator, the
 * second on a model handle (kept across Load* calls and rebuilt evaluators). Not to be called while another
 * thread evaluates on the same handle. */
bool CbHipEvaluatorSetSmallBatchSlicing(CbHipEvaluatorHandle* evaluator, bool enabled);
bool CbHipSetSmallBatchSlicing(void* modelHandle, bool enabled);

/* ---- extensions on a ModelCalcerHandle (c_api.h) ------------------------------------------ */

/* The evaluator bound to a model handle (created on first use on the enabled device). Owned by
 * the handle; invalidated by the next Load* / CbHipLoad* / CbHipBuild* call on it. */
CbHipEvaluatorHandle* CbHipGetEvaluator(void* modelHandle);

/* IModelEvaluator::SetFeatureLayout (catboost/libs/model/evaluation_interface.h:17-82; the reference's
 * CUDA evaluator refuses layouts, cuda/evaluator.cpp:129,176): tells where the model's features sit in
 * the caller's data. A feature whose position in the model is p is then read at floatFeatureIndexes[p]
 * or catFeatureIndexes[p] of the separate float / categorical arrays, and at flatIndexes[p] of flat
 * vectors (TFeatureLayout::GetRemappedPosition). A null list leaves those positions as the model has
 * them; three nulls remove the layout. Every used feature needs an entry in a list that is given. The
 * vector sizes every Calc* then asks for are the largest position read plus one. Applies to all later
 * calls on the handle, host and device entry points alike (the handle's evaluator is rebuilt: pointers
 * from CbHipGetEvaluator are invalidated); a Load* call keeps it. */
bool CbHipSetFeatureLayout(void* modelHandle, const uint32_t* floatFeatureIndexes, size_t floatFeatureIndexesSize,
                           const uint32_t* catFeatureIndexes, size_t catFeatureIndexesSize, const uint32_t* flatIndexes,
                           size_t flatIndexesSize);

/* Install a model given as raw tables (the AddBinTree / AddLeafValue route of TModelTrees,
 * catboost/libs/model/model.cpp:238-254). */
bool CbHipLoadModelFromArrays(void* modelHandle, const CbHipModelArrays* model);

/* A split of a tree under construction (TModelSplit, catboost/libs/model/split.h:27-100). */
typedef struct CbHipModelSplit {
    int32_t Type;         /* 0 float feature, 2 one-hot feature (ESplitType, split.h:20-25) */
    int32_t FeatureIndex; /* float feature index or categorical feature index */
    float Border;
    int32_t Value;        /* hashed category for one-hot splits */
} CbHipModelSplit;

/* TObliviousTreeBuilder (catboost/libs/model/model_build_helper.cpp:128-204): feature descriptions
 * come from `features` (borders ignored: only borders used by splits are kept), tree t has
 * treeDepths[t] splits taken in order from `splits` and (1 << depth) * ApproxDimension leaf
 * values taken in order from `leafValues` ([leaf * dim + k]). Scale and Bias of `features` apply. */
bool CbHipBuildObliviousModel(void* modelHandle, const CbHipModelArrays* features, int32_t treeCount,
                              const int32_t* treeDepths, const CbHipModelSplit* splits, const double* leafValues);

/* TNonSymmetricTreeModelBuilder (model_build_helper.cpp:206-304). Trees arrive as node arrays:
 * node i of tree t is a split (nodeIsSplit != 0, children nodeLeft / nodeRight as indexes into
 * the same tree's node range, condition nodeSplits[i]) or a leaf whose ApproxDimension values
 * start at nodeValues[nodeValueOffset[i]]. treeNodeOffsets has treeCount + 1 entries; the root
 * of a tree is its first node. */
bool CbHipBuildNonSymmetricModel(void* modelHandle, const CbHipModelArrays* features, int32_t treeCount,
                                 const int32_t* treeNodeOffsets, const int32_t* nodeIsSplit,
                                 const CbHipModelSplit* nodeSplits, const int32_t* nodeLeft, const int32_t* nodeRight,
                                 const int64_t* nodeValueOffset, const double* nodeValues);

/* The "json" model format: what ReadModel(path, EModelType::Json) does for the reference's bindings
 * (catboost/libs/model/model_export/json_model_helpers.cpp:583-608 ConvertJsonToCatboostModel; the JVM
 * binding's loadModel(stream, "json")). Float, one-hot categorical and CTR features with their tables
 * (CtrDataFromJson, :531-580), oblivious and non-symmetric trees, scale and bias. As in the reference
 * the format loses TModelCtrBase::TargetBorderClassifierIdx and the fraction of a mean CTR's sum. */
bool CbHipLoadFullModelFromJsonFile(void* modelHandle, const char* filename);
bool CbHipLoadFullModelFromJsonBuffer(void* modelHandle, const void* jsonText, size_t jsonTextSize);

/* TFullModel::Save (catboost/libs/model/model.cpp:1113-1163). The buffer is malloc'd. */
bool CbHipSaveModelToFile(void* modelHandle, const char* filename);
bool CbHipSaveModelToBuffer(void* modelHandle, void** buffer, size_t* size);
/* TModelTrees::ConvertObliviousToAsymmetric (model.cpp:634-674) */
bool CbHipConvertObliviousToAsymmetric(void* modelHandle);
/* TFullModel::SetScaleAndBias (model.cpp:700-709) */
bool CbHipSetScaleAndBias(void* modelHandle, double scale, const double* bias, size_t biasSize);
bool CbHipSetModelInfo(void* modelHandle, const char* key, const char* value);

/* Host-resident contiguous row-major matrix features[doc * stride + flat index]: one bulk copy
 * instead of one pointer per document. */
bool CbHipCalcFlatContiguous(void* modelHandle, const float* features, size_t docCount, size_t stride,
                             size_t treeStart, size_t treeEnd, double* result, size_t resultSize);
/* TFullModel::CalcLeafIndexes over flat rows (model.h:1280-1302): indexes[doc * trees + t]. */
bool CbHipCalcLeafIndexesFlat(void* modelHandle, size_t docCount, const float** floatFeatures,
                              size_t floatFeaturesSize, size_t treeStart, size_t treeEnd, uint32_t* indexes,
                              size_t indexesSize);
/* Bins of flat rows in the reference layout; binsSize must equal docCount * bucket count. */
bool CbHipQuantizeFlat(void* modelHandle, size_t docCount, const float** floatFeatures, size_t floatFeaturesSize,
                       uint8_t* bins, size_t binsSize);
/* Same for split float / hashed categorical rows. */
bool CbHipQuantizeWithHashedCatFeatures(void* modelHandle, size_t docCount, const float** floatFeatures,
                                        size_t floatFeaturesSize, const int** catFeatures, size_t catFeaturesSize,
                                        uint8_t* bins, size_t binsSize);
uint32_t CbHipModelBucketCount(void* modelHandle);

/* ---- prediction types on host arrays (no GPU involved; CbHipApplyPredictionTypeDevice is the
 * device version) ----------------------------------------------------------------------- */

/* values[i] = exp(values[i]) as NCB::FastExpWithInfInplace computes it on an AVX2 host
 * (catboost/libs/helpers/math_utils.cpp:14-27, contrib/libs/fmath/fmath.hpp:565-648). */
void CbHipFastExpInplace(double* values, size_t count);
/* Raw formula values raw[doc * dim + k] -> the prediction type, block by block like
 * TEvalResultProcessor::PostprocessBlock (catboost/libs/model/eval_processing.h:174-240).
 * `result` holds docCount values for APT_CLASS, docCount * dim otherwise. */
bool CbHipApplyPredictionType(int predictionType, size_t dim, size_t docCount, const double* raw, double* result);

#if defined(__cplusplus)
}
#endif
#endif
