// HIP evaluator of a CatBoost tree ensemble on one MI355X (gfx950).
// Takes the place of the reference's CUDA evaluation context
// (catboost/libs/model/cuda/evaluator.cuh:20-97: TGPUModelData, TGPUDataInput, TCudaQuantizedData,
// TGPUCatboostEvaluationContext) and of the host side of TGpuEvaluator
// (catboost/libs/model/cuda/evaluator.cpp:14-416). No HIP types appear in this header.
#pragma once

#include "model.h"

#include <memory>
#include <mutex>
#include <string>

namespace cbamd {

// Where a batch of documents lives. Pointers are device pointers for the *Device calls.
struct TFeatureBatch {
    enum ELayout {
        FlatRows = 0,     // Floats[doc * Stride + FlatIndex]; categorical hashes bit-cast in the same row
        FlatColumns = 1,  // Floats[FlatIndex * Stride + doc]
        SplitRows = 2,    // Floats[doc * Stride + Index], Cats[doc * CatStride + Index] (hashed)
    };
    ELayout Layout = FlatRows;
    const float* Floats = nullptr;
    size_t Stride = 0;
    const int32_t* Cats = nullptr;
    size_t CatStride = 0;
};

struct TKernelTimes {
    float BinarizeMs = 0.f;
    float EvalMs = 0.f;
};

class THipEvaluator {
public:
    // Uploads the model tables (model upload of cuda/evaluator.cpp:30-84, re-laid out as SoA).
    // `ctrTables`: the tables of the model's static CTR provider; needed when the model has CTR features.
    // `layout`: where the model's features sit in the callers' data (TFeatureLayout,
    // evaluation_interface.h:17-69); it is resolved into the device tables here, so it costs nothing per call
    THipEvaluator(const TModelTrees& trees, int deviceId, const std::vector<TCtrValueTable>* ctrTables = nullptr,
                  const TFeatureLayout* layout = nullptr);
    ~THipEvaluator();
    THipEvaluator(const THipEvaluator&) = delete;
    THipEvaluator& operator=(const THipEvaluator&) = delete;

    size_t GetTreeCount() const { return TreeCount; }
    int GetApproxDimension() const { return ApproxDimension; }
    uint32_t GetBucketCount() const { return BucketCount; }

    // Bytes of the quantized buffer for docCount documents:
    // ceil(docCount / 256) blocks x max(1, buckets) x 256 bytes.
    size_t QuantizedBytes(size_t docCount) const;

    // ---- device-resident data; `stream` is a hipStream_t (nullptr = the evaluator's own stream)
    void QuantizeDevice(const TFeatureBatch& batch, size_t docCount, uint8_t* bins, void* stream);
    void EvalQuantizedDevice(const uint8_t* bins, size_t docCount, size_t treeStart, size_t treeEnd,
                             double* results, void* stream);
    // Small batches on the register-resident kernels: the trees are cut into TreeSlicesFor(docCount) slices that
    // run on workgroups of their own and store raw sums into `partials` (TreeSliceScratchDoubles(docCount)
    // doubles, the caller's), which a second kernel adds up in slice order. One slice: the plain launch. The
    // sums of a slice are in tree order; adding the slices' sums rounds differently from one pass over all
    // trees (within the 1e-9 relative bar, the same for every call).
    uint32_t TreeSlicesFor(size_t docCount) const;
    size_t TreeSliceScratchDoubles(size_t docCount) const;
    void EvalQuantizedSlicedDevice(const uint8_t* bins, size_t docCount, double* results, double* partials, void* stream);
    // binarize + evaluate in one launch of a fused kernel, the bins in registers only; false (and nothing
    // launched) when the model, the batch layout or the tree range has no fused kernel
    // (anyBatchSize: also below the batch size from which the fused launch is the faster one)
    bool EvalRowsFusedDevice(const TFeatureBatch& batch, size_t docCount, size_t treeStart, size_t treeEnd,
                             double* results, void* stream, bool anyBatchSize = false);
    // index of the fused kernel tables that such a call would use (0 flat rows, 1 split rows), -1 when it takes
    // the two launches: the one test that EvalRowsFusedDevice, the host pipeline and DescribeKernels share
    int FusedLayoutFor(int layout, size_t stride, size_t docCount, size_t treeStart, size_t treeEnd, bool anyBatchSize) const;
    // Small batches (fewer than 256 workgroups of the register kernels) are cut into slices of the trees by the
    // calls that own their scratch memory; off: every sum is one pass in tree order, the CPU evaluator's
    // order of additions, at the price of the small-batch speed-up. Set it before the calls it should govern.
    void SetSmallBatchSlicing(bool on);
    bool SmallBatchSlicing() const;
    void LeafIndexesQuantizedDevice(const uint8_t* bins, size_t docCount, size_t treeStart, size_t treeEnd,
                                    uint32_t* indexes, void* stream);
    // bins in the reference's layout: blocks of 128 docs, [block][bucket][doc in block]
    void ExportQuantizedDevice(const uint8_t* bins, size_t docCount, uint8_t* referenceLayout, void* stream);
    // raw[doc * dim + k] of documents [firstDoc, firstDoc + docCount) of a batch of totalDocs -> the
    // prediction type (EApiPredictionType), as TEvalResultProcessor::PostprocessBlock does block by block
    // (catboost/libs/model/eval_processing.h:174-240); result: one value per document for Class, dim otherwise
    void ApplyPredictionTypeDevice(int predictionType, size_t firstDoc, size_t totalDocs, size_t docCount,
                                   const double* raw, double* result, void* stream);
    // binarize + evaluate with a scratch bin buffer owned by the evaluator; records kernel times
    void CalcDevice(const TFeatureBatch& batch, size_t docCount, size_t treeStart, size_t treeEnd,
                    double* results, void* stream);
    // the same two launches with the bins in a fixed array that every GPU holds from library load on:
    // no allocation, no synchronisation, nothing recorded. At most kNoAllocScratchBytes of bins per call
    // (QuantizedBytes tells); calls that overlap on one GPU share the array and race
    static constexpr size_t kNoAllocScratchBytes = size_t(32) << 20;
    void CalcDeviceNoAlloc(const TFeatureBatch& batch, size_t docCount, size_t treeStart, size_t treeEnd,
                           double* results, void* stream);
    void Synchronize(void* stream);
    TKernelTimes LastKernelTimes() const;
    // which kernels a whole-model call (CalcDevice, the host entry points) on docCount documents of the given
    // layout (TFeatureBatch::ELayout) and row stride (in values; 0: the model's own row width) launches:
    // "fused=<kernel>" or "binarize=<kernel>;evaluate=<kernel>". Calls for a range of the trees are not described.
    std::string DescribeKernels(int layout, size_t docCount, size_t stride = 0) const;

    // ---- host-resident data: stage -> binarize -> evaluate -> copy back, in document chunks.
    // rows[doc] points at rowLen floats (FlatRows / SplitRows) or columns[f] at docCount floats.
    // `predictionType` (EApiPredictionType) is applied on the device before the results are copied back;
    // `results` then holds one value per document for Class, dim values otherwise.
    void CalcHostRows(const float* const* rows, size_t rowLen, bool flat, const int32_t* const* catRows,
                      size_t catRowLen, size_t docCount, size_t treeStart, size_t treeEnd, double* results,
                      int predictionType = 0);
    void CalcHostColumns(const float* const* columns, size_t columnCount, size_t docCount, size_t treeStart,
                         size_t treeEnd, double* results, int predictionType = 0);
    void LeafIndexesHostRows(const float* const* rows, size_t rowLen, bool flat, const int32_t* const* catRows,
                             size_t catRowLen, size_t docCount, size_t treeStart, size_t treeEnd, uint32_t* indexes);
    void QuantizeHostRows(const float* const* rows, size_t rowLen, bool flat, const int32_t* const* catRows,
                          size_t catRowLen, size_t docCount, uint8_t* referenceLayout);

    struct TImpl;

private:
    void SetLastTimes(const TKernelTimes& times);
    std::unique_ptr<TImpl> Impl;
    size_t TreeCount = 0;
    int ApproxDimension = 1;
    uint32_t BucketCount = 0;
    TKernelTimes LastTimes;
    mutable std::mutex TimesLock;  // callers of one evaluator run side by side; the last one to finish leaves its times
};

// Number of HIP devices visible; throws TModelError when the runtime reports an error.
int GetHipDeviceCount();

}  // namespace cbamd
