// Device code of the HIP evaluator (gfx950, wave64).
//
// Quantized layout ("bins"): documents are grouped in blocks of 256; inside a block one wave
// lane owns the four documents {lane, lane + 64, lane + 128, lane + 192} and keeps their bins of
// one bucket in one dword, so
//     bins[((block * buckets + bucket) * 64 + lane) * 4 + j]  is the bin of document
//     block * 256 + j * 64 + lane.
// A wave reads or writes the 256 bytes of one (block, bucket) pair with a single coalesced dword
// access per lane, and per-document results (doc = base + j * 64 + lane) are coalesced as well.
// Bin values are those of the reference's BinarizeFeatures (cpu/quantization.h:333-529):
// float bucket -> number of borders strictly below the value, one-hot bucket -> 1 + index of the
// matching value (0 when none).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace cbamd::dev {

constexpr int kDocsPerBlock = 256;
constexpr int kWave = 64;
constexpr int kBucketFlagNanToInf = 1;  // HasNans && NanValueTreatment == AsTrue
constexpr int kBucketFlagOneHot = 2;
constexpr uint32_t kXcdCount = 8;       // accelerator dies of an MI355X, each with its own L2
constexpr int kBucketTile = 16;         // buckets binarized per workgroup (small: ~20 KB of LDS, 7 workgroups per CU)
constexpr int kMaxBucketValues = 256;   // 254 values, padded

constexpr int kBucketFlagCtr = 4;        // bucket of a CTR feature: filled by CtrBinarizeKernel

struct TBinarizeTables {
    uint32_t BucketCount;          // buckets the binarize kernels fill: float and one-hot features
    uint32_t BucketPitch;          // buckets per document block in `bins` (those and the CTR buckets)
    const uint32_t* BucketSrc;     // source column of the bucket in the chosen layout
    const uint32_t* BucketOffset;  // [BucketCount + 1] offsets into Values
    const uint32_t* BucketFlags;
    const uint32_t* Values;        // float borders (sorted ascending) or one-hot values, as bits
    // float buckets, row binarize kernel: a uniform grid of kLutCells cells over the bucket's borders
    // gives the search a start and a short window instead of the whole border array
    const uint4* Grid;             // per bucket: lowest border, cells per unit (both fp32 bits), search steps, 0
    const uint32_t* Lut;           // per bucket kLutCells bytes: first border the search looks at, per cell
};

struct TTreeTables {
    const uint32_t* Splits;       // per tree split / node: bucket | xorMask << 16 | splitIdx << 24
    const uint32_t* TreeStart;    // first split (oblivious) or first node (non-symmetric) of a tree
    const uint32_t* TreeSize;     // depth (oblivious) or node count (non-symmetric)
    const uint32_t* FirstLeaf;    // index of the tree's first value in Leaves
    const uint32_t* StepNodes;    // non-symmetric: left diff | right diff << 16
    const uint32_t* NodeToLeaf;   // non-symmetric: value index of a terminal node
    const double* Leaves;
    const double* Bias;
    double Scale;
    int Dim;
};

// number of sorted borders strictly below v; `borders` holds 1 << LOG2P entries, the real ones
// first and +inf after them
template <int LOG2P>
__device__ __forceinline__ uint32_t CountBelow(const uint32_t* borders, float v) {
    const uint32_t* p = borders;
#pragma unroll
    for (uint32_t step = 1u << (LOG2P - 1); step >= 1; step >>= 1) {
        const float b = __uint_as_float(p[step - 1]);
        p = (b < v) ? p + step : p;
    }
    return static_cast<uint32_t>(p - borders);
}

constexpr int kLutCells = 256;

// Cell of a value in a bucket's grid: (v - lo) * scale, truncated, negative and NaN to 0, at most
// kLutCells - 1. Subtract and multiply are separate roundings, and the host computes the borders'
// cells with the very same operations (GridCell in hip_evaluator.hip), so cell(b) <= cell(v)
// whenever b <= v: every border in a lower cell is below v, every border in a higher cell above.
__device__ __forceinline__ uint32_t GridCell(float v, float lo, float scale) {
    const float t = __fmul_rn(__fsub_rn(v, lo), scale);
    uint32_t c;
    asm("v_cvt_u32_f32 %0, %1" : "=v"(c) : "v"(t));  // saturating, NaN -> 0
    return min(c, static_cast<uint32_t>(kLutCells - 1));
}

// Number of borders strictly below v, searching only the window the value's cell points at:
// `lut[cell]` borders are known to be below v, the next 2 * topStep - 1 entries hold every border of
// the cell (and then higher ones or the +inf padding, which never count).
__device__ __forceinline__ uint32_t CountBelowInCell(const uint32_t* borders, const uint8_t* lut, float lo, float scale,
                                                     uint32_t topStep, float v) {
    const uint32_t* p = borders + lut[GridCell(v, lo, scale)];
    for (uint32_t step = topStep; step >= 1; step >>= 1) {
        const float b = __uint_as_float(p[step - 1]);
        p = (b < v) ? p + step : p;
    }
    return static_cast<uint32_t>(p - borders);
}

__device__ __forceinline__ uint32_t OneHotBin(const uint32_t* values, uint32_t count, uint32_t v) {
    uint32_t bin = 0;
    for (uint32_t i = 0; i < count; ++i) {
        bin |= (values[i] == v) ? (i + 1) : 0u;
    }
    return bin;
}

constexpr int kTilePitch = kDocsPerBlock + 1;  // dwords per bucket row of the transposed tile

// Row-major input: floats[doc * stride + column]; hashed categorical values either bit-cast in
// the same row (CATS_MATRIX == false) or in cats[doc * catStride + column].
// One workgroup owns kBucketTile buckets and walks `blocksPerGroup` consecutive 256-document
// blocks: the bucket values stay in LDS (1 << LOG2P slots per bucket, every bucket of the model
// has fewer values than that), each block's 256 x kBucketTile feature tile is fetched with row-contiguous
// loads into registers one block ahead, transposed through a padded LDS tile and binarized by a
// branch-free binary search; a wave writes the 256 bytes of one (block, bucket) pair at once.
// Rows past the last document are read as the last document (their bins are never used).
// grid = ceil(doc blocks / blocksPerGroup) * ceil(buckets / kBucketTile), block = 256 threads,
// dynamic LDS = (kBucketTile << LOG2P) * 4 + kBucketTile * kLutCells + kBucketTile * kTilePitch * 4 bytes.
template <int LOG2P, bool CATS_MATRIX>
__global__ __launch_bounds__(256) void BinarizeRowsKernel(const float* __restrict__ floats, uint32_t stride,
                                                          const int32_t* __restrict__ cats, uint32_t catStride,
                                                          uint32_t docCount, TBinarizeTables tab,
                                                          uint32_t blocksPerGroup, uint32_t* __restrict__ bins) {
    constexpr uint32_t kSlots = 1u << LOG2P;
    constexpr int kRowsPerPass = 256 / kBucketTile;        // rows per pass of 256 threads
    constexpr int kPasses = kDocsPerBlock / kRowsPerPass;  // values per thread and block
    extern __shared__ uint32_t sBinarize[];
    uint32_t* sValues = sBinarize;                           // [kBucketTile][kSlots]
    uint32_t* sLut = sBinarize + kBucketTile * kSlots;       // [kBucketTile][kLutCells / 4]
    uint32_t* sTile = sLut + kBucketTile * (kLutCells / 4);  // [kBucketTile][kTilePitch]

    const uint32_t tid = threadIdx.x;
    const uint32_t tileCount = (tab.BucketCount + kBucketTile - 1) / kBucketTile;
    // Workgroups go round-robin to the 8 XCDs, each with an L2 of its own. The bucket tiles of one
    // document group share cache lines (a row piece of 128 bytes is not line aligned), so they are
    // given to workgroups of the same XCD that start one after the other: XCD x owns a contiguous
    // range of the work list.
    const uint32_t perXcd = gridDim.x / kXcdCount, extra = gridDim.x % kXcdCount;
    const uint32_t xcd = blockIdx.x % kXcdCount;
    const uint32_t work = xcd * perXcd + min(xcd, extra) + blockIdx.x / kXcdCount;
    const uint32_t b0 = (work % tileCount) * kBucketTile;
    const uint32_t nb = min(static_cast<uint32_t>(kBucketTile), tab.BucketCount - b0);
    const uint32_t blockCount = (docCount + kDocsPerBlock - 1) / kDocsPerBlock;
    const uint32_t blockBegin = (work / tileCount) * blocksPerGroup;
    const uint32_t blockEnd = min(blockBegin + blocksPerGroup, blockCount);

    for (uint32_t i = tid; i < kBucketTile * kSlots; i += 256) {
        const uint32_t bb = i >> LOG2P, k = i & (kSlots - 1);
        uint32_t v = 0x7f800000u;  // +inf
        if (bb < nb) {
            const uint32_t off = tab.BucketOffset[b0 + bb];
            const uint32_t cnt = tab.BucketOffset[b0 + bb + 1] - off;
            if (k < cnt) {
                v = tab.Values[off + k];
            }
        }
        sValues[i] = v;
    }
    for (uint32_t i = tid; i < kBucketTile * (kLutCells / 4); i += 256) {
        const uint32_t bb = i / (kLutCells / 4);
        sLut[i] = bb < nb ? tab.Lut[static_cast<size_t>(b0) * (kLutCells / 4) + i] : 0u;
    }

    // role of this thread while loading: bucket `myB` of rows myRow0, myRow0 + 8, ...; threads of
    // buckets past the end of the model re-read the last bucket and their values are ignored
    const uint32_t myB = tid % kBucketTile;
    const uint32_t myRow0 = tid / kBucketTile;
    const uint32_t mySrcBucket = b0 + min(myB, nb - 1);
    const uint32_t mySrc = tab.BucketSrc[mySrcBucket];
    const uint32_t* myBase = reinterpret_cast<const uint32_t*>(floats);
    uint32_t myStride = stride;
    if (CATS_MATRIX && (tab.BucketFlags[mySrcBucket] & kBucketFlagOneHot) != 0) {
        myBase = reinterpret_cast<const uint32_t*>(cats);
        myStride = catStride;
    }
    uint32_t* myTileSlot = sTile + myB * kTilePitch + myRow0;

    uint32_t regs[kPasses];
#define CBAMD_LOAD_BLOCK(blockIndex)                                                                   \
    do {                                                                                               \
        const uint32_t firstDoc = (blockIndex) * kDocsPerBlock;                                        \
        if (firstDoc + kDocsPerBlock <= docCount) {                                                    \
            const uint32_t* rowPtr = myBase + static_cast<size_t>(firstDoc + myRow0) * myStride + mySrc; \
            _Pragma("unroll") for (int i = 0; i < kPasses; ++i) {                                      \
                regs[i] = rowPtr[static_cast<size_t>(i) * kRowsPerPass * myStride];                    \
            }                                                                                          \
        } else {                                                                                       \
            _Pragma("unroll") for (int i = 0; i < kPasses; ++i) {                                      \
                const uint32_t doc = min(firstDoc + myRow0 + i * kRowsPerPass, docCount - 1);          \
                regs[i] = myBase[static_cast<size_t>(doc) * myStride + mySrc];                         \
            }                                                                                          \
        }                                                                                              \
    } while (0)

    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    // the buckets this wave binarizes in every block (wave, wave + 4, ...) and their grids
    constexpr int kBucketsPerWave = kBucketTile / (256 / kWave);
    uint32_t myFlags[kBucketsPerWave], myTopStep[kBucketsPerWave];
    float myLo[kBucketsPerWave], myScale[kBucketsPerWave];
#pragma unroll
    for (int k = 0; k < kBucketsPerWave; ++k) {
        const uint32_t bucket = b0 + min(wave + k * (256 / kWave), nb - 1);
        const uint4 grid = tab.Grid[bucket];
        myFlags[k] = __builtin_amdgcn_readfirstlane(tab.BucketFlags[bucket]);
        myLo[k] = __uint_as_float(__builtin_amdgcn_readfirstlane(grid.x));
        myScale[k] = __uint_as_float(__builtin_amdgcn_readfirstlane(grid.y));
        const uint32_t steps = __builtin_amdgcn_readfirstlane(grid.z);
        myTopStep[k] = steps ? 1u << (steps - 1) : 0u;
    }
    if (blockBegin < blockEnd) {
        CBAMD_LOAD_BLOCK(blockBegin);
    }
    for (uint32_t block = blockBegin; block < blockEnd; ++block) {
        __syncthreads();  // the previous block's tile has been consumed (and sValues is complete)
#pragma unroll
        for (int i = 0; i < kPasses; ++i) {
            myTileSlot[i * kRowsPerPass] = regs[i];
        }
        __syncthreads();
        if (block + 1 < blockEnd) {
            CBAMD_LOAD_BLOCK(block + 1);  // in flight while this block is binarized
        }
        // this lane's dword of the block's first bucket of the tile; bucket bb sits bb * 256 bytes further
        uint32_t* blockBins = bins + (static_cast<size_t>(block) * tab.BucketPitch + b0) * kWave + lane;
#pragma unroll
        for (int k = 0; k < kBucketsPerWave; ++k) {
            const uint32_t bb = wave + k * (256 / kWave);
            if (bb >= nb) {
                break;
            }
            const uint32_t* values = sValues + bb * kSlots;
            const uint32_t* column = sTile + bb * kTilePitch + lane;
            uint32_t packed = 0;
            if (myFlags[k] & kBucketFlagOneHot) {
                const uint32_t count = tab.BucketOffset[b0 + bb + 1] - tab.BucketOffset[b0 + bb];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    packed |= OneHotBin(values, count, column[j * kWave]) << (8 * j);
                }
            } else {
                // the lane's four documents go through the search side by side: one pass of the loop
                // control and one LDS round trip per step for all four (CountBelowInCell, four at once)
                const uint8_t* lut = reinterpret_cast<const uint8_t*>(sLut + bb * (kLutCells / 4));
                float v[4];
                uint32_t below[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[j] = __uint_as_float(column[j * kWave]);
                }
                if (myFlags[k] & kBucketFlagNanToInf) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        v[j] = isnan(v[j]) ? __uint_as_float(0x7f800000u) : v[j];
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    below[j] = static_cast<uint32_t>(lut[GridCell(v[j], myLo[k], myScale[k])]) * 4;  // byte offsets
                }
                const uint8_t* valueBytes = reinterpret_cast<const uint8_t*>(values);
                for (uint32_t step4 = __builtin_amdgcn_readfirstlane(myTopStep[k]) * 4; step4 >= 4; step4 >>= 1) {
                    const uint8_t* probe = valueBytes + step4 - 4;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float b = *reinterpret_cast<const float*>(probe + below[j]);
                        below[j] += (b < v[j]) ? step4 : 0u;
                    }
                }
                packed = (below[0] >> 2) | (below[1] << 6) | (below[2] << 14) | (below[3] << 22);
            }
            blockBins[bb * kWave] = packed;
        }
    }
#undef CBAMD_LOAD_BLOCK
}

// Column-major input: floats[column * stride + doc] (categorical hashes bit-cast in their column). The work of a
// workgroup is that of BinarizeRowsKernel - kBucketTile buckets, their borders and search tables in LDS,
// `blocksPerGroup` consecutive 256-document blocks, every wave a bucket at a time for the block's 256 documents,
// a lane its four documents side by side - without the tile: a lane's values are neighbours of the other lanes' in
// the column, so they are loaded straight into registers, all buckets of the wave's turn before the first search.
// grid = ceil(doc blocks / blocksPerGroup) * ceil(buckets / kBucketTile), block = 256 threads,
// dynamic LDS = (kBucketTile << LOG2P) * 4 + kBucketTile * kLutCells bytes.
template <int LOG2P>
__global__ __launch_bounds__(256) void BinarizeColumnsKernel(const float* __restrict__ floats, size_t stride,
                                                             uint32_t docCount, TBinarizeTables tab,
                                                             uint32_t blocksPerGroup, uint32_t* __restrict__ bins) {
    constexpr uint32_t kSlots = 1u << LOG2P;
    extern __shared__ uint32_t sBinarize[];
    uint32_t* sValues = sBinarize;                      // [kBucketTile][kSlots]
    uint32_t* sLut = sBinarize + kBucketTile * kSlots;  // [kBucketTile][kLutCells / 4]
    const uint32_t tid = threadIdx.x;
    const uint32_t tileCount = (tab.BucketCount + kBucketTile - 1) / kBucketTile;
    const uint32_t b0 = (blockIdx.x % tileCount) * kBucketTile;
    const uint32_t nb = min(static_cast<uint32_t>(kBucketTile), tab.BucketCount - b0);
    const uint32_t blockCount = (docCount + kDocsPerBlock - 1) / kDocsPerBlock;
    const uint32_t blockBegin = (blockIdx.x / tileCount) * blocksPerGroup;
    const uint32_t blockEnd = min(blockBegin + blocksPerGroup, blockCount);
    for (uint32_t i = tid; i < kBucketTile * kSlots; i += 256) {
        const uint32_t bb = i >> LOG2P, k = i & (kSlots - 1);
        uint32_t v = 0x7f800000u;  // +inf
        if (bb < nb) {
            const uint32_t off = tab.BucketOffset[b0 + bb];
            const uint32_t cnt = tab.BucketOffset[b0 + bb + 1] - off;
            if (k < cnt) {
                v = tab.Values[off + k];
            }
        }
        sValues[i] = v;
    }
    for (uint32_t i = tid; i < kBucketTile * (kLutCells / 4); i += 256) {
        const uint32_t bb = i / (kLutCells / 4);
        sLut[i] = bb < nb ? tab.Lut[static_cast<size_t>(b0) * (kLutCells / 4) + i] : 0u;
    }
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    constexpr int kBucketsPerWave = kBucketTile / (256 / kWave);
    uint32_t myFlags[kBucketsPerWave], myTopStep[kBucketsPerWave], myCount[kBucketsPerWave];
    float myLo[kBucketsPerWave], myScale[kBucketsPerWave];
    const uint32_t* myColumn[kBucketsPerWave];
#pragma unroll
    for (int k = 0; k < kBucketsPerWave; ++k) {
        const uint32_t bucket = b0 + min(wave + k * (256 / kWave), nb - 1);
        const uint4 grid = tab.Grid[bucket];
        myFlags[k] = __builtin_amdgcn_readfirstlane(tab.BucketFlags[bucket]);
        myLo[k] = __uint_as_float(__builtin_amdgcn_readfirstlane(grid.x));
        myScale[k] = __uint_as_float(__builtin_amdgcn_readfirstlane(grid.y));
        const uint32_t steps = __builtin_amdgcn_readfirstlane(grid.z);
        myTopStep[k] = steps ? 1u << (steps - 1) : 0u;
        myCount[k] = __builtin_amdgcn_readfirstlane(tab.BucketOffset[bucket + 1] - tab.BucketOffset[bucket]);
        myColumn[k] = reinterpret_cast<const uint32_t*>(floats) +
                      static_cast<size_t>(__builtin_amdgcn_readfirstlane(tab.BucketSrc[bucket])) * stride;
    }
    __syncthreads();  // the tables are in LDS
    for (uint32_t block = blockBegin; block < blockEnd; ++block) {
        // documents past the last one are read as the last one (their bins are never used)
        uint32_t doc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            doc[j] = min(block * kDocsPerBlock + j * kWave + lane, docCount - 1);
        }
        uint32_t raw[kBucketsPerWave][4];
#pragma unroll
        for (int k = 0; k < kBucketsPerWave; ++k) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                raw[k][j] = myColumn[k][doc[j]];
            }
        }
        uint32_t* blockBins = bins + (static_cast<size_t>(block) * tab.BucketPitch + b0) * kWave + lane;
#pragma unroll
        for (int k = 0; k < kBucketsPerWave; ++k) {
            const uint32_t bb = wave + k * (256 / kWave);
            if (bb >= nb) {
                break;
            }
            const uint32_t* values = sValues + bb * kSlots;
            uint32_t packed = 0;
            if (myFlags[k] & kBucketFlagOneHot) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    packed |= OneHotBin(values, myCount[k], raw[k][j]) << (8 * j);
                }
            } else {
                const uint8_t* lut = reinterpret_cast<const uint8_t*>(sLut + bb * (kLutCells / 4));
                float v[4];
                uint32_t below[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[j] = __uint_as_float(raw[k][j]);
                }
                if (myFlags[k] & kBucketFlagNanToInf) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        v[j] = isnan(v[j]) ? __uint_as_float(0x7f800000u) : v[j];
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    below[j] = static_cast<uint32_t>(lut[GridCell(v[j], myLo[k], myScale[k])]) * 4;  // byte offsets
                }
                const uint8_t* valueBytes = reinterpret_cast<const uint8_t*>(values);
                for (uint32_t step4 = __builtin_amdgcn_readfirstlane(myTopStep[k]) * 4; step4 >= 4; step4 >>= 1) {
                    const uint8_t* probe = valueBytes + step4 - 4;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float b = *reinterpret_cast<const float*>(probe + below[j]);
                        below[j] += (b < v[j]) ? step4 : 0u;
                    }
                }
                packed = (below[0] >> 2) | (below[1] << 6) | (below[2] << 14) | (below[3] << 22);
            }
            blockBins[bb * kWave] = packed;
        }
    }
}

// ---- CTR (target statistics) features -------------------------------------------------------
// What TStaticCtrProvider::CalcCtrs (catboost/libs/model/static_ctr_provider.cpp:14-131) and the
// binarization of its results (cpu/quantization.h:304-325) do per block, done per document here.

struct TCtrFeatureDev {
    uint32_t ItemBegin, ItemEnd;  // the projection: entries of TCtrTablesDev::Items
    uint32_t HashBuckets;         // first 12-byte bucket of the CTR's table in IndexBuckets
    uint32_t HashMask;            // buckets of the table - 1
    uint32_t BlobOffset;          // first dword of the table's rows in Blob
    uint32_t Type;                // ECtrType
    int32_t TargetBorderIdx;
    int32_t TargetClassesCount;
    int32_t CounterDenominator;
    float PriorNum, PriorDenom, Shift, Scale;
    uint32_t FirstBucket, BucketCount;  // where the binarized CTR goes
    uint32_t SameProjectionAsPrevious;  // the feature before this one hashes the same items
};

constexpr uint32_t kCtrItemCat = 0;       // hashed categorical value of column SrcFlat / SrcSplit
constexpr uint32_t kCtrItemBinGe = 1;     // float split: bin of bucket SrcFlat >= Value
constexpr uint32_t kCtrItemBinEq = 2;     // one-hot split: bin of bucket SrcFlat == Value

struct TCtrItemDev {
    uint32_t Kind, SrcFlat, SrcSplit, Value;  // a categorical item keeps its row of the staged tile in Value
};

struct TCtrTablesDev {
    const TCtrFeatureDev* Features;
    const TCtrItemDev* Items;
    const uint32_t* IndexBuckets;  // {hash low, hash high, row} per bucket (helpers/dense_hash_view.h:12-26)
    const uint32_t* Blob;
    // the categorical columns the projections read, as flat and as categorical feature indexes
    const uint32_t* CatColumnsFlat;
    const uint32_t* CatColumnsSplit;
    uint32_t CatColumnCount;
    uint32_t FeatureCount;
};

// hashed categorical values of a batch: Base[doc * DocStride + column * ColumnStride]
struct TCatSource {
    const uint32_t* Base;
    size_t DocStride, ColumnStride;
    uint32_t SplitColumns;  // columns are categorical feature indexes (not flat feature indexes)
};

__device__ __forceinline__ uint64_t CtrCalcHash(uint64_t a, uint64_t b) {  // catboost/libs/model/hash.h:11-14
    constexpr uint64_t kMagicMult = 0x4906ba494954cb65ull;
    return kMagicMult * (a + kMagicMult * b);
}

// TModelCtr::Calc, online_ctr.h:290-293: two roundings each for the quotient and the affine map
__device__ __forceinline__ float CtrCalc(const TCtrFeatureDev& f, float countInClass, float totalCount) {
    const float ctr = __fdiv_rn(__fadd_rn(countInClass, f.PriorNum), __fadd_rn(totalCount, f.PriorDenom));
    return __fmul_rn(__fadd_rn(ctr, f.Shift), f.Scale);
}

constexpr uint32_t kCtrNotFound = 0xffffffffu;

// TDenseIndexHashView::GetIndex, helpers/dense_hash_view.h:46-56; the probe sequence ends at the first
// empty bucket, and after one pass over the table at the latest
__device__ __forceinline__ uint32_t CtrTableRow(const TCtrTablesDev& ctr, const TCtrFeatureDev& f, uint64_t hash) {
    const uint32_t lo = static_cast<uint32_t>(hash), hi = static_cast<uint32_t>(hash >> 32);
    uint32_t zz = lo & f.HashMask;
    for (uint32_t probes = 0; probes <= f.HashMask; ++probes) {
        const uint32_t* bucket = ctr.IndexBuckets + 3 * (static_cast<size_t>(f.HashBuckets) + zz);
        const uint32_t blo = bucket[0], bhi = bucket[1];
        if ((blo & bhi) == 0xffffffffu) {
            return kCtrNotFound;
        }
        if (blo == lo && bhi == hi) {
            return bucket[2];
        }
        zz = (zz + 1) & f.HashMask;
    }
    return kCtrNotFound;
}

// static_ctr_provider.cpp:52-126, one branch per CTR type
__device__ __forceinline__ float CtrValue(const TCtrTablesDev& ctr, const TCtrFeatureDev& f, uint32_t row) {
    const uint32_t* blob = ctr.Blob + f.BlobOffset;
    if (f.Type == 2 || f.Type == 3) {  // mean of the target: {float Sum; int Count}
        if (row == kCtrNotFound) {
            return CtrCalc(f, 0.f, 0.f);
        }
        return CtrCalc(f, __uint_as_float(blob[2 * static_cast<size_t>(row)]),
                       static_cast<float>(static_cast<int32_t>(blob[2 * static_cast<size_t>(row) + 1])));
    }
    if (f.Type == 4 || f.Type == 5) {  // Counter, FeatureFreq
        const float denominator = static_cast<float>(f.CounterDenominator);
        if (row == kCtrNotFound) {
            return CtrCalc(f, 0.f, denominator);
        }
        return CtrCalc(f, static_cast<float>(static_cast<int32_t>(blob[row])), denominator);
    }
    const int32_t classes = f.TargetClassesCount;
    if (f.Type == 1) {  // Buckets
        if (row == kCtrNotFound) {
            return CtrCalc(f, 0.f, 0.f);
        }
        const uint32_t* history = blob + static_cast<size_t>(row) * classes;
        int32_t total = 0;
        for (int32_t c = 0; c < classes; ++c) {
            total += static_cast<int32_t>(history[c]);
        }
        return CtrCalc(f, static_cast<float>(static_cast<int32_t>(history[f.TargetBorderIdx])), static_cast<float>(total));
    }
    // Borders
    if (classes > 2) {
        int32_t good = 0, total = 0;
        if (row != kCtrNotFound) {
            const uint32_t* history = blob + static_cast<size_t>(row) * classes;
            for (int32_t c = 0; c < f.TargetBorderIdx + 1; ++c) {
                total += static_cast<int32_t>(history[c]);
            }
            for (int32_t c = f.TargetBorderIdx + 1; c < classes; ++c) {
                good += static_cast<int32_t>(history[c]);
            }
            total += good;
        }
        return CtrCalc(f, static_cast<float>(good), static_cast<float>(total));
    }
    if (row == kCtrNotFound) {
        return CtrCalc(f, 0.f, 0.f);
    }
    const int32_t n0 = static_cast<int32_t>(blob[2 * static_cast<size_t>(row)]);
    const int32_t n1 = static_cast<int32_t>(blob[2 * static_cast<size_t>(row) + 1]);
    return CtrCalc(f, static_cast<float>(n1), static_cast<float>(n0 + n1));
}

// Tables whose row is one or two dwords (all but the class histograms of more than two classes): the dwords of
// a row, read once for all the features of the table, and the value of a feature from them (as CtrValue).
__device__ __forceinline__ bool CtrRowIsShort(const TCtrFeatureDev& f) {
    return (f.Type >= 2 && f.Type <= 5) || (f.Type != 1 && f.TargetClassesCount <= 2);
}

__device__ __forceinline__ uint2 CtrShortRow(const TCtrTablesDev& ctr, const TCtrFeatureDev& f, uint32_t row) {
    const uint32_t* blob = ctr.Blob + f.BlobOffset;
    if (row == kCtrNotFound) {
        return make_uint2(0u, 0u);
    }
    if (f.Type == 4 || f.Type == 5) {
        return make_uint2(blob[row], 0u);
    }
    return make_uint2(blob[2 * static_cast<size_t>(row)], blob[2 * static_cast<size_t>(row) + 1]);
}

__device__ __forceinline__ float CtrValueOfShortRow(const TCtrFeatureDev& f, uint32_t row, uint2 dwords) {
    if (f.Type == 2 || f.Type == 3) {
        if (row == kCtrNotFound) {
            return CtrCalc(f, 0.f, 0.f);
        }
        return CtrCalc(f, __uint_as_float(dwords.x), static_cast<float>(static_cast<int32_t>(dwords.y)));
    }
    if (f.Type == 4 || f.Type == 5) {
        const float denominator = static_cast<float>(f.CounterDenominator);
        if (row == kCtrNotFound) {
            return CtrCalc(f, 0.f, denominator);
        }
        return CtrCalc(f, static_cast<float>(static_cast<int32_t>(dwords.x)), denominator);
    }
    if (row == kCtrNotFound) {
        return CtrCalc(f, 0.f, 0.f);
    }
    const int32_t n0 = static_cast<int32_t>(dwords.x), n1 = static_cast<int32_t>(dwords.y);
    return CtrCalc(f, static_cast<float>(n1), static_cast<float>(n0 + n1));
}

// grid = (document blocks, CTR features), one wave per workgroup: lane l computes the CTR of documents
// l, l + 64, l + 128, l + 192 of the block from the block's float / one-hot bins (already written)
// and the hashed categorical values, and writes the bins of the CTR's buckets.
__global__ __launch_bounds__(64) void CtrBinarizeKernel(TCatSource cats, uint32_t docCount, TCtrTablesDev ctr,
                                                        TBinarizeTables tab, uint32_t* __restrict__ bins) {
    const uint32_t block = blockIdx.x, lane = threadIdx.x;
    const TCtrFeatureDev f = ctr.Features[blockIdx.y];
    uint64_t hash[4] = {0, 0, 0, 0};
    for (uint32_t i = f.ItemBegin; i < f.ItemEnd; ++i) {
        const TCtrItemDev item = ctr.Items[i];
        if (item.Kind == kCtrItemCat) {
            const size_t column = cats.SplitColumns ? item.SrcSplit : item.SrcFlat;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const size_t doc = min(block * kDocsPerBlock + j * kWave + lane, docCount - 1);
                const int32_t v = static_cast<int32_t>(cats.Base[doc * cats.DocStride + column * cats.ColumnStride]);
                hash[j] = CtrCalcHash(hash[j], static_cast<uint64_t>(static_cast<int64_t>(v)));
            }
        } else {
            const uint32_t word = bins[(static_cast<size_t>(block) * tab.BucketPitch + item.SrcFlat) * kWave + lane];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t bin = (word >> (8 * j)) & 0xffu;
                const bool holds = item.Kind == kCtrItemBinGe ? bin >= item.Value : bin == item.Value;
                hash[j] = CtrCalcHash(hash[j], holds ? 1u : 0u);
            }
        }
    }
    float value[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        value[j] = CtrValue(ctr, f, CtrTableRow(ctr, f, hash[j]));
    }
    for (uint32_t k = 0; k < f.BucketCount; ++k) {
        const uint32_t bucket = f.FirstBucket + k;
        const uint32_t begin = tab.BucketOffset[bucket], end = tab.BucketOffset[bucket + 1];
        uint32_t count[4] = {0, 0, 0, 0};
        for (uint32_t b = begin; b < end; ++b) {
            const float border = __uint_as_float(tab.Values[b]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                count[j] += value[j] > border ? 1u : 0u;
            }
        }
        bins[(static_cast<size_t>(block) * tab.BucketPitch + bucket) * kWave + lane] =
            count[0] | (count[1] << 8) | (count[2] << 16) | (count[3] << 24);
    }
}

// The same for models whose CTR projections read at most kCtrMaxTileColumns categorical columns:
// grid = (document blocks, groups of kCtrGroup CTR features), 4 waves per workgroup. The block's hashed
// categorical values are staged once per workgroup into LDS ([column][document], read without bank
// conflicts), each wave then works through kCtrGroup / 4 consecutive CTR features and keeps the hash
// when the next feature has the same projection (features are sorted by projection).
constexpr uint32_t kCtrGroup = 16;
constexpr uint32_t kCtrMaxTileColumns = 60;
constexpr uint32_t kCtrTilePitch = kDocsPerBlock + 1;

__global__ __launch_bounds__(256) void CtrBinarizeTileKernel(TCatSource cats, uint32_t docCount, TCtrTablesDev ctr,
                                                             TBinarizeTables tab, uint32_t* __restrict__ bins) {
    extern __shared__ uint32_t sCats[];  // [CatColumnCount][kCtrTilePitch]
    const uint32_t block = blockIdx.x, tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t columns = ctr.CatColumnCount;
    const uint32_t* columnList = cats.SplitColumns ? ctr.CatColumnsSplit : ctr.CatColumnsFlat;
    const size_t firstDoc = static_cast<size_t>(block) * kDocsPerBlock;
    for (uint32_t i = tid; i < columns * kDocsPerBlock; i += 256) {
        // neighbouring threads read neighbouring addresses: columns of one row, or documents of one column
        const uint32_t c = cats.ColumnStride == 1 ? i % columns : i / kDocsPerBlock;
        const uint32_t d = cats.ColumnStride == 1 ? i / columns : i % kDocsPerBlock;
        const size_t doc = min(firstDoc + d, static_cast<size_t>(docCount) - 1);
        sCats[c * kCtrTilePitch + d] = cats.Base[doc * cats.DocStride + static_cast<size_t>(columnList[c]) * cats.ColumnStride];
    }
    __syncthreads();
    constexpr uint32_t kPerWave = kCtrGroup / 4;
    const uint32_t first = blockIdx.y * kCtrGroup + wave * kPerWave;
    uint64_t hash[4] = {0, 0, 0, 0};
    uint32_t row[4] = {kCtrNotFound, kCtrNotFound, kCtrNotFound, kCtrNotFound};
    uint2 rowDwords[4] = {};
    uint32_t tableOfRows = 0;  // HashBuckets of the table that row[] was looked up in
    for (uint32_t k = 0; k < kPerWave && first + k < ctr.FeatureCount; ++k) {
        const TCtrFeatureDev f = ctr.Features[first + k];
        if (k == 0 || !f.SameProjectionAsPrevious) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                hash[j] = 0;
            }
            for (uint32_t i = f.ItemBegin; i < f.ItemEnd; ++i) {
                const TCtrItemDev item = ctr.Items[i];
                if (item.Kind == kCtrItemCat) {
                    const uint32_t* column = sCats + item.Value * kCtrTilePitch + lane;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int32_t v = static_cast<int32_t>(column[j * kWave]);
                        hash[j] = CtrCalcHash(hash[j], static_cast<uint64_t>(static_cast<int64_t>(v)));
                    }
                } else {
                    const uint32_t word = bins[(static_cast<size_t>(block) * tab.BucketPitch + item.SrcFlat) * kWave + lane];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t bin = (word >> (8 * j)) & 0xffu;
                        const bool holds = item.Kind == kCtrItemBinGe ? bin >= item.Value : bin == item.Value;
                        hash[j] = CtrCalcHash(hash[j], holds ? 1u : 0u);
                    }
                }
            }
        }
        // features that differ only in prior, target border, shift or scale read the same row of the same table
        const bool shortRow = CtrRowIsShort(f);
        if (k == 0 || !f.SameProjectionAsPrevious || f.HashBuckets != tableOfRows) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                row[j] = CtrTableRow(ctr, f, hash[j]);
            }
            if (shortRow) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    rowDwords[j] = CtrShortRow(ctr, f, row[j]);
                }
            }
            tableOfRows = f.HashBuckets;
        }
        float value[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            value[j] = shortRow ? CtrValueOfShortRow(f, row[j], rowDwords[j]) : CtrValue(ctr, f, row[j]);
        }
        for (uint32_t b = 0; b < f.BucketCount; ++b) {
            const uint32_t bucket = f.FirstBucket + b;
            const uint32_t begin = tab.BucketOffset[bucket], end = tab.BucketOffset[bucket + 1];
            uint32_t count[4] = {0, 0, 0, 0};
            for (uint32_t x = begin; x < end; ++x) {
                const float border = __uint_as_float(tab.Values[x]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    count[j] += value[j] > border ? 1u : 0u;
                }
            }
            bins[(static_cast<size_t>(block) * tab.BucketPitch + bucket) * kWave + lane] =
                count[0] | (count[1] << 8) | (count[2] << 16) | (count[3] << 24);
        }
    }
}

// Final value of one output cell: Scale * sum (+ Bias[k] when the range starts at tree 0),
// as ApplyScaleAndBias (catboost/libs/model/scale_and_bias.cpp:4-50). No fused multiply-add.
__device__ __forceinline__ double Finish(double sum, double scale, double bias, bool addBias) {
    double r = __dmul_rn(scale, sum);
    if (addBias) {
        r = __dadd_rn(r, bias);
    }
    return r;
}

// Oblivious trees, any model: one wave per 256-document block, four documents per lane, leaf
// sums kept in registers in fp64 and accumulated in tree order (as the CPU evaluator does).
// DCHUNK output dimensions are accumulated per pass over the trees.
// mode: kEvalContinue - the sums start from the raw sums of earlier trees found in `out`; kEvalRaw - store raw
// sums (neither scaled nor biased) for a launch that continues them; `addBias` tells the launch that finishes
// whether the whole range started at tree 0 (0 no, 1 yes, 2: this launch is the whole range, treeBegin tells).
// grid = ceil(doc blocks / 4), block = 256 threads.
constexpr uint32_t kEvalContinue = 1;
constexpr uint32_t kEvalRaw = 2;

template <int DCHUNK>
__global__ __launch_bounds__(256) void EvalObliviousKernel(const uint32_t* __restrict__ bins, size_t docCount,
                                                           uint32_t bucketCount, TTreeTables tt, uint32_t treeBegin,
                                                           uint32_t treeEnd, double* out, uint32_t mode,
                                                           uint32_t addBiasFlag) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const size_t block = static_cast<size_t>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
    const size_t blockCount = (docCount + kDocsPerBlock - 1) / kDocsPerBlock;
    if (block >= blockCount) {
        return;
    }
    const uint32_t* myBins = bins + block * bucketCount * kWave + lane;
    const int dim = tt.Dim;
    const bool addBias = addBiasFlag == 2 ? treeBegin == 0 : addBiasFlag != 0;
    for (int d0 = 0; d0 < dim; d0 += DCHUNK) {
        double acc[4][DCHUNK];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const size_t doc = block * kDocsPerBlock + j * kWave + lane;
#pragma unroll
            for (int k = 0; k < DCHUNK; ++k) {
                acc[j][k] = 0.0;
                if ((mode & kEvalContinue) && doc < docCount && (DCHUNK == 1 || d0 + k < dim)) {
                    acc[j][k] = out[doc * dim + d0 + k];
                }
            }
        }
        for (uint32_t t = treeBegin; t < treeEnd; ++t) {
            const uint32_t first = tt.TreeStart[t];
            const uint32_t depth = tt.TreeSize[t];
            uint32_t idx0 = 0, idx1 = 0, idx2 = 0, idx3 = 0;
            for (uint32_t d = 0; d < depth; ++d) {
                const uint32_t sp = tt.Splits[first + d];
                const uint32_t w = myBins[(sp & 0xffffu) * kWave];
                const uint32_t x = (sp >> 16) & 0xffu;
                const uint32_t s = sp >> 24;
                idx0 |= static_cast<uint32_t>(((w & 0xffu) ^ x) >= s) << d;
                idx1 |= static_cast<uint32_t>((((w >> 8) & 0xffu) ^ x) >= s) << d;
                idx2 |= static_cast<uint32_t>((((w >> 16) & 0xffu) ^ x) >= s) << d;
                idx3 |= static_cast<uint32_t>(((w >> 24) ^ x) >= s) << d;
            }
            const double* leaf = tt.Leaves + tt.FirstLeaf[t] + d0;
            const uint32_t idx[4] = {idx0, idx1, idx2, idx3};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const double* p = leaf + static_cast<size_t>(idx[j]) * dim;
#pragma unroll
                for (int k = 0; k < DCHUNK; ++k) {
                    if (DCHUNK == 1 || d0 + k < dim) {
                        acc[j][k] = __dadd_rn(acc[j][k], p[k]);
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const size_t doc = block * kDocsPerBlock + j * kWave + lane;
            if (doc < docCount) {
#pragma unroll
                for (int k = 0; k < DCHUNK; ++k) {
                    if (DCHUNK == 1 || d0 + k < dim) {
                        out[doc * dim + d0 + k] =
                            (mode & kEvalRaw) ? acc[j][k] : Finish(acc[j][k], tt.Scale, tt.Bias[d0 + k], addBias);
                    }
                }
            }
        }
    }
}

// Small batches on the register-resident kernels: every slice of the trees left its raw sums in
// partials[slice][count]; adds them in slice order and finishes like ApplyScaleAndBias. One thread per value.
__global__ __launch_bounds__(256) void CombineSlicesKernel(const double* __restrict__ partials, uint32_t slices,
                                                           size_t count, double scale, const double* __restrict__ bias,
                                                           int dim, double* __restrict__ out) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= count) {
        return;
    }
    double sum = partials[i];
    for (uint32_t s = 1; s < slices; ++s) {
        sum = __dadd_rn(sum, partials[s * count + i]);
    }
    out[i] = Finish(sum, scale, bias[i % static_cast<size_t>(dim)], true);
}

// Packed tree table of the tile kernel: 16 dwords per tree. Slots 0..7 hold the tree's levels
// (slot d = split d, unused levels padded with a split that is false for every bin), slot 8 the
// index of the tree's first leaf value. A level is
//   7-bit form: bucket << 8 | (128 - splitIdx)          (all bins and split indexes <= 127, no xor)
//   8-bit form: bucket << 16 | xorMask << 8 | splitIdx
constexpr int kPackedTreeDwords = 16;
constexpr int kPackedFirstLeafSlot = 8;

// Bit 7 of every byte of the result tells whether (bin ^ xorMask) >= splitIdx for the four
// documents packed in `a`. 7-bit form: adding (128 - splitIdx) to every byte carries into bit 7
// exactly when bin >= splitIdx. 8-bit form: the unsigned compare is the carry out of
// x + ~splitIdx + 1 taken per byte, x = bin ^ xorMask:
//   carry = (x & ns) | ((x | ns) & low), ns = ~splitIdx, low = (x & 0x7f) + (ns & 0x7f) + 1.
template <bool SEVEN_BIT>
__device__ __forceinline__ uint32_t CompareBytes(uint32_t a, uint32_t level) {
    if (SEVEN_BIT) {
        return a + (level & 0xffu) * 0x01010101u;
    }
    const uint32_t s = level & 0xffu;
    const uint32_t x = a ^ (((level >> 8) & 0xffu) * 0x01010101u);
    const uint32_t ns = (~s) & 0xffu;
    const uint32_t low = (x & 0x7f7f7f7fu) + ((ns & 0x7fu) + 1u) * 0x01010101u;
    const uint32_t nsr = ns * 0x01010101u;
    return (x & nsr) | ((x | nsr) & low);
}

// byte offset of a level's bucket inside the LDS tile (256 bytes per bucket)
template <bool SEVEN_BIT>
__device__ __forceinline__ uint32_t LevelTileOffset(uint32_t level) {
    return SEVEN_BIT ? (level & 0xffffff00u) : ((level >> 16) << 8);
}

// Leaf indexes of one tree for the four documents of a lane, one byte each: MAXD levels, every
// one an LDS dword read, a byte-parallel compare and a shift-in of the four result bits (the
// first split ends up in bit 0).
template <bool SEVEN_BIT, int MAXD>
__device__ __forceinline__ uint32_t TreeIndexes(const uint8_t* laneTile, uint32_t packedRow) {
    uint32_t idx4 = 0;
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        const uint32_t level = __builtin_amdgcn_readlane(packedRow, d);
        const uint32_t a = *reinterpret_cast<const uint32_t*>(laneTile + LevelTileOffset<SEVEN_BIT>(level));
        const uint32_t r = CompareBytes<SEVEN_BIT>(a, level);
        idx4 = (r & 0x80808080u) | ((idx4 >> 1) & 0x7f7f7f7fu);
    }
    return idx4 >> (8 - MAXD);
}

// Oblivious trees of depth <= MAXD <= 8 whose bins fit an LDS tile: one workgroup of kTileWaves
// waves per 256-document block. The block's bins (buckets x 256 bytes) are copied to LDS once;
// the waves share the tile and split the trees among themselves (tree t goes to wave
// t % kTileWaves), four documents per lane. A wave fetches a tree's packed row with one 64-byte
// load (two trees ahead) and broadcasts the levels from it. Per-wave partial sums (fp64) are added
// in wave order through an LDS accumulator behind the tile, and the last wave writes the results.
//
// Leaf values. DCHUNK == 1 (one-dimensional models): `leaves` is the model's array and slot 8 of a
// packed row the tree's first value. DCHUNK > 1: `leaves` is a copy padded to DCHUNK values per
// leaf, one run of (leaf count) x DCHUNK values per tree and chunk of DCHUNK dimensions (zeros
// behind the last dimension); slot 9 is the tree's first padded value and slot 10 its leaf count.
// A lane adds all DCHUNK values of a leaf without looking at the dimension; only the final store
// does. LEAF_LDS: every wave copies the (1 << MAXD) * DCHUNK values of its current tree and chunk
// into a private LDS region with row-contiguous 16-byte loads, one tree ahead through registers
// when that takes at most 8 loads per lane, and gathers from there; otherwise the values are
// gathered straight from global memory. `leaves` must be readable for (1 << MAXD) * DCHUNK values
// past the first value of the last tree.
// WAVES waves share a block (tree t goes to wave t % WAVES): kTileWaves, or kWideTileWaves when the
// tile is so large that only one workgroup fits a CU: the waves of a workgroup wait on LDS round trips
// most of the time, and sixteen of them hide what eight cannot (400 buckets: 1.75 instead of 2.79 ms).
// grid = doc blocks, block = 64 * WAVES threads, dynamic LDS = buckets * 256 (rounded up to
// 8) + 256 * DCHUNK * 8 [+ WAVES * (1 << MAXD) * DCHUNK * 8 with LEAF_LDS] bytes.
constexpr int kTileWaves = 8;
constexpr int kWideTileWaves = 16;
constexpr int kPackedPaddedLeafSlot = 9;
constexpr int kPackedLeafCountSlot = 10;

template <bool SEVEN_BIT, int MAXD, int DCHUNK, bool LEAF_LDS, int WAVES>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(2, 4))) void EvalObliviousTileKernel(
    const uint32_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ packedTrees,
    const double* __restrict__ leaves, const double* __restrict__ bias, double scale, int dim, uint32_t treeBegin,
    uint32_t treeEnd, double* __restrict__ out) {
    static_assert(DCHUNK == 1 || DCHUNK % 2 == 0, "padded leaf rows are copied in 16-byte pairs");
    constexpr uint32_t kTreeDoubles = (1u << MAXD) * DCHUNK;    // values of one tree and chunk in LDS
    constexpr uint32_t kTreePairs = kTreeDoubles / 2;
    constexpr int kPairsPerLane = static_cast<int>((kTreePairs + kWave - 1) / kWave);
    constexpr bool kPrefetch = kPairsPerLane <= 8;  // registers of the copy that runs one tree ahead
    constexpr int kPrefetchRegs = kPrefetch ? kPairsPerLane : 1;
    constexpr int kFirstSlot = DCHUNK == 1 ? kPackedFirstLeafSlot : kPackedPaddedLeafSlot;
    extern __shared__ uint32_t sTile[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x;
    const uint32_t tileDwords = bucketCount * kWave;
    const uint32_t* src = bins + block * tileDwords;
    for (uint32_t i = tid; i < tileDwords; i += 64 * WAVES) {
        sTile[i] = src[i];
    }
    const bool addBias = treeBegin == 0;
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + lane * 4;
    const uint32_t slot = lane & (kPackedTreeDwords - 1);
    double* sRed = reinterpret_cast<double*>(sTile + ((tileDwords + 1) & ~1u));
    double* sLeaf = sRed + kDocsPerBlock * DCHUNK + wave * kTreeDoubles;  // per-wave leaf region
    for (int d0 = 0; d0 < dim; d0 += DCHUNK) {
        __syncthreads();  // tile is loaded / the previous chunk's accumulator has been read
        const uint32_t chunk = static_cast<uint32_t>(d0) / DCHUNK;
        double acc[4][DCHUNK];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int k = 0; k < DCHUNK; ++k) {
                acc[j][k] = 0.0;
            }
        }
        double2 pref[kPrefetchRegs];
#pragma unroll
        for (int i = 0; i < kPrefetchRegs; ++i) {
            pref[i] = {0.0, 0.0};
        }
        // first value of this chunk of the tree whose packed row is `rowValue`
#define CBAMD_TREE_VALUES(rowValue)                                                               \
    (leaves + __builtin_amdgcn_readlane(rowValue, kFirstSlot) +                                   \
     (DCHUNK == 1 ? 0u : chunk * __builtin_amdgcn_readlane(rowValue, kPackedLeafCountSlot) * DCHUNK))
#define CBAMD_FETCH_LEAVES(rowValue)                                                              \
    do {                                                                                          \
        const double2* src2 = reinterpret_cast<const double2*>(CBAMD_TREE_VALUES(rowValue));     \
        _Pragma("unroll") for (int i = 0; i < kPrefetchRegs; ++i) {                               \
            if (static_cast<uint32_t>(i + 1) * kWave <= kTreePairs || i * kWave + lane < kTreePairs) { \
                pref[i] = src2[i * kWave + lane];                                                 \
            }                                                                                     \
        }                                                                                         \
    } while (0)
        // packed rows are fetched two trees ahead so that the next tree's row has arrived by the
        // time its leaf values are requested
#define CBAMD_FETCH_ROW(tree) \
    ((tree) < treeEnd ? packedTrees[static_cast<size_t>(tree) * kPackedTreeDwords + slot] : 0u)
        uint32_t t = treeBegin + wave;
        uint32_t row = CBAMD_FETCH_ROW(t);
        uint32_t rowNext = CBAMD_FETCH_ROW(t + WAVES);
        if (LEAF_LDS && kPrefetch && t < treeEnd) {
            CBAMD_FETCH_LEAVES(row);
        }
        while (t < treeEnd) {
            const uint32_t tNext = t + WAVES;
            const uint32_t rowNext2 = CBAMD_FETCH_ROW(tNext + WAVES);
            const double* leaf = CBAMD_TREE_VALUES(row);
            if (LEAF_LDS) {
                // publish this tree's leaf values in the wave's region; the previous tree's gathers
                // were issued before these stores and LDS serves one wave's requests in order
                double2* dst2 = reinterpret_cast<double2*>(sLeaf);
                if (kPrefetch) {
#pragma unroll
                    for (int i = 0; i < kPrefetchRegs; ++i) {
                        if (static_cast<uint32_t>(i + 1) * kWave <= kTreePairs || i * kWave + lane < kTreePairs) {
                            dst2[i * kWave + lane] = pref[i];
                        }
                    }
                    if (tNext < treeEnd) {
                        CBAMD_FETCH_LEAVES(rowNext);
                    }
                } else {
                    const double2* src2 = reinterpret_cast<const double2*>(leaf);
                    for (uint32_t i = lane; i < kTreePairs; i += kWave) {
                        dst2[i] = src2[i];
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                leaf = sLeaf;
            }
            const uint32_t idx4 = TreeIndexes<SEVEN_BIT, MAXD>(laneTile, row);
            if (DCHUNK == 1) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[j][0] = __dadd_rn(acc[j][0], leaf[(idx4 >> (8 * j)) & 0xffu]);
                }
            } else {
                // the DCHUNK values of the next document's leaf are requested before the current
                // document's are added (the scheduling fences keep the two groups apart)
                double val[2][DCHUNK];
#pragma unroll
                for (int k = 0; k < DCHUNK; ++k) {
                    val[0][k] = leaf[(idx4 & 0xffu) * DCHUNK + k];
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (j < 3) {
#pragma unroll
                        for (int k = 0; k < DCHUNK; ++k) {
                            val[(j + 1) & 1][k] = leaf[((idx4 >> (8 * (j + 1))) & 0xffu) * DCHUNK + k];
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int k = 0; k < DCHUNK; ++k) {
                        acc[j][k] = __dadd_rn(acc[j][k], val[j & 1][k]);
                    }
                }
            }
            if (LEAF_LDS) {
                __builtin_amdgcn_wave_barrier();
            }
            t = tNext;
            row = rowNext;
            rowNext = rowNext2;
        }
#undef CBAMD_FETCH_ROW
#undef CBAMD_FETCH_LEAVES
#undef CBAMD_TREE_VALUES
        // waves add their partial sums in wave order into the LDS accumulator; the last wave
        // finishes the values and writes them out
        for (uint32_t w = 0; w + 1 < WAVES; ++w) {
            if (wave == w) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int k = 0; k < DCHUNK; ++k) {
                        double* cell = sRed + (j * kWave + lane) * DCHUNK + k;
                        *cell = (w == 0) ? acc[j][k] : __dadd_rn(*cell, acc[j][k]);
                    }
                }
            }
            __syncthreads();
        }
        if (wave == WAVES - 1) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const size_t doc = block * kDocsPerBlock + j * kWave + lane;
#pragma unroll
                for (int k = 0; k < DCHUNK; ++k) {
                    if (doc < docCount && (DCHUNK == 1 || d0 + k < dim)) {
                        const double sum = __dadd_rn(sRed[(j * kWave + lane) * DCHUNK + k], acc[j][k]);
                        out[doc * dim + d0 + k] = Finish(sum, scale, bias[d0 + k], addBias);
                    }
                }
            }
        }
    }
}

// One-dimensional oblivious models whose bins do not fit the 256-document tile (more than ~600
// buckets): the same scheme on half a block. A workgroup copies the bins of 128 documents
// (buckets x 128 bytes, two documents per lane: documents (2 * half + j) * 64 + lane of the block)
// and its waves split the trees; everything else is EvalObliviousTileKernel with DCHUNK == 1 and
// leaf values through LDS. `leaves` holds (1 << MAXD) values per tree at a fixed pitch.
// The packed rows come in the form chosen per tree (bit 31 of slot kPackedFormSlot): the 7-bit form
// when the tree has no one-hot split and all float bins of the model fit 7 bits, else the 8-bit form;
// a model with a few one-hot splits pays the longer compare only in the trees that have them.
// A 7-bit row holds what a level needs ready for use, so that a level costs two lane reads and no scalar
// arithmetic: slot d the byte offset of the level's bucket in the half tile (bucket * 128), slot 8 + d
// (128 - splitIdx) * 0x0101. An 8-bit row holds bucket << 16 | xorMask << 8 | splitIdx in slot d.
// grid = 2 * doc blocks, block = 64 * kTileWaves threads, dynamic LDS = buckets * 128 (rounded up
// to 8) + 128 * 8 + kTileWaves * (1 << MAXD) * 8 bytes.
constexpr int kPackedFormSlot = 8;  // mixed table, bit 31: clear = 7-bit form, set = 8-bit form

template <bool SEVEN_BIT, int MAXD>
__device__ __forceinline__ uint32_t TreeIndexesPair(const uint8_t* laneTile, uint32_t packedRow) {
    uint32_t idx2 = 0;
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        uint32_t r;
        if (SEVEN_BIT) {
            const uint32_t a = *reinterpret_cast<const uint16_t*>(laneTile + __builtin_amdgcn_readlane(packedRow, d));
            r = a + __builtin_amdgcn_readlane(packedRow, 8 + d);
        } else {
            const uint32_t level = __builtin_amdgcn_readlane(packedRow, d);
            const uint32_t a = *reinterpret_cast<const uint16_t*>(laneTile + (LevelTileOffset<false>(level) >> 1));
            r = CompareBytes<false>(a, level);
        }
        // bits 7 and 15 from r, the rest from the shifted index: one v_bfi. What a sum carries past bit 15
        // moves down one bit per level and is replaced when it reaches bit 15.
        idx2 = (r & 0x8080u) | ((idx2 >> 1) & ~0x8080u);
    }
    return (idx2 & 0xffffu) >> (8 - MAXD);
}

template <int MAXD>
__global__ __launch_bounds__(64 * kTileWaves) void EvalObliviousHalfTileKernel(
    const uint16_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ packedMixed,
    const double* __restrict__ leaves, const double* __restrict__ bias, double scale, uint32_t treeBegin,
    uint32_t treeEnd, double* __restrict__ out) {
    constexpr uint32_t kTreePairs = (1u << MAXD) / 2;
    constexpr int kPrefetchRegs = static_cast<int>((kTreePairs + kWave - 1) / kWave);
    extern __shared__ uint32_t sTile[];
    uint16_t* sTile16 = reinterpret_cast<uint16_t*>(sTile);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x >> 1;
    const uint32_t half = blockIdx.x & 1;
    const uint32_t tileWords = bucketCount * kWave;
    const uint16_t* src = bins + block * tileWords * 2 + half;
    for (uint32_t i = tid; i < tileWords; i += 64 * kTileWaves) {
        sTile16[i] = src[2 * i];
    }
    const bool addBias = treeBegin == 0;
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + lane * 2;
    const uint32_t slot = lane & (kPackedTreeDwords - 1);
    double* sRed = reinterpret_cast<double*>(sTile + ((tileWords / 2 + 1) & ~1u));
    double* sLeaf = sRed + 2 * kWave + wave * (1u << MAXD);  // per-wave leaf region
    __syncthreads();  // tile is loaded
    double acc[2] = {0.0, 0.0};
    // A wave has only one partner on its SIMD here (the tile leaves room for one workgroup per CU),
    // so what it needs from global memory is requested kAhead of its trees ahead: the packed row
    // and the leaf values ((1 << MAXD) doubles per tree at a fixed pitch) of tree t + kAhead * 8
    // go into the registers that tree t has just given up.
    constexpr int kAhead = 4;
    uint32_t rows[kAhead];
    double2 pref[kAhead][kPrefetchRegs];
#define CBAMD_FETCH_TREE(k, tree)                                                                 \
    do {                                                                                          \
        const uint32_t fetchTree = (tree);                                                        \
        rows[k] = 0u;                                                                             \
        if (fetchTree < treeEnd) {                                                                \
            rows[k] = packedMixed[static_cast<size_t>(fetchTree) * kPackedTreeDwords + slot];     \
            const double2* src2 = reinterpret_cast<const double2*>(leaves) + static_cast<size_t>(fetchTree) * kTreePairs; \
            _Pragma("unroll") for (int i = 0; i < kPrefetchRegs; ++i) {                           \
                if (static_cast<uint32_t>(i + 1) * kWave <= kTreePairs || i * kWave + lane < kTreePairs) { \
                    pref[k][i] = src2[i * kWave + lane];                                          \
                }                                                                                 \
            }                                                                                     \
        }                                                                                         \
    } while (0)
    uint32_t t = treeBegin + wave;
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
#pragma unroll
        for (int i = 0; i < kPrefetchRegs; ++i) {
            pref[k][i] = {0.0, 0.0};
        }
        CBAMD_FETCH_TREE(k, t + k * kTileWaves);
    }
    while (t < treeEnd) {
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            if (t < treeEnd) {
                // publish this tree's leaf values in the wave's region; the previous tree's gathers
                // were issued before these stores and LDS serves one wave's requests in order
                double2* dst2 = reinterpret_cast<double2*>(sLeaf);
#pragma unroll
                for (int i = 0; i < kPrefetchRegs; ++i) {
                    if (static_cast<uint32_t>(i + 1) * kWave <= kTreePairs || i * kWave + lane < kTreePairs) {
                        dst2[i * kWave + lane] = pref[k][i];
                    }
                }
                const uint32_t row = rows[k];
                CBAMD_FETCH_TREE(k, t + kAhead * kTileWaves);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                uint32_t idx2;
                if (__builtin_amdgcn_readlane(row, kPackedFormSlot) >> 31) {
                    idx2 = TreeIndexesPair<false, MAXD>(laneTile, row);
                } else {
                    idx2 = TreeIndexesPair<true, MAXD>(laneTile, row);
                }
                acc[0] = __dadd_rn(acc[0], sLeaf[idx2 & 0xffu]);
                acc[1] = __dadd_rn(acc[1], sLeaf[(idx2 >> 8) & 0xffu]);
                __builtin_amdgcn_wave_barrier();
                t += kTileWaves;
            }
        }
    }
#undef CBAMD_FETCH_TREE
    // waves add their partial sums in wave order into the LDS accumulator; the last wave
    // finishes the values and writes them out
    for (uint32_t w = 0; w + 1 < kTileWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                double* cell = sRed + j * kWave + lane;
                *cell = (w == 0) ? acc[j] : __dadd_rn(*cell, acc[j]);
            }
        }
        __syncthreads();
    }
    if (wave == kTileWaves - 1) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const size_t doc = block * kDocsPerBlock + (2 * half + j) * kWave + lane;
            if (doc < docCount) {
                out[doc] = Finish(__dadd_rn(sRed[j * kWave + lane], acc[j]), scale, bias[0], addBias);
            }
        }
    }
}

// The same half tile with two trees in flight per wave: lanes 0..31 evaluate one tree and lanes 32..63 the
// next one, each lane for four documents of the tile (one LDS dword: the bins of documents
// (2 * half + j) * 64 + 2 * m + i, byte 2 * i + j, for lane m of either group), so a level costs one LDS read
// and one byte-parallel compare for 2 x 128 (tree, document) pairs instead of 128. Needs every bin of the
// tile below 128 (the 7-bit compare; a one-hot level xors first: (bin ^ (~value & 0x7f)) + 1 carries into
// bit 7 exactly when bin == value).
// `pairRows` holds 8 dwords per tree, one per level: byte offset of the level's bucket in the tile (bucket * 128,
// bits 7-16) | xor byte (bits 0-6) | the value added to each of the four bins << 24, slot 0 also bit 23 when some
// level of the tree xors (PackedPairTreeIndexes). Levels past the tree's depth are zero (bucket 0, add 0: never
// true). A lane keeps its tree's row in registers (two 16-byte loads, the same addresses for the 32 lanes of a
// group; with offsets and values to add as a dword each the row took four, and the kernel, which is bound by the
// bytes its lanes receive over the vector memory path, 49 ms instead of 41 on 10M documents x 5000 trees) and the wave
// publishes the two trees' leaf values, which are contiguous in `leaves` (1 << MAXD doubles per tree), in its
// own LDS region. Waves take the pairs round robin; a last tree without a partner is done by wave 0 with both
// groups on the same tree and only the first one adding. Partial sums (one per wave and group) are added in a
// fixed order at the end. The fetches run kPairAhead rounds ahead of the walk without looking at the tree range:
// both tables end with kPairTreePadding trees' worth of zeros. The LDS reads of a pair's levels are issued a round
// before the arithmetic on them, behind the previous pair's leaf values going into the region, so a round's
// instructions never wait for reads of its own (a null tree's levels read row 0).
// With `tileMap` the tile has rowCount rows (MapTileBins) and the offsets in pairRows name rows, not buckets.
// grid = 2 * doc blocks, block = 64 * kTileWaves threads, dynamic LDS = rows * 128 (rounded up to 16) +
// kTileWaves * 2 * max(1 << MAXD, 128) * 8 bytes (the leaf regions, later the partial sums).
constexpr uint32_t kPairRowXorFlag = 1u << 23;  // slot 0 of a tree's row: some level xors
constexpr int kPairAhead = 3;
constexpr int kPairTreePadding = 2 * kTileWaves * kPairAhead;

// Rows of a tile that splits the buckets of more than 127 values in two (`tileMap`, a dword per row: bits 0-15 the
// bucket, bits 16.. what becomes of its bins: 0 as they are, 1 min(bin, 127), 2 max(bin - 127, 0)), byte-parallel.
// A split "bin >= s" of such a bucket then reads the first row (s <= 127) or the second (with s - 127), and every
// level of the model is a 7-bit compare.
// A one-hot bucket of more than 127 values (bins 1 + index of the value) takes two rows as well: the bins up to 127
// as they are and 0 for the others (kTileMapOneHotLow), and bin - 127 for the bins from 128 on, 0 for the others
// (kTileMapHigh does exactly that); "bin == v" reads the first row for v <= 127 and the second, with v - 127,
// otherwise: both are 7-bit equalities against a value that is not 0.
constexpr uint32_t kTileMapLow = 1, kTileMapHigh = 2, kTileMapOneHotLow = 3;

__device__ __forceinline__ uint32_t MapTileBins(uint32_t bins4, uint32_t mode) {
    const uint32_t high = bins4 & 0x80808080u;  // bytes above 127
    if (mode == kTileMapLow) {
        return (bins4 | (high - (high >> 7))) & 0x7f7f7f7fu;
    }
    if (mode == kTileMapOneHotLow) {
        return bins4 & ~((high >> 7) * 0xffu);
    }
    if (mode == kTileMapHigh) {
        return ((bins4 & 0x7f7f7f7fu) + 0x01010101u) & ((high >> 7) * 0xffu);
    }
    return bins4;
}

// The same walk on a tree's row in its packed form, one dword per level: bits 7-16 the byte offset of the level's
// row in a tile of 128-byte rows, bits 0-6 the xor byte, bits 24-31 the value added to each of the four bins (bit
// 23 of slot 0: some level of the tree xors). laneOffset is the lane's offset inside a row; the tile starts at LDS
// address 0 (the kernel has no other LDS). A pair of trees then costs a lane two 16-byte loads instead of four:
// the pair-tile kernel is bound by the bytes that the vector memory path delivers to its lanes.
// SIX: every bin of the tile is below 64. The even levels then carry the byte (64 - split), so that their result
// lands in bit 6 while the following level's lands in bit 7, and a pair of levels joins the index with one shift
// and two bit-field inserts: eighteen instructions for eight levels where the one-level-at-a-time form takes
// twenty-four (a one-hot level on an even position xors with the low six bits of its mask).
template <bool XOR, int MAXD, bool SIX>
__device__ __forceinline__ uint32_t PackedPairTreeIndexes(uint32_t laneOffset, const uint4 (&desc)[2]) {
    const uint32_t levels[8] = {desc[0].x, desc[0].y, desc[0].z, desc[0].w, desc[1].x, desc[1].y, desc[1].z, desc[1].w};
    uint32_t a[MAXD];
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        a[d] = *reinterpret_cast<const __attribute__((address_space(3))) uint32_t*>((levels[d] & 0x1ff80u) | laneOffset);
    }
    // one wait for the eight reads (lgkmcnt 0, the other counters untouched)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_sched_barrier(0);
    uint32_t r[MAXD];
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        uint32_t v = a[d];
        if (XOR) {
            const uint32_t x = levels[d] & 0x7fu;
            v ^= __builtin_amdgcn_perm(x, x, 0u);  // the xor byte four times
        }
        r[d] = v + __builtin_amdgcn_perm(levels[d], levels[d], 0x03030303u);  // byte 3 four times
    }
    uint32_t idx4 = 0;
    if constexpr (SIX) {
        static_assert(MAXD % 2 == 0, "levels in pairs");
#pragma unroll
        for (int d = 0; d < MAXD; d += 2) {
            // bit 7 of the odd level, bit 6 of the even one; below them what is left of the even level's sum, which
            // only the first pair lets through: those six bits leave the byte with the shifts that follow (MAXD 8)
            // or end below the six bits that index the leaves (MAXD 6)
            const uint32_t pair = (r[d + 1] & 0x80808080u) | (r[d] & 0x7f7f7f7fu);
            idx4 = d == 0 ? pair : (pair & 0xc0c0c0c0u) | ((idx4 >> 2) & 0x3f3f3f3fu);
        }
    } else {
#pragma unroll
        for (int d = 0; d < MAXD; ++d) {
            idx4 = (r[d] & 0x80808080u) | (idx4 >> 1);
        }
    }
    return idx4;
}

// The two halves of PackedPairTreeIndexes for a kernel that keeps the reads of a tree's levels one round ahead of
// the arithmetic on them: the reads alone, and the walk on what they returned.
template <int MAXD>
__device__ __forceinline__ void ReadPackedPairLevels(uint32_t laneOffset, const uint4 (&desc)[2], uint32_t (&a)[MAXD]) {
    const uint32_t levels[8] = {desc[0].x, desc[0].y, desc[0].z, desc[0].w, desc[1].x, desc[1].y, desc[1].z, desc[1].w};
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        a[d] = *reinterpret_cast<const __attribute__((address_space(3))) uint32_t*>((levels[d] & 0x1ff80u) | laneOffset);
    }
}

template <bool XOR, int MAXD, bool SIX>
__device__ __forceinline__ uint32_t WalkPackedPairLevels(const uint32_t (&a)[MAXD], const uint4 (&desc)[2]) {
    const uint32_t levels[8] = {desc[0].x, desc[0].y, desc[0].z, desc[0].w, desc[1].x, desc[1].y, desc[1].z, desc[1].w};
    uint32_t r[MAXD];
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        uint32_t v = a[d];
        if (XOR) {
            const uint32_t x = levels[d] & 0x7fu;
            v ^= __builtin_amdgcn_perm(x, x, 0u);  // the xor byte four times
        }
        r[d] = v + __builtin_amdgcn_perm(levels[d], levels[d], 0x03030303u);  // byte 3 four times
    }
    uint32_t idx4 = 0;
    if constexpr (SIX) {
        static_assert(MAXD % 2 == 0, "levels in pairs");
#pragma unroll
        for (int d = 0; d < MAXD; d += 2) {
            const uint32_t pair = (r[d + 1] & 0x80808080u) | (r[d] & 0x7f7f7f7fu);
            idx4 = d == 0 ? pair : (pair & 0xc0c0c0c0u) | ((idx4 >> 2) & 0x3f3f3f3fu);
        }
    } else {
#pragma unroll
        for (int d = 0; d < MAXD; ++d) {
            idx4 = (r[d] & 0x80808080u) | (idx4 >> 1);
        }
    }
    return idx4;
}

template <bool XOR, int MAXD>
__device__ __forceinline__ uint32_t PairTreeIndexes(const uint8_t* laneTile, const uint4 (&desc)[4]) {
    const uint32_t offs[8] = {desc[0].x, desc[0].y, desc[0].z, desc[0].w, desc[1].x, desc[1].y, desc[1].z, desc[1].w};
    const uint32_t adds[8] = {desc[2].x, desc[2].y, desc[2].z, desc[2].w, desc[3].x, desc[3].y, desc[3].z, desc[3].w};
    uint32_t a[MAXD];
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        // rows of trees that never xor hold the plain offset
        a[d] = *reinterpret_cast<const uint32_t*>(laneTile + (XOR ? offs[d] & 0x007fffffu : offs[d]));
    }
    // one wait for the eight reads instead of one per read: LDS returns them in order a few cycles apart, and
    // every wait takes an issue slot (lgkmcnt 0, the other counters untouched)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_sched_barrier(0);
    uint32_t idx4 = 0;
#pragma unroll
    for (int d = 0; d < MAXD; ++d) {
        uint32_t v = a[d];
        if (XOR) {
            v ^= __builtin_amdgcn_perm(offs[d], offs[d], 0x03030303u);  // the xor byte four times
        }
        // the level's four result bits go to bit 7 of the bytes; earlier levels move down one bit and never
        // reach the byte below within eight levels
        idx4 = ((v + adds[d]) & 0x80808080u) | (idx4 >> 1);
    }
    return idx4;
}

template <int MAXD, bool SIX>
__global__ __launch_bounds__(64 * kTileWaves) void EvalObliviousPairTileKernel(
    const uint16_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ tileMap,
    uint32_t rowCount, const uint4* __restrict__ pairRows, const double2* __restrict__ leaves2,
    const double* __restrict__ bias, double scale, uint32_t treeBegin, uint32_t treeEnd, double* __restrict__ out) {
    constexpr uint32_t kLeaves = 1u << MAXD;
    constexpr int kLeafRegs = MAXD == 8 ? 4 : 1;  // 16-byte pieces of a pair's 2 * kLeaves leaf values per lane
    static_assert(MAXD == 8 || MAXD == 6, "64 or 256 leaves per tree");
    // s_waitcnt that lets the loads of two pairs (two 16-byte pieces of a row and kLeafRegs of leaf values each)
    // stay in flight: vmcnt in bits 0-3 and 14-15, the other counters untouched
    // (of the pair behind the oldest, its row has to be there as well: its levels are read a round early)
    constexpr int kLoadsBehind = kLeafRegs + (2 + kLeafRegs);
    constexpr int kWaitForOldestPair = (kLoadsBehind & 0xf) | ((kLoadsBehind >> 4) << 14) | 0x0f70;
    // s_waitcnt for the level reads of this round: the previous round's gathers and this round's stores were issued
    // behind them (LDS serves a wave's requests in order); vmcnt and expcnt untouched
    constexpr int kWaitForLevelReads = 0xc07f | ((4 + kLeafRegs) << 8);
    constexpr int kWaitForGathers = 0xc07f | ((kLeafRegs + MAXD) << 8);
    extern __shared__ uint32_t sTile[];
    uint16_t* sTile16 = reinterpret_cast<uint16_t*>(sTile);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x >> 1;
    const uint32_t half = blockIdx.x & 1;
    const uint32_t tileWords = rowCount * kWave;  // rowCount = bucketCount without a map
    const uint16_t* src = bins + block * (bucketCount * kWave) * 2 + half;
    if (tileMap == nullptr) {
        for (uint32_t i = tid; i < tileWords; i += 64 * kTileWaves) {
            sTile16[i] = src[2 * i];
        }
    } else {
        for (uint32_t row = wave; row < rowCount; row += kTileWaves) {
            const uint32_t entry = tileMap[row];
            const uint32_t bins2 = src[2 * ((entry & 0xffffu) * kWave + lane)];
            sTile16[row * kWave + lane] = static_cast<uint16_t>(MapTileBins(bins2, entry >> 16));
        }
    }
    const uint32_t group = lane >> 5;
    const uint32_t tileBytes = (tileWords * 2 + 15) & ~15u;
    double* leafArea = reinterpret_cast<double*>(reinterpret_cast<uint8_t*>(sTile) + tileBytes);
    double2* sLeafWave2 = reinterpret_cast<double2*>(leafArea + wave * 2 * kLeaves);
    const double* sLeafMine = leafArea + wave * 2 * kLeaves + group * kLeaves;
    const uint32_t laneOffset = (lane & 31) * 4;
    __syncthreads();  // tile is loaded

    const uint32_t treeCount = treeEnd - treeBegin;
    const uint32_t pairCount = treeCount / 2;
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    constexpr int kAhead = kPairAhead;
    uint4 rows[kAhead][2];
    double2 pref[kAhead][kLeafRegs];
    // what a lane fetches of the pair that starts at tree `first`: its group's row and its pieces of the
    // two trees' leaf values
    const uint4* myRows = pairRows + group * 2;
    const double2* myLeaves = leaves2 + lane;
#define CBAMD_FETCH_PAIR(k, first)                                                                 \
    do {                                                                                           \
        const uint4* row = myRows + static_cast<size_t>(first) * 2;                                \
        _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                            \
            rows[k][i] = row[i];                                                                   \
        }                                                                                          \
        /* the row first: the round before the pair's own waits for it alone */                   \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        const double2* values = myLeaves + static_cast<size_t>(first) * (kLeaves / 2);             \
        _Pragma("unroll") for (int i = 0; i < kLeafRegs; ++i) {                                    \
            pref[k][i] = values[i * kWave];                                                        \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
    } while (0)
    // the pair's leaf values into the wave's LDS region (the previous pair's gathers were issued before these
    // stores and LDS serves one wave's requests in order), then the levels: four leaf indexes per lane
#define CBAMD_PUBLISH_AND_WALK(k, idx4)                                                            \
    do {                                                                                           \
        _Pragma("unroll") for (int i = 0; i < kLeafRegs; ++i) {                                    \
            sLeafWave2[i * kWave + lane] = pref[k][i];                                             \
        }                                                                                          \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                     \
        __builtin_amdgcn_wave_barrier();                                                           \
        const uint32_t flags =                                                                     \
            __builtin_amdgcn_readlane(rows[k][0].x, 0) | __builtin_amdgcn_readlane(rows[k][0].x, 32); \
        if (flags & kPairRowXorFlag) {                                                             \
            idx4 = PackedPairTreeIndexes<true, MAXD, SIX>(laneOffset, rows[k]);                    \
        } else {                                                                                   \
            idx4 = PackedPairTreeIndexes<false, MAXD, SIX>(laneOffset, rows[k]);                   \
        }                                                                                          \
    } while (0)

    // One round of a wave: the leaf values that the previous round gathered are added while this round's LDS
    // reads are under way; the registers of this pair take the pair kAhead rounds ahead as soon as every level
    // has read them (the loads then land in those registers), and the gathers go out last.
    double gathered[4] = {0.0, 0.0, 0.0, 0.0};
    uint32_t levelBins[kAhead][MAXD];  // what the reads of a pair's levels returned, issued a round before their use
#define CBAMD_PAIR_ROUND(k)                                                                        \
    do {                                                                                           \
        constexpr int kn = (k + 1) % kAhead;                                                       \
        uint32_t idx4;                                                                             \
        /* one wait for this pair's loads and the next pair's row: the later loads stay in flight */ \
        __builtin_amdgcn_s_waitcnt(kWaitForOldestPair);                                            \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        _Pragma("unroll") for (int i = 0; i < kLeafRegs; ++i) {                                    \
            sLeafWave2[i * kWave + lane] = pref[k][i];                                             \
        }                                                                                          \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                     \
        __builtin_amdgcn_wave_barrier();                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        __builtin_amdgcn_s_waitcnt(kWaitForLevelReads);                                            \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        /* the next pair's levels are read while this pair's are worked on */                     \
        ReadPackedPairLevels<MAXD>(laneOffset, rows[kn], levelBins[kn]);                           \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        const uint32_t flags =                                                                     \
            __builtin_amdgcn_readlane(rows[k][0].x, 0) | __builtin_amdgcn_readlane(rows[k][0].x, 32); \
        if (flags & kPairRowXorFlag) {                                                             \
            idx4 = WalkPackedPairLevels<true, MAXD, SIX>(levelBins[k], rows[k]);                   \
        } else {                                                                                   \
            idx4 = WalkPackedPairLevels<false, MAXD, SIX>(levelBins[k], rows[k]);                  \
        }                                                                                          \
        /* the previous round's gathers: this round's stores and reads were issued behind them */ \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        __builtin_amdgcn_s_waitcnt(kWaitForGathers);                                               \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            acc[q] = __dadd_rn(acc[q], gathered[q]);                                               \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        CBAMD_FETCH_PAIR(k, treeBegin + 2 * (p + kAhead * kTileWaves));                            \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            gathered[q] = sLeafMine[(idx4 >> (8 * q + 8 - MAXD)) & (kLeaves - 1)];                 \
        }                                                                                          \
        __builtin_amdgcn_wave_barrier();                                                           \
        p += kTileWaves;                                                                           \
    } while (0)

    uint32_t p = wave;
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
        // (written before the loads so that the arrays stay in registers)
#pragma unroll
        for (int i = 0; i < kLeafRegs; ++i) {
            pref[k][i] = {0.0, 0.0};
        }
        CBAMD_FETCH_PAIR(k, treeBegin + 2 * (p + k * kTileWaves));
    }
    static_assert(kAhead == 3, "the rounds below are written out for three register sets");
#pragma unroll
    for (int k = 1; k < kAhead; ++k) {
#pragma unroll
        for (int d = 0; d < MAXD; ++d) {
            levelBins[k][d] = 0;
        }
    }
    ReadPackedPairLevels<MAXD>(laneOffset, rows[0], levelBins[0]);  // the first pair's levels
    __builtin_amdgcn_s_waitcnt(0xc07f);  // (so that the rounds' waits need not cover this way into the loop)
    // whole turns of the three register sets without a branch between the rounds, so that the waits for
    // the loads count only the loads that are older than the one needed
    while (p + 2 * kTileWaves < pairCount) {
        CBAMD_PAIR_ROUND(0);
        CBAMD_PAIR_ROUND(1);
        CBAMD_PAIR_ROUND(2);
    }
    if (p < pairCount) {
        CBAMD_PAIR_ROUND(0);
        if (p < pairCount) {
            CBAMD_PAIR_ROUND(1);
        }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        acc[q] = __dadd_rn(acc[q], gathered[q]);
    }
    if ((treeCount & 1) && wave == 0) {
        // the last tree has no partner: both groups walk it (its row and its leaf values twice), the first adds
        const uint4* row = pairRows + static_cast<size_t>(treeEnd - 1) * 2;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            rows[0][i] = row[i];
        }
        const double2* values = leaves2 + static_cast<size_t>(treeEnd - 1) * (kLeaves / 2);
#pragma unroll
        for (int i = 0; i < kLeafRegs; ++i) {
            pref[0][i] = values[(i * kWave + lane) & (kLeaves / 2 - 1)];
        }
        uint32_t idx4;
        CBAMD_PUBLISH_AND_WALK(0, idx4);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const double v = sLeafMine[(idx4 >> (8 * q + 8 - MAXD)) & (kLeaves - 1)];
            acc[q] = __dadd_rn(acc[q], group == 0 ? v : 0.0);
        }
        __builtin_amdgcn_wave_barrier();
    }
#undef CBAMD_PAIR_ROUND
#undef CBAMD_FETCH_PAIR
#undef CBAMD_PUBLISH_AND_WALK
    __syncthreads();  // every wave is through with its leaf region: the area now takes the partial sums
    // partial sums as [wave][group][document of the tile], then one thread per document adds the sixteen
    double* sRed = leafArea;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        // byte q of a lane's dword: document (q & 1) * 64 + 2 * (lane & 31) + (q >> 1) of the tile
        const uint32_t docInTile = (q & 1) * kWave + 2 * (lane & 31) + (q >> 1);
        sRed[(wave * 2 + group) * 128 + docInTile] = acc[q];
    }
    __syncthreads();
    if (tid < 128) {
        double sum = sRed[tid];
#pragma unroll
        for (int part = 1; part < 2 * kTileWaves; ++part) {
            sum = __dadd_rn(sum, sRed[part * 128 + tid]);
        }
        const size_t doc = block * kDocsPerBlock + (2 * half + (tid >> 6)) * kWave + (tid & 63);
        if (doc < docCount) {
            out[doc] = Finish(sum, scale, bias[0], treeBegin == 0);
        }
    }
}

// The same with four trees per wave on a quarter of a block, for models whose rows do not fit the half tile: the
// tile holds the bins of 64 documents (documents quarter * 64 + l of the block in byte l of a row), lanes 16 g ..
// 16 g + 15 walk tree g of a quad of trees, each lane for the four documents of one dword. The rows are pairRows
// with 64 bytes per row of the tile; rows and leaf values are fetched three rounds ahead, so both tables end with
// kQuadTreePadding null trees.
// WAVES = 8, or 4 when the rows leave LDS for four waves' regions only.
// grid = 4 * doc blocks, block = 64 * WAVES threads, dynamic LDS = rows * 64 (rounded up to 16) +
// WAVES * 4 * (1 << MAXD) * 8 bytes (the leaf regions, later the partial sums).
constexpr int kQuadTreePadding = 4 * kTileWaves * kPairAhead;

template <int MAXD, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void EvalObliviousQuadTileKernel(
    const uint8_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ tileMap,
    uint32_t rowCount, const uint4* __restrict__ pairRows, const double2* __restrict__ leaves2,
    const double* __restrict__ bias, double scale, uint32_t treeBegin, uint32_t treeEnd, double* __restrict__ out) {
    constexpr uint32_t kLeaves = 1u << MAXD;
    constexpr int kLeafRegs = MAXD == 8 ? 8 : 2;  // 16-byte pieces of a quad's 4 * kLeaves leaf values per lane
    static_assert(MAXD == 8 || MAXD == 6, "64 or 256 leaves per tree");
    extern __shared__ uint32_t sTile[];
    uint8_t* sTile8 = reinterpret_cast<uint8_t*>(sTile);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x >> 2;
    const uint32_t quarter = blockIdx.x & 3;
    const uint32_t tileBytesUsed = rowCount * kWave;  // rowCount = bucketCount without a map
    const uint8_t* src = bins + block * (bucketCount * kWave) * 4 + quarter;
    if (tileMap == nullptr) {
        for (uint32_t i = tid; i < tileBytesUsed; i += 64 * WAVES) {
            sTile8[i] = src[4 * i];
        }
    } else {
        for (uint32_t row = wave; row < rowCount; row += WAVES) {
            const uint32_t entry = tileMap[row];
            const uint32_t bin = src[4 * ((entry & 0xffffu) * kWave + lane)];
            sTile8[row * kWave + lane] = static_cast<uint8_t>(MapTileBins(bin, entry >> 16));
        }
    }
    const uint32_t group = lane >> 4;
    const uint32_t tileBytes = (tileBytesUsed + 15) & ~15u;
    double* leafArea = reinterpret_cast<double*>(reinterpret_cast<uint8_t*>(sTile) + tileBytes);
    double2* sLeafWave2 = reinterpret_cast<double2*>(leafArea + wave * 4 * kLeaves);
    const double* sLeafMine = leafArea + wave * 4 * kLeaves + group * kLeaves;
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + (lane & 15) * 4;
    __syncthreads();  // tile is loaded

    const uint32_t treeCount = treeEnd - treeBegin;
    const uint32_t pairCount = treeCount / 4;  // whole quads of trees
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    constexpr int kAhead = kPairAhead;
    uint4 rows[kAhead][4];
    double2 pref[kAhead][kLeafRegs];
    // what a lane fetches of the quad that starts at tree `first`: its group's row and its pieces of the
    // four trees' leaf values
    const uint4* myRows = pairRows + group * 4;
    const double2* myLeaves = leaves2 + lane;
#define CBAMD_FETCH_PAIR(k, first)                                                                 \
    do {                                                                                           \
        const uint4* row = myRows + static_cast<size_t>(first) * 4;                                \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                            \
            rows[k][i] = row[i];                                                                   \
        }                                                                                          \
        const double2* values = myLeaves + static_cast<size_t>(first) * (kLeaves / 2);             \
        _Pragma("unroll") for (int i = 0; i < kLeafRegs; ++i) {                                    \
            pref[k][i] = values[i * kWave];                                                        \
        }                                                                                          \
    } while (0)
    // the quad's leaf values into the wave's LDS region (the previous quad's gathers were issued before these
    // stores and LDS serves one wave's requests in order), then the levels: four leaf indexes per lane
#define CBAMD_PUBLISH_AND_WALK(k, idx4)                                                            \
    do {                                                                                           \
        _Pragma("unroll") for (int i = 0; i < kLeafRegs; ++i) {                                    \
            sLeafWave2[i * kWave + lane] = pref[k][i];                                             \
        }                                                                                          \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                     \
        __builtin_amdgcn_wave_barrier();                                                           \
        const uint32_t flags =                                                                     \
            __builtin_amdgcn_readlane(rows[k][0].x, 0) | __builtin_amdgcn_readlane(rows[k][0].x, 16) | \
            __builtin_amdgcn_readlane(rows[k][0].x, 32) | __builtin_amdgcn_readlane(rows[k][0].x, 48); \
        if (flags & kPairRowXorFlag) {                                                             \
            idx4 = PairTreeIndexes<true, MAXD>(laneTile, rows[k]);                                 \
        } else {                                                                                   \
            idx4 = PairTreeIndexes<false, MAXD>(laneTile, rows[k]);                                \
        }                                                                                          \
    } while (0)

    // One round of a wave: the leaf values that the previous round gathered are added while this round's LDS
    // reads are under way; the registers of this quad take the quad kAhead rounds ahead as soon as every level
    // has read them (the loads then land in those registers), and the gathers go out last.
    constexpr int kLoadsBehind = 2 * (4 + kLeafRegs);
    constexpr int kWaitLoads = 0x0f70 | (kLoadsBehind & 15) | ((kLoadsBehind >> 4) << 14);  // vmcnt(kLoadsBehind)
    double gathered[4] = {0.0, 0.0, 0.0, 0.0};
#define CBAMD_PAIR_ROUND(k)                                                                        \
    do {                                                                                           \
        uint32_t idx4;                                                                             \
        /* one wait for this quad's loads: those of the two quads behind it stay in flight */       \
        __builtin_amdgcn_s_waitcnt(kWaitLoads);                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        CBAMD_PUBLISH_AND_WALK(k, idx4);                                                           \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            acc[q] = __dadd_rn(acc[q], gathered[q]);                                               \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        CBAMD_FETCH_PAIR(k, treeBegin + 4 * (p + kAhead * WAVES));                            \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            gathered[q] = sLeafMine[(idx4 >> (8 * q + 8 - MAXD)) & (kLeaves - 1)];                 \
        }                                                                                          \
        __builtin_amdgcn_wave_barrier();                                                           \
        p += WAVES;                                                                           \
    } while (0)

    uint32_t p = wave;
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
        // (written before the loads so that the arrays stay in registers)
#pragma unroll
        for (int i = 0; i < kLeafRegs; ++i) {
            pref[k][i] = {0.0, 0.0};
        }
        CBAMD_FETCH_PAIR(k, treeBegin + 4 * (p + k * WAVES));
    }
    static_assert(kAhead == 3, "the rounds below are written out for three register sets");
    // whole turns of the three register sets without a branch between the rounds, so that the waits for
    // the loads count only the loads that are older than the one needed
    while (p + 2 * WAVES < pairCount) {
        CBAMD_PAIR_ROUND(0);
        CBAMD_PAIR_ROUND(1);
        CBAMD_PAIR_ROUND(2);
    }
    if (p < pairCount) {
        CBAMD_PAIR_ROUND(0);
        if (p < pairCount) {
            CBAMD_PAIR_ROUND(1);
        }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        acc[q] = __dadd_rn(acc[q], gathered[q]);
    }
    const uint32_t rest = treeCount & 3;
    if (rest && wave == 0) {
        // the last one to three trees: a group without a tree of its own walks the last one and adds nothing
        const uint32_t base = treeEnd - rest;
        const uint4* row = pairRows + static_cast<size_t>(base + min(group, rest - 1)) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            rows[0][i] = row[i];
        }
#pragma unroll
        for (int i = 0; i < kLeafRegs; ++i) {
            const uint32_t piece = i * kWave + lane;  // of the four trees' regions, kLeaves / 2 pieces each
            const uint32_t tree = base + min(piece / (kLeaves / 2), rest - 1);
            pref[0][i] = leaves2[static_cast<size_t>(tree) * (kLeaves / 2) + piece % (kLeaves / 2)];
        }
        uint32_t idx4;
        CBAMD_PUBLISH_AND_WALK(0, idx4);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const double v = sLeafMine[(idx4 >> (8 * q + 8 - MAXD)) & (kLeaves - 1)];
            acc[q] = __dadd_rn(acc[q], group < rest ? v : 0.0);
        }
        __builtin_amdgcn_wave_barrier();
    }
#undef CBAMD_PAIR_ROUND
#undef CBAMD_FETCH_PAIR
#undef CBAMD_PUBLISH_AND_WALK
    __syncthreads();  // every wave is through with its leaf region: the area now takes the partial sums
    // partial sums as [wave][group][document of the tile], then one thread per document adds the thirty-two
    double* sRed = leafArea;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        // byte q of a lane's dword: document 4 * (lane & 15) + q of the tile
        sRed[(wave * 4 + group) * kWave + 4 * (lane & 15) + q] = acc[q];
    }
    __syncthreads();
    if (tid < kWave) {
        double sum = sRed[tid];
#pragma unroll
        for (int part = 1; part < 4 * WAVES; ++part) {
            sum = __dadd_rn(sum, sRed[part * kWave + tid]);
        }
        const size_t doc = block * kDocsPerBlock + quarter * kWave + tid;
        if (doc < docCount) {
            out[doc] = Finish(sum, scale, bias[0], treeBegin == 0);
        }
    }
}

// Models of 7-bit bins whose 256-document tile fits LDS, one tree per wave: the walk of
// EvalObliviousPairTileKernel on the whole tile. A tree's row is `tileRows` (the format of pairRows with
// bucket * 256 as the byte offset); its address is the same in every lane, so it comes through scalar loads
// and a level is an LDS read and three vector instructions with no lane reads and no scalar arithmetic. The
// leaf values go through the wave's LDS region; rows and values are fetched kPairAhead rounds ahead without
// looking at the tree range (both tables end with kRowTilePadding trees' worth of zeros). Waves take the trees
// round robin; their partial sums are added in wave order through an accumulator in LDS at the end.
// Leaf values: one dimension: (1 << MAXD) values per tree. Several dimensions: a workgroup sums DIMS (2 or 4)
// of them at a time, slice after slice of the model's dimensions over the same tile, every slice with another
// walk of the trees; `leaves2` is [slice][tree][piece][leaf] pairs of values (16 bytes: dimensions 2 * piece and
// 2 * piece + 1 of the slice, zeros past the model's last dimension), sliceStride pairs per slice. A wave's
// 16-byte gathers of one piece then spread over all groups of four LDS banks, which leaf rows of 32 bytes would
// not.
// With `tileMap` the tile has rowCount rows (MapTileBins) and the offsets in tileRows name rows, not buckets.
// grid = doc blocks, block = 64 * WAVES, dynamic LDS = rows * 256 (rounded up to 16) + 256 * DIMS * 8 (the
// accumulator) + WAVES * (1 << MAXD) * DIMS * 8 bytes (the leaf regions).
constexpr int kRowTilePadding = kWideTileWaves * kPairAhead;
static_assert(kRowTilePadding <= kPairTreePadding, "the two kernels share the padded leaf table");

template <int MAXD, int WAVES, int DIMS>
__global__ __launch_bounds__(64 * WAVES) void EvalObliviousRowTileKernel(
    const uint32_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ tileMap,
    uint32_t rowCount, const uint4* __restrict__ tileRows, const double2* __restrict__ leaves2,
    const double* __restrict__ bias, double scale, uint32_t dim, size_t sliceStride, uint32_t treeBegin,
    uint32_t treeEnd, double* __restrict__ out) {
    constexpr uint32_t kLeaves = 1u << MAXD;
    constexpr uint32_t kTreePieces = kLeaves * DIMS / 2;     // 16-byte pieces of a tree's leaf values (of a slice)
    constexpr int kLeafRegs = kTreePieces > kWave ? static_cast<int>(kTreePieces / kWave) : 1;
    constexpr uint32_t kPieceMask = kTreePieces - 1;         // 32 pieces: the upper lanes repeat the lower lanes' pieces
    constexpr int kPairsPerLeaf = DIMS > 1 ? DIMS / 2 : 1;
    constexpr bool kPipelined = DIMS <= 2;  // the values gathered in a round are added during the next one
    static_assert(MAXD == 8 || MAXD == 6, "64 or 256 leaves per tree");
    static_assert(DIMS == 1 || DIMS == 2 || DIMS == 4, "one value or whole pairs per leaf");
    static_assert(WAVES <= kWideTileWaves, "the tables are padded for that many waves");
    extern __shared__ uint32_t sTile[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x;
    const uint32_t tileDwords = rowCount * kWave;  // rowCount = bucketCount without a map
    const uint32_t* src = bins + block * (bucketCount * kWave);
    if (tileMap == nullptr) {
        for (uint32_t i = tid; i < tileDwords; i += 64 * WAVES) {
            sTile[i] = src[i];
        }
    } else {
        for (uint32_t row = wave; row < rowCount; row += WAVES) {
            const uint32_t entry = tileMap[row];
            sTile[row * kWave + lane] = MapTileBins(src[(entry & 0xffffu) * kWave + lane], entry >> 16);
        }
    }
    const uint32_t tileBytes = (tileDwords * 4 + 15) & ~15u;
    double* sRed = reinterpret_cast<double*>(reinterpret_cast<uint8_t*>(sTile) + tileBytes);  // [DIMS][256 documents]
    double* leafArea = sRed + kDocsPerBlock * DIMS;
    double2* sLeafWave2 = reinterpret_cast<double2*>(leafArea + wave * kLeaves * DIMS);
    const double* sLeafMine = leafArea + wave * kLeaves * DIMS;
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + lane * 4;
    const uint32_t treeCount = treeEnd - treeBegin;
    constexpr int kAhead = kPairAhead;
    static_assert(kAhead == 3, "the rounds below are written out for three register sets");

#define CBAMD_FETCH_TREE(k, tree)                                                                  \
    do {                                                                                           \
        const uint4* row = tileRows + static_cast<size_t>(tree) * 4;                               \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                            \
            rows[k][i] = row[i];                                                                   \
        }                                                                                          \
        const double2* values = myLeaves + static_cast<size_t>(tree) * kTreePieces;                \
        _Pragma("unroll") for (int i = 0; i < kLeafRegs; ++i) {                                    \
            pref[k][i] = values[i * kWave];                                                        \
        }                                                                                          \
    } while (0)
    // the tree's leaf values into the wave's LDS region (the previous tree's gathers were issued before these
    // stores and LDS serves one wave's requests in order), then the levels: four leaf indexes per lane
#define CBAMD_PUBLISH_AND_WALK(k, idx4)                                                            \
    do {                                                                                           \
        _Pragma("unroll") for (int i = 0; i < kLeafRegs; ++i) {                                    \
            sLeafWave2[(i * kWave + lane) & kPieceMask] = pref[k][i];                              \
        }                                                                                          \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                     \
        __builtin_amdgcn_wave_barrier();                                                           \
        if (__builtin_amdgcn_readfirstlane(rows[k][0].x) & kPairRowXorFlag) {                      \
            idx4 = PairTreeIndexes<true, MAXD>(laneTile, rows[k]);                                 \
        } else {                                                                                   \
            idx4 = PairTreeIndexes<false, MAXD>(laneTile, rows[k]);                                \
        }                                                                                          \
    } while (0)
    // One round of a wave, as in the two-tree kernel: the values that the previous round gathered are added
    // while this round's LDS reads are under way, the registers of this tree take the tree kAhead rounds ahead
    // as soon as every level has read them, and the gathers go out last.
    constexpr int kLoadsBehind = 2 * kLeafRegs;  // vector loads of the two rounds behind the one that is waited for
    constexpr int kWaitLoads = 0x0f70 | (kLoadsBehind & 15) | ((kLoadsBehind >> 4) << 14);  // vmcnt(kLoadsBehind)
#define CBAMD_TREE_ROUND(k)                                                                        \
    do {                                                                                           \
        uint32_t idx4;                                                                             \
        __builtin_amdgcn_s_waitcnt(kWaitLoads);                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        CBAMD_PUBLISH_AND_WALK(k, idx4);                                                           \
        if constexpr (kPipelined) {                                                                \
            _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                        \
                _Pragma("unroll") for (int c = 0; c < DIMS; ++c) {                                 \
                    acc[q][c] = __dadd_rn(acc[q][c], gathered[q][c]);                              \
                }                                                                                  \
            }                                                                                      \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        CBAMD_FETCH_TREE(k, treeBegin + p + kAhead * WAVES);                                       \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            const uint32_t leaf = (idx4 >> (8 * q + 8 - MAXD)) & (kLeaves - 1);                    \
            if constexpr (DIMS == 1) {                                                             \
                gathered[q][0] = sLeafMine[leaf];                                                  \
            } else {                                                                               \
                _Pragma("unroll") for (int piece = 0; piece < kPairsPerLeaf; ++piece) {            \
                    const double2 pair = reinterpret_cast<const double2*>(sLeafMine)[piece * kLeaves + leaf]; \
                    gathered[q][2 * piece] = pair.x;                                               \
                    gathered[q][2 * piece + 1] = pair.y;                                           \
                }                                                                                  \
            }                                                                                      \
        }                                                                                          \
        if constexpr (!kPipelined) {                                                               \
            /* four dimensions: no registers for values in flight across a round */               \
            _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                        \
                _Pragma("unroll") for (int c = 0; c < DIMS; ++c) {                                 \
                    acc[q][c] = __dadd_rn(acc[q][c], gathered[q][c]);                              \
                    gathered[q][c] = 0.0;                                                          \
                }                                                                                  \
            }                                                                                      \
        }                                                                                          \
        __builtin_amdgcn_wave_barrier();                                                           \
        p += WAVES;                                                                                \
    } while (0)

    const uint32_t slices = (dim + DIMS - 1) / DIMS;
    for (uint32_t slice = 0; slice < slices; ++slice) {
        __syncthreads();  // tile is loaded / the previous slice's accumulator has been read
        double acc[4][DIMS], gathered[4][DIMS];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int c = 0; c < DIMS; ++c) {
                acc[q][c] = 0.0;
                gathered[q][c] = 0.0;
            }
        }
        uint4 rows[kAhead][4];
        double2 pref[kAhead][kLeafRegs];
        const double2* myLeaves = leaves2 + slice * sliceStride + (lane & kPieceMask);
        uint32_t p = wave;
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            // (written before the loads so that the arrays stay in registers)
#pragma unroll
            for (int i = 0; i < kLeafRegs; ++i) {
                pref[k][i] = {0.0, 0.0};
            }
            CBAMD_FETCH_TREE(k, treeBegin + p + k * WAVES);
        }
        // whole turns of the three register sets without a branch between the rounds, so that the waits for
        // the loads count only the loads that are older than the one needed
        while (p + 2 * WAVES < treeCount) {
            CBAMD_TREE_ROUND(0);
            CBAMD_TREE_ROUND(1);
            CBAMD_TREE_ROUND(2);
        }
        if (p < treeCount) {
            CBAMD_TREE_ROUND(0);
            if (p < treeCount) {
                CBAMD_TREE_ROUND(1);
            }
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int c = 0; c < DIMS; ++c) {
                acc[q][c] = __dadd_rn(acc[q][c], gathered[q][c]);
            }
        }
        // waves add their partial sums in wave order into the LDS accumulator; the last wave finishes the values
        // and writes them out (byte q of a lane's dword: document q * 64 + lane)
        for (uint32_t w = 0; w + 1 < WAVES; ++w) {
            if (wave == w) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
#pragma unroll
                    for (int c = 0; c < DIMS; ++c) {
                        double* cell = sRed + c * kDocsPerBlock + q * kWave + lane;
                        *cell = (w == 0) ? acc[q][c] : __dadd_rn(*cell, acc[q][c]);
                    }
                }
            }
            __syncthreads();
        }
        if (wave == WAVES - 1) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const size_t doc = block * kDocsPerBlock + q * kWave + lane;
#pragma unroll
                for (int c = 0; c < DIMS; ++c) {
                    const uint32_t d = slice * DIMS + c;
                    if (doc < docCount && d < dim) {
                        const double sum = __dadd_rn(sRed[c * kDocsPerBlock + q * kWave + lane], acc[q][c]);
                        out[doc * dim + d] = Finish(sum, scale, bias[d], treeBegin == 0);
                    }
                }
            }
        }
    }
#undef CBAMD_TREE_ROUND
#undef CBAMD_FETCH_TREE
#undef CBAMD_PUBLISH_AND_WALK
}

// One-dimensional models of depth 9 to 16 on the same tile, one tree per wave: the walk of the row-tile kernel
// in two halves. `deepRows` holds 32 dwords per tree: the first sixteen as in tileRows for the levels 0..7, the
// second sixteen for the levels 8..8 + HIGH - 1 (levels past the tree's depth: row 0, add 0, never true; the
// flag of slot 0 says whether any level of the tree xors). The two halves give a byte per document each,
// together the leaf index; a tree's table has up to 512 KB, so the leaf values are gathered from global memory,
// `leaves` + firstLeaf[tree], and added one round later. Rows come two rounds ahead (scalar loads: the address
// is the same in every lane). Both tables end with kRowTilePadding null trees.
// grid = doc blocks, block = 64 * WAVES, dynamic LDS = rows * 256 (rounded up to 16) + 256 * 8 bytes.
template <int HIGH, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void EvalObliviousDeepTileKernel(
    const uint32_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ tileMap,
    uint32_t rowCount, const uint4* __restrict__ deepRows, const uint32_t* __restrict__ firstLeaf,
    const double* __restrict__ leaves, const double* __restrict__ bias, double scale, uint32_t treeBegin,
    uint32_t treeEnd, double* __restrict__ out) {
    static_assert(HIGH == 4 || HIGH == 8, "levels 8..11 or 8..15 in the second half");
    extern __shared__ uint32_t sTile[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x;
    const uint32_t tileDwords = rowCount * kWave;  // rowCount = bucketCount without a map
    const uint32_t* src = bins + block * (bucketCount * kWave);
    if (tileMap == nullptr) {
        for (uint32_t i = tid; i < tileDwords; i += 64 * WAVES) {
            sTile[i] = src[i];
        }
    } else {
        for (uint32_t row = wave; row < rowCount; row += WAVES) {
            const uint32_t entry = tileMap[row];
            sTile[row * kWave + lane] = MapTileBins(src[(entry & 0xffffu) * kWave + lane], entry >> 16);
        }
    }
    const uint32_t tileBytes = (tileDwords * 4 + 15) & ~15u;
    double* sRed = reinterpret_cast<double*>(reinterpret_cast<uint8_t*>(sTile) + tileBytes);  // [256 documents]
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + lane * 4;
    const uint32_t treeCount = treeEnd - treeBegin;
    __syncthreads();  // tile is loaded

    double acc[4] = {0.0, 0.0, 0.0, 0.0}, gathered[4] = {0.0, 0.0, 0.0, 0.0};
    uint4 rows[2][2][4];
    uint32_t first[2];
#define CBAMD_FETCH_DEEP(k, tree)                                                                  \
    do {                                                                                           \
        const uint4* row = deepRows + static_cast<size_t>(tree) * 8;                               \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                            \
            rows[k][0][i] = row[i];                                                                \
            rows[k][1][i] = row[4 + i];                                                            \
        }                                                                                          \
        first[k] = firstLeaf[tree];                                                                \
    } while (0)
#define CBAMD_DEEP_ROUND(k)                                                                        \
    do {                                                                                           \
        uint32_t low4, high4;                                                                      \
        if (__builtin_amdgcn_readfirstlane(rows[k][0][0].x) & kPairRowXorFlag) {                   \
            low4 = PairTreeIndexes<true, 8>(laneTile, rows[k][0]);                                 \
            high4 = PairTreeIndexes<true, HIGH>(laneTile, rows[k][1]);                             \
        } else {                                                                                   \
            low4 = PairTreeIndexes<false, 8>(laneTile, rows[k][0]);                                \
            high4 = PairTreeIndexes<false, HIGH>(laneTile, rows[k][1]);                            \
        }                                                                                          \
        const double* treeLeaves = leaves + __builtin_amdgcn_readfirstlane(first[k]);              \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            acc[q] = __dadd_rn(acc[q], gathered[q]);                                               \
        }                                                                                          \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            const uint32_t leaf = ((low4 >> (8 * q)) & 0xffu) |                                    \
                                  (((high4 >> (8 * q + 8 - HIGH)) & ((1u << HIGH) - 1)) << 8);     \
            gathered[q] = treeLeaves[leaf];                                                        \
        }                                                                                          \
        CBAMD_FETCH_DEEP(k, treeBegin + p + 2 * WAVES);                                            \
        p += WAVES;                                                                                \
    } while (0)

    uint32_t p = wave;
    CBAMD_FETCH_DEEP(0, treeBegin + p);
    CBAMD_FETCH_DEEP(1, treeBegin + p + WAVES);
    while (p + WAVES < treeCount) {
        CBAMD_DEEP_ROUND(0);
        CBAMD_DEEP_ROUND(1);
    }
    if (p < treeCount) {
        CBAMD_DEEP_ROUND(0);
    }
#undef CBAMD_DEEP_ROUND
#undef CBAMD_FETCH_DEEP
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        acc[q] = __dadd_rn(acc[q], gathered[q]);
    }
    // waves add their partial sums in wave order into the LDS accumulator; the last wave finishes the values
    // and writes them out (byte q of a lane's dword: document q * 64 + lane)
    for (uint32_t w = 0; w + 1 < WAVES; ++w) {
        if (wave == w) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                double* cell = sRed + q * kWave + lane;
                *cell = (w == 0) ? acc[q] : __dadd_rn(*cell, acc[q]);
            }
        }
        __syncthreads();
    }
    if (wave == WAVES - 1) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const size_t doc = block * kDocsPerBlock + q * kWave + lane;
            if (doc < docCount) {
                out[doc] = Finish(__dadd_rn(sRed[q * kWave + lane], acc[q]), scale, bias[0], treeBegin == 0);
            }
        }
    }
}

// EvalObliviousDeepTileKernel for models of several dimensions: the same tile, rows and walk; a workgroup sums two
// dimensions, those from blockIdx.y * 2 on (every slice of the dimensions walks the trees again). `leaves` holds the
// values slice by slice, [slice][tree][leaf][2] (zeros past the last dimension), `firstLeaf` counts leaves and
// `sliceLeaves` is the number of leaves of all trees, so that a leaf's two values come with one 16-byte load:
// gathered as two strided doubles from the model's own table the kernel was no faster than the plain one (the
// gathers' way through the texture path is what it waits for). A kernel of its own: as a template parameter of
// the one-dimensional kernel the second dimension cost that kernel 5 %.
// grid = (doc blocks, ceil(dim / 2)), block = 64 * WAVES, dynamic LDS = rows * 256 (rounded up to 16) + 2 * 256 * 8 bytes.
template <int HIGH, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void EvalObliviousDeepTilePairsKernel(
    const uint32_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ tileMap,
    uint32_t rowCount, const uint4* __restrict__ deepRows, const uint32_t* __restrict__ firstLeaf,
    const double* __restrict__ leaves, const double* __restrict__ bias, double scale, uint32_t dim, uint32_t sliceLeaves,
    uint32_t treeBegin, uint32_t treeEnd, double* __restrict__ out) {
    static_assert(HIGH == 4 || HIGH == 8, "levels 8..11 or 8..15 in the second half");
    constexpr int DIMS = 2;
    const uint32_t d0 = blockIdx.y * DIMS;
    leaves += static_cast<size_t>(blockIdx.y) * sliceLeaves * 2;
    extern __shared__ uint32_t sTile[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x;
    const uint32_t tileDwords = rowCount * kWave;  // rowCount = bucketCount without a map
    const uint32_t* src = bins + block * (bucketCount * kWave);
    if (tileMap == nullptr) {
        for (uint32_t i = tid; i < tileDwords; i += 64 * WAVES) {
            sTile[i] = src[i];
        }
    } else {
        for (uint32_t row = wave; row < rowCount; row += WAVES) {
            const uint32_t entry = tileMap[row];
            sTile[row * kWave + lane] = MapTileBins(src[(entry & 0xffffu) * kWave + lane], entry >> 16);
        }
    }
    const uint32_t tileBytes = (tileDwords * 4 + 15) & ~15u;
    double* sRed = reinterpret_cast<double*>(reinterpret_cast<uint8_t*>(sTile) + tileBytes);  // [DIMS][256 documents]
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + lane * 4;
    const uint32_t treeCount = treeEnd - treeBegin;
    __syncthreads();  // tile is loaded

    double acc[4][DIMS], gathered[4][DIMS];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int c = 0; c < DIMS; ++c) {
            acc[q][c] = 0.0;
            gathered[q][c] = 0.0;
        }
    }
    uint4 rows[2][2][4];
    uint32_t first[2];
#define CBAMD_FETCH_DEEP2(k, tree)                                                                  \
    do {                                                                                           \
        const uint4* row = deepRows + static_cast<size_t>(tree) * 8;                               \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                            \
            rows[k][0][i] = row[i];                                                                \
            rows[k][1][i] = row[4 + i];                                                            \
        }                                                                                          \
        first[k] = firstLeaf[tree];                                                                \
    } while (0)
#define CBAMD_DEEP_ROUND2(k)                                                                        \
    do {                                                                                           \
        uint32_t low4, high4;                                                                      \
        if (__builtin_amdgcn_readfirstlane(rows[k][0][0].x) & kPairRowXorFlag) {                   \
            low4 = PairTreeIndexes<true, 8>(laneTile, rows[k][0]);                                 \
            high4 = PairTreeIndexes<true, HIGH>(laneTile, rows[k][1]);                             \
        } else {                                                                                   \
            low4 = PairTreeIndexes<false, 8>(laneTile, rows[k][0]);                                \
            high4 = PairTreeIndexes<false, HIGH>(laneTile, rows[k][1]);                            \
        }                                                                                          \
        const double* treeLeaves = leaves + static_cast<size_t>(__builtin_amdgcn_readfirstlane(first[k])) * DIMS; \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            _Pragma("unroll") for (int c = 0; c < DIMS; ++c) {                                     \
                acc[q][c] = __dadd_rn(acc[q][c], gathered[q][c]);                                  \
            }                                                                                      \
        }                                                                                          \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                            \
            const uint32_t leaf = ((low4 >> (8 * q)) & 0xffu) |                                    \
                                  (((high4 >> (8 * q + 8 - HIGH)) & ((1u << HIGH) - 1)) << 8);     \
            const double2 pair = reinterpret_cast<const double2*>(treeLeaves)[leaf];               \
            gathered[q][0] = pair.x;                                                               \
            gathered[q][1] = pair.y;                                                               \
        }                                                                                          \
        CBAMD_FETCH_DEEP2(k, treeBegin + p + 2 * WAVES);                                            \
        p += WAVES;                                                                                \
    } while (0)

    uint32_t p = wave;
    CBAMD_FETCH_DEEP2(0, treeBegin + p);
    CBAMD_FETCH_DEEP2(1, treeBegin + p + WAVES);
    while (p + WAVES < treeCount) {
        CBAMD_DEEP_ROUND2(0);
        CBAMD_DEEP_ROUND2(1);
    }
    if (p < treeCount) {
        CBAMD_DEEP_ROUND2(0);
    }
#undef CBAMD_DEEP_ROUND2
#undef CBAMD_FETCH_DEEP2
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int c = 0; c < DIMS; ++c) {
            acc[q][c] = __dadd_rn(acc[q][c], gathered[q][c]);
        }
    }
    // waves add their partial sums in wave order into the LDS accumulator; the last wave finishes the values
    // and writes them out (byte q of a lane's dword: document q * 64 + lane)
    for (uint32_t w = 0; w + 1 < WAVES; ++w) {
        if (wave == w) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int c = 0; c < DIMS; ++c) {
                    double* cell = sRed + c * kDocsPerBlock + q * kWave + lane;
                    *cell = (w == 0) ? acc[q][c] : __dadd_rn(*cell, acc[q][c]);
                }
            }
        }
        __syncthreads();
    }
    if (wave == WAVES - 1) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const size_t doc = block * kDocsPerBlock + q * kWave + lane;
#pragma unroll
            for (int c = 0; c < DIMS; ++c) {
                if (doc < docCount && d0 + c < dim) {
                    out[doc * dim + d0 + c] = Finish(__dadd_rn(sRed[c * kDocsPerBlock + q * kWave + lane], acc[q][c]), scale,
                                                     bias[d0 + c], treeBegin == 0);
                }
            }
        }
    }
}

__device__ __forceinline__ uint32_t BinOfDoc(const uint8_t* bins, size_t doc, uint32_t bucketCount, uint32_t bucket) {
    const size_t block = doc / kDocsPerBlock;
    const uint32_t r = static_cast<uint32_t>(doc % kDocsPerBlock);
    return bins[((block * bucketCount + bucket) * kWave + (r % kWave)) * 4 + r / kWave];
}

// Walks one non-symmetric tree for one document; returns the terminal node id
// (CalcIndexesNonSymmetric, cpu/evaluator_impl.cpp:462-493).
__device__ __forceinline__ uint32_t WalkNonSymmetric(const uint8_t* bins, size_t doc, uint32_t bucketCount,
                                                     const TTreeTables& tt, uint32_t tree) {
    uint32_t node = tt.TreeStart[tree];
    for (;;) {
        const uint32_t sp = tt.Splits[node];
        const uint32_t st = tt.StepNodes[node];
        const uint32_t b = BinOfDoc(bins, doc, bucketCount, sp & 0xffffu);
        const bool right = ((b ^ ((sp >> 16) & 0xffu)) >= (sp >> 24));
        const uint32_t diff = right ? (st >> 16) : (st & 0xffffu);
        if (diff == 0) {
            return node;
        }
        node += diff;
    }
}

// Non-symmetric trees: one thread per document. grid = ceil(docs / 256), block = 256.
template <int DCHUNK>
__global__ __launch_bounds__(256) void EvalNonSymmetricKernel(const uint8_t* __restrict__ bins, size_t docCount,
                                                              uint32_t bucketCount, TTreeTables tt, uint32_t treeBegin,
                                                              uint32_t treeEnd, double* __restrict__ out) {
    const size_t doc = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (doc >= docCount) {
        return;
    }
    const int dim = tt.Dim;
    const bool addBias = treeBegin == 0;
    for (int d0 = 0; d0 < dim; d0 += DCHUNK) {
        double acc[DCHUNK];
#pragma unroll
        for (int k = 0; k < DCHUNK; ++k) {
            acc[k] = 0.0;
        }
        for (uint32_t t = treeBegin; t < treeEnd; ++t) {
            const uint32_t node = WalkNonSymmetric(bins, doc, bucketCount, tt, t);
            const double* p = tt.Leaves + tt.NodeToLeaf[node] + d0;
#pragma unroll
            for (int k = 0; k < DCHUNK; ++k) {
                if (DCHUNK == 1 || d0 + k < dim) {
                    acc[k] = __dadd_rn(acc[k], p[k]);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < DCHUNK; ++k) {
            if (DCHUNK == 1 || d0 + k < dim) {
                out[doc * dim + d0 + k] = Finish(acc[k], tt.Scale, tt.Bias[d0 + k], addBias);
            }
        }
    }
}

// Non-symmetric trees over an LDS tile of bins: one workgroup of kTileWaves waves per
// 256-document block, the waves split the trees in groups of kNsGroup consecutive trees, four
// documents per lane walk the trees of a group side by side (4 * kNsGroup independent chains).
// The trees come re-laid level by level: an entry is 8 bytes,
//   x: NO_XOR   bucket << 8 | splitIdx << 24          (bucket << 8 = offset of the bucket in the tile)
//      else     bucket | xorMask << 16 | splitIdx << 24
//   y: byte offset (entry index * 8, relative to the tree's first entry) of the left child in the
//      low half and of the right child in the high half.
// A terminal entry has x = 0 (true for every bin), its own offset as right child and, in the low
// half of y, the index of its leaf relative to the tree's first leaf. All lanes take the same
// number of steps (the height of the tallest tree of the group): a lane that has reached its leaf
// stays there. Since
// the lanes of a wave are always on the same level, their gathers of a step fall into the few
// cache lines of that level.
// treeRows: 4 dwords per tree: first entry, height, first leaf value, unused.
// grid = doc blocks, block = 64 * kTileWaves, dynamic LDS = buckets * 256 (rounded up to 8) +
// 256 * DCHUNK * 8 bytes.
constexpr int kNsGroup = 4;

template <bool NO_XOR, int DCHUNK>
__global__ __launch_bounds__(64 * kTileWaves) void EvalNonSymmetricTileKernel(
    const uint32_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint2* __restrict__ entries,
    const uint4* __restrict__ treeRows, const double* __restrict__ leaves, const double* __restrict__ bias, double scale,
    int dim, uint32_t treeBegin, uint32_t treeEnd, double* __restrict__ out) {
    extern __shared__ uint32_t sTile[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x;
    const uint32_t tileDwords = bucketCount * kWave;
    const uint32_t* src = bins + block * tileDwords;
    for (uint32_t i = tid; i < tileDwords; i += 64 * kTileWaves) {
        sTile[i] = src[i];
    }
    const bool addBias = treeBegin == 0;
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + lane * 4;
    double* sRed = reinterpret_cast<double*>(sTile + ((tileDwords + 1) & ~1u));
    for (int d0 = 0; d0 < dim; d0 += DCHUNK) {
        __syncthreads();  // tile is loaded / the previous chunk's accumulator has been read
        double acc[4][DCHUNK];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int k = 0; k < DCHUNK; ++k) {
                acc[j][k] = 0.0;
            }
        }
        // a wave walks kNsGroup trees at a time (trees t0 .. t0 + kNsGroup - 1), i.e. 4 * kNsGroup
        // independent chains per lane, to cover the latency of the entry gathers
        for (uint32_t t0 = treeBegin + wave * kNsGroup; t0 < treeEnd; t0 += kTileWaves * kNsGroup) {
            const char* base[kNsGroup];
            uint32_t firstLeaf[kNsGroup];
            uint32_t height = 0;
#pragma unroll
            for (int g = 0; g < kNsGroup; ++g) {
                // trees past the end walk tree t0 again and are not added
                const uint4 row = treeRows[t0 + g < treeEnd ? t0 + g : t0];
                base[g] = reinterpret_cast<const char*>(entries + __builtin_amdgcn_readfirstlane(row.x));
                height = max(height, static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(row.y)));
                firstLeaf[g] = __builtin_amdgcn_readfirstlane(row.z);
            }
            uint32_t off[kNsGroup][4];
#pragma unroll
            for (int g = 0; g < kNsGroup; ++g) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    off[g][j] = 0;
                }
            }
            for (uint32_t step = 0; step < height; ++step) {
                uint2 node[kNsGroup][4];
#pragma unroll
                for (int g = 0; g < kNsGroup; ++g) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        node[g][j] = *reinterpret_cast<const uint2*>(base[g] + off[g][j]);
                    }
                }
#pragma unroll
                for (int g = 0; g < kNsGroup; ++g) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t x = node[g][j].x;
                        uint32_t bin;
                        if (NO_XOR) {
                            bin = laneTile[(x & 0xffffffu) + j];
                        } else {
                            bin = laneTile[((x & 0xffffu) << 8) + j] ^ ((x >> 16) & 0xffu);
                        }
                        const uint32_t shift = bin >= (x >> 24) ? 16u : 0u;
                        off[g][j] = (node[g][j].y >> shift) & 0xffffu;
                    }
                }
            }
#pragma unroll
            for (int g = 0; g < kNsGroup; ++g) {
                if (t0 + g < treeEnd) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint2 last = *reinterpret_cast<const uint2*>(base[g] + off[g][j]);
                        const uint32_t leafRel = last.y & 0xffffu;
                        const double* p = leaves + firstLeaf[g] +
                                          (DCHUNK == 1 ? leafRel : leafRel * static_cast<uint32_t>(dim)) + d0;
#pragma unroll
                        for (int k = 0; k < DCHUNK; ++k) {
                            if (DCHUNK == 1 || d0 + k < dim) {
                                acc[j][k] = __dadd_rn(acc[j][k], p[k]);
                            }
                        }
                    }
                }
            }
        }
        // waves add their partial sums in wave order into the LDS accumulator; the last wave
        // finishes the values and writes them out
        for (uint32_t w = 0; w + 1 < kTileWaves; ++w) {
            if (wave == w) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int k = 0; k < DCHUNK; ++k) {
                        double* cell = sRed + (j * kWave + lane) * DCHUNK + k;
                        *cell = (w == 0) ? acc[j][k] : __dadd_rn(*cell, acc[j][k]);
                    }
                }
            }
            __syncthreads();
        }
        if (wave == kTileWaves - 1) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const size_t doc = block * kDocsPerBlock + j * kWave + lane;
#pragma unroll
                for (int k = 0; k < DCHUNK; ++k) {
                    if (doc < docCount && (DCHUNK == 1 || d0 + k < dim)) {
                        const double sum = __dadd_rn(sRed[(j * kWave + lane) * DCHUNK + k], acc[j][k]);
                        out[doc * dim + d0 + k] = Finish(sum, scale, bias[d0 + k], addBias);
                    }
                }
            }
        }
    }
}

// One-dimensional non-symmetric models without xor masks whose trees have at most kNsLdsEntries
// entries, whole model: as EvalNonSymmetricTileKernel, but a wave walks its trees out of a copy in
// its own LDS region (an LDS gather costs a fraction of a gather from global memory). Consecutive
// trees are grouped into units of up to kNsUnitTrees trees and ENTRIES entries; a wave takes
// a unit at a time and walks its trees side by side (4 documents x kNsUnitTrees chains per lane).
// A compact entry is one dword:
//   bits 0-7 splitIdx, bits 8-17 the 256-byte LDS row that holds the bucket's bins (so entry & 0x3ff00 is its
//   address), bits 21-31 index of the left child relative to the unit's first entry.
// Both addresses of a step take one instruction: the bin's is (entry & 0x3ff00) | lane offset, the pair's the
// funnel shift {wave, entry} >> 19, because wave w keeps its entries at LDS address w * 8 KB. Regions shorter than
// 8 KB leave gaps, and the rows of the bins fill them: NsLdsTileRow() says where bucket b goes, for the copy of
// the tile here and for the entries on the host.
// The kernel is bound by the latency of this chain of LDS reads, so the workgroup has as many waves as LDS has
// room for: WAVES regions of ENTRIES entries, ENTRIES at least the largest tree of the model
// (16 x 1024, 12 x 1536 or 8 x 2048).
// The two children of a node sit side by side at an even index (the root is entry 0, entry 1 is
// unused), so one 8-byte LDS read, issued together with the read of the node's bin, brings both
// and the compare only selects: one LDS round trip per level. A terminal entry points at its own
// pair and compares so that it selects itself (even index: splitIdx 255, false for every bin;
// odd index: splitIdx 0, true for every bin, which no real split has). The next unit's entries
// are fetched into registers while the current unit is walked: sixteen bytes per lane and whole rounds of
// the wave, with neither bounds nor branches - every unit starts at a multiple of four entries and `entries`
// ends with ENTRIES spare ones (a copy written with a test per round cost a taken branch each way per round,
// a tenth of the kernel's time). valuesByEntry holds the leaf value of every terminal entry, indexed like
// `entries`; a unit's values are requested behind its walk and added after the next unit's walk, two sets of
// registers taking turns.
// unitRows: 8 dwords per unit: first entry, height of the tallest tree, number of entries, first entry of the
// second tree relative to the unit's, that of the third tree | number of trees << 16, and the model's numbers
// of the three trees: a call for the trees [treeBegin, treeEnd) adds the values of those only and passes over
// the units that hold none of them.
// Models of several dimensions: a workgroup sums DIMS of them, those from blockIdx.y * DIMS on (every slice of
// the dimensions walks the trees again), and valuesByEntry is [slice][entryCount] rows of DIMS values (zeros past
// the last dimension), so that a leaf's values come with one aligned load; they are read and added right behind
// the unit's walk, with the other waves of the SIMD to cover the wait.
// grid = (doc blocks, ceil(dim / DIMS)), block = 64 * WAVES, dynamic LDS = NsLdsTileRows(buckets, WAVES, ENTRIES) * 256
// + 256 * 8 * DIMS bytes; no other LDS in the kernel.
constexpr int kNsLdsEntries = 2048;
constexpr int kNsUnitTrees = 3;

// The 256-byte LDS row of bucket b's bins: the 8 KB of a wave start with its entries (entries / 64 rows) and the
// rows that are left take bins; the other buckets follow the last wave's 8 KB.
__host__ __device__ constexpr uint32_t NsLdsTileRow(uint32_t bucket, uint32_t waves, uint32_t entries) {
    const uint32_t regionRows = entries / 64, gapRows = 32 - regionRows;
    const uint32_t divisor = gapRows ? gapRows : 1;  // regions of 8 KB leave no gap
    return bucket < gapRows * waves ? 32 * (bucket / divisor) + regionRows + bucket % divisor
                                    : 32 * waves + bucket - gapRows * waves;
}

// Rows of LDS up to the end of the bins
__host__ __device__ constexpr uint32_t NsLdsTileRows(uint32_t buckets, uint32_t waves, uint32_t entries) {
    const uint32_t gapRows = (32 - entries / 64) * waves;
    return 32 * waves + (buckets > gapRows ? buckets - gapRows : 0);
}

// A load of a scalar from an LDS address given as a number (the dynamic LDS of a kernel without other LDS
// starts at 0).
template <class T>
__device__ __forceinline__ T LdsLoad(uint32_t address) {
    return *reinterpret_cast<const __attribute__((address_space(3))) T*>(address);
}

__device__ __forceinline__ double LeafRowValue(const double2& row, int k) {
    return k == 0 ? row.x : row.y;
}

__device__ __forceinline__ double LeafRowValue(const double4& row, int k) {
    return k == 0 ? row.x : k == 1 ? row.y : k == 2 ? row.z : row.w;
}

template <int WAVES, int ENTRIES, int DIMS>
__global__ __launch_bounds__(64 * WAVES) void EvalNonSymmetricLdsKernel(
    const uint32_t* __restrict__ bins, size_t docCount, uint32_t bucketCount, const uint32_t* __restrict__ entries,
    const uint4* __restrict__ unitRows, uint32_t unitCount, const double* __restrict__ valuesByEntry,
    const double* __restrict__ bias, double scale, uint32_t dim, uint32_t entryCount, uint32_t treeBegin,
    uint32_t treeEnd, double* __restrict__ out) {
    constexpr int kFetch = ENTRIES / (4 * kWave);  // rounds of a wave's copy, sixteen bytes per lane
    static_assert(ENTRIES <= kNsLdsEntries && ENTRIES % (4 * kWave) == 0, "a region holds whole rounds of a wave's copy");
    extern __shared__ uint32_t sTile[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x;
    const uint32_t tileDwords = bucketCount * kWave;
    const uint32_t* src = bins + block * tileDwords;
    for (uint32_t i = tid; i < tileDwords; i += 64 * WAVES) {
        sTile[NsLdsTileRow(i / kWave, WAVES, ENTRIES) * kWave + (i & (kWave - 1))] = src[i];
    }
    const uint32_t laneOff = lane * 4;
    double* sRed = reinterpret_cast<double*>(sTile + NsLdsTileRows(bucketCount, WAVES, ENTRIES) * kWave);
    uint32_t* sEntries = sTile + wave * kNsLdsEntries;  // 8 KB per wave, the first ENTRIES * 4 bytes of them
    const uint32_t bucketMask = 0x3ff00u;
    __syncthreads();  // tile is loaded

    // A unit's entries come as whole rounds, whatever its size: a unit starts at a multiple of four entries and
    // the table ends with ENTRIES spare ones, so the copy needs neither a bound nor a branch (entries past the
    // unit's are never followed).
    using TEntries4 = uint32_t __attribute__((ext_vector_type(4)));
    TEntries4 fetched[kFetch];
#define CBAMD_STORE_UNIT()                                                                                  \
    do {                                                                                                    \
        _Pragma("unroll") for (int i = 0; i < kFetch; ++i) {                                                \
            reinterpret_cast<TEntries4*>(sEntries)[i * kWave + lane] = fetched[i];                          \
        }                                                                                                   \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                              \
        __builtin_amdgcn_wave_barrier();                                                                    \
    } while (0)
#define CBAMD_FETCH_UNIT(rowValue)                                                                          \
    do {                                                                                                    \
        const uint32_t fFirst = __builtin_amdgcn_readfirstlane((rowValue).x);                               \
        const TEntries4* fSource = reinterpret_cast<const TEntries4*>(entries + fFirst) + lane;             \
        _Pragma("unroll") for (int i = 0; i < kFetch; ++i) {                                                \
            fetched[i] = fSource[i * kWave];                                                                \
        }                                                                                                   \
    } while (0)

    double acc[4][DIMS];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int k = 0; k < DIMS; ++k) {
            acc[j][k] = 0.0;
        }
    }
    // one dimension: a unit's values are requested behind its walk and added behind the next unit's. Two sets
    // of them take turns (the loop below is written out for two units), so that the loads of one unit never
    // wait for registers that the sums of the unit before still read.
    double pending[2][kNsUnitTrees][4];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
        for (int g = 0; g < kNsUnitTrees; ++g) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                pending[p][g][j] = 0.0;
            }
        }
    }
    int lastSet = -1;  // the set whose values are not added yet
    const uint32_t d0 = blockIdx.y * DIMS;
    const double* sliceValues = valuesByEntry + static_cast<size_t>(blockIdx.y) * entryCount * DIMS;
    uint32_t u = wave;
    uint4 row = make_uint4(0, 0, 0, 0), row2 = make_uint4(0, 0, 0, 0);
    if (u < unitCount) {
        row = unitRows[2 * u];
        row2 = unitRows[2 * u + 1];
        CBAMD_FETCH_UNIT(row);
    }
    const auto walkUnit = [&](double (&mineSet)[kNsUnitTrees][4], const double (&otherSet)[kNsUnitTrees][4]) {
        const uint32_t first = __builtin_amdgcn_readfirstlane(row.x);
        const uint32_t height = __builtin_amdgcn_readfirstlane(row.y);
        const uint32_t packed = __builtin_amdgcn_readfirstlane(row2.x);
        const uint32_t trees = packed >> 16;
        // trees the unit does not have walk its first tree again; their values are not added
        const uint32_t start[kNsUnitTrees] = {0u, trees > 1 ? __builtin_amdgcn_readfirstlane(row.w) : 0u,
                                              trees > 2 ? (packed & 0xffffu) : 0u};
        const uint32_t treeOf[kNsUnitTrees] = {static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(row2.y)),
                                               static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(row2.z)),
                                               static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(row2.w))};
        bool wanted[kNsUnitTrees];
        bool anyWanted = false;
#pragma unroll
        for (int g = 0; g < kNsUnitTrees; ++g) {
            wanted[g] = static_cast<uint32_t>(g) < trees && treeOf[g] - treeBegin < treeEnd - treeBegin;
            anyWanted = anyWanted || wanted[g];
        }
        if (anyWanted) {
            // the previous unit's reads were issued before these stores and LDS serves one wave in order
            CBAMD_STORE_UNIT();
        }
        const uint32_t uNext = u + WAVES;
        uint4 rowNext = make_uint4(0, 0, 0, 0), row2Next = make_uint4(0, 0, 0, 0);
        if (uNext < unitCount) {
            rowNext = unitRows[2 * uNext];
            row2Next = unitRows[2 * uNext + 1];
            CBAMD_FETCH_UNIT(rowNext);
        }
        // The first step starts at the root for all four documents of a lane: one read of the children, one of the
        // four bins (a terminal root selects itself like any other terminal entry, so the step is safe for a tree
        // of one leaf).
        uint32_t entry[kNsUnitTrees][4];
#pragma unroll
        for (int g = 0; g < kNsUnitTrees; ++g) {
            const uint32_t rootEntry = anyWanted ? sEntries[start[g]] : 0u;
            if (anyWanted && height > 0) {
                const uint64_t pair = LdsLoad<uint64_t>(__builtin_amdgcn_alignbit(wave, rootEntry, 19));
                uint32_t binAddr;
                asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(binAddr) : "v"(rootEntry), "s"(bucketMask), "v"(laneOff));
                const uint32_t bins4 = LdsLoad<uint32_t>(binAddr);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    entry[g][j] = static_cast<uint32_t>(((bins4 >> (8 * j)) & 0xffu) >= (rootEntry & 0xffu) ? pair >> 32 : pair);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    entry[g][j] = rootEntry;
                }
            }
        }
        for (uint32_t step = 1; step < (anyWanted ? height : 0u); ++step) {
            uint64_t pair[kNsUnitTrees][4];  // the two children of a chain's node, left in the low half
            uint32_t bin[kNsUnitTrees][4];
#pragma unroll
            for (int g = 0; g < kNsUnitTrees; ++g) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t e = entry[g][j];
                    // bits 18-20 of an entry are clear: e >> 19 is the byte offset of the pair of children in
                    // the wave's region, whose number comes in from above (kNsLdsEntries * 4 = 1 << 13)
                    pair[g][j] = LdsLoad<uint64_t>(__builtin_amdgcn_alignbit(wave, e, 19));
                    uint32_t binAddr;
                    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(binAddr) : "v"(e), "s"(bucketMask), "v"(laneOff));
                    bin[g][j] = LdsLoad<uint8_t>(binAddr + j);
                }
            }
#pragma unroll
            for (int g = 0; g < kNsUnitTrees; ++g) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    entry[g][j] = static_cast<uint32_t>(bin[g][j] >= (entry[g][j] & 0xffu) ? pair[g][j] >> 32 : pair[g][j]);
                }
            }
        }
        uint32_t idx[kNsUnitTrees][4];
#pragma unroll
        for (int g = 0; g < kNsUnitTrees; ++g) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                idx[g][j] = (entry[g][j] >> 21) + ((entry[g][j] & 0xffu) == 0 ? 1u : 0u);
            }
        }
        if constexpr (DIMS == 1) {
#pragma unroll
            for (int g = 0; g < kNsUnitTrees; ++g) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[j][0] = __dadd_rn(acc[j][0], otherSet[g][j]);
                }
            }
#pragma unroll
            for (int g = 0; g < kNsUnitTrees; ++g) {
                if (wanted[g]) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        mineSet[g][j] = valuesByEntry[first + idx[g][j]];
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        mineSet[g][j] = 0.0;
                    }
                }
            }
        } else {
#pragma unroll
            for (int g = 0; g < kNsUnitTrees; ++g) {
                if (wanted[g]) {
                    using TLeafRow = typename std::conditional<DIMS == 2, double2, double4>::type;
                    TLeafRow value[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        value[j] = reinterpret_cast<const TLeafRow*>(sliceValues)[first + idx[g][j]];
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
#pragma unroll
                        for (int k = 0; k < DIMS; ++k) {
                            acc[j][k] = __dadd_rn(acc[j][k], LeafRowValue(value[j], k));
                        }
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        u = uNext;
        row = rowNext;
        row2 = row2Next;
    };
    while (u < unitCount) {
        walkUnit(pending[0], pending[1]);
        lastSet = 0;
        if (u >= unitCount) {
            break;
        }
        walkUnit(pending[1], pending[0]);
        lastSet = 1;
    }
#undef CBAMD_FETCH_UNIT
#undef CBAMD_STORE_UNIT
    if constexpr (DIMS == 1) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            if (lastSet == p) {
#pragma unroll
                for (int g = 0; g < kNsUnitTrees; ++g) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        acc[j][0] = __dadd_rn(acc[j][0], pending[p][g][j]);
                    }
                }
            }
        }
    }
    // waves add their partial sums in wave order into the LDS accumulator; the last wave
    // finishes the values and writes them out
    for (uint32_t w = 0; w + 1 < WAVES; ++w) {
        if (wave == w) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int k = 0; k < DIMS; ++k) {
                    double* cell = sRed + (k * 4 + j) * kWave + lane;
                    *cell = (w == 0) ? acc[j][k] : __dadd_rn(*cell, acc[j][k]);
                }
            }
        }
        __syncthreads();
    }
    if (wave == WAVES - 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const size_t doc = block * kDocsPerBlock + j * kWave + lane;
#pragma unroll
            for (int k = 0; k < DIMS; ++k) {
                if (doc < docCount && d0 + k < dim) {
                    out[doc * dim + d0 + k] =
                        Finish(__dadd_rn(sRed[(k * 4 + j) * kWave + lane], acc[j][k]), scale, bias[d0 + k], treeBegin == 0);
                }
            }
        }
    }
}

// Leaf indexes [doc][tree - treeBegin] for both tree kinds (CalcLeafIndexesGeneric,
// cpu/evaluator.h:174-253; non-symmetric numbering cpu/evaluator_impl.cpp:626-633).
__global__ __launch_bounds__(256) void LeafIndexesKernel(const uint8_t* __restrict__ bins, size_t docCount,
                                                         uint32_t bucketCount, TTreeTables tt, int oblivious,
                                                         uint32_t treeBegin, uint32_t treeEnd,
                                                         uint32_t* __restrict__ out) {
    const size_t doc = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (doc >= docCount) {
        return;
    }
    const size_t treeCount = treeEnd - treeBegin;
    for (uint32_t t = treeBegin; t < treeEnd; ++t) {
        uint32_t result;
        if (oblivious) {
            const uint32_t first = tt.TreeStart[t];
            const uint32_t depth = tt.TreeSize[t];
            uint32_t idx = 0;
            for (uint32_t d = 0; d < depth; ++d) {
                const uint32_t sp = tt.Splits[first + d];
                const uint32_t b = BinOfDoc(bins, doc, bucketCount, sp & 0xffffu);
                idx |= static_cast<uint32_t>((b ^ ((sp >> 16) & 0xffu)) >= (sp >> 24)) << d;
            }
            result = idx;
        } else {
            const uint32_t node = WalkNonSymmetric(bins, doc, bucketCount, tt, t);
            result = (tt.NodeToLeaf[node] - tt.FirstLeaf[t]) / static_cast<uint32_t>(tt.Dim);
        }
        out[doc * treeCount + (t - treeBegin)] = result;
    }
}

// Leaf indexes of oblivious trees of depth <= 8 whose 256-document tile of bins fits LDS: the byte-parallel walk of
// the tile kernel (four documents per lane, a tree per wave and turn), and rows of the output written whole. A
// workgroup of four waves takes a block of 256 documents and the trees in groups of 64: wave w walks trees
// 16 w .. 16 w + 15 of the group and leaves each tree's four index bytes per lane in LDS ([lane][tree], 65 dwords
// per lane); then wave j writes, document by document, the 64 indexes of documents 64 j .. 64 j + 63: one 256-byte
// store per document and group where the plain kernel stores four bytes per (document, tree) a row apart.
// packedTrees as in EvalObliviousTileKernel. grid = doc blocks, block = 256, dynamic LDS = buckets * 256 + 64 * 65 * 4.
constexpr int kLeafIndexGroup = 64;
constexpr int kLeafIndexPitch = kLeafIndexGroup + 1;

template <bool SEVEN_BIT>
__global__ __launch_bounds__(256) void LeafIndexesTileKernel(const uint32_t* __restrict__ bins, size_t docCount,
                                                             uint32_t bucketCount, const uint32_t* __restrict__ packedTrees,
                                                             uint32_t treeBegin, uint32_t treeEnd,
                                                             uint32_t* __restrict__ out) {
    extern __shared__ uint32_t sTile[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const size_t block = blockIdx.x;
    const uint32_t tileDwords = bucketCount * kWave;
    const uint32_t* src = bins + block * tileDwords;
    for (uint32_t i = tid; i < tileDwords; i += 256) {
        sTile[i] = src[i];
    }
    uint32_t* stage = sTile + tileDwords;
    const uint8_t* laneTile = reinterpret_cast<const uint8_t*>(sTile) + lane * 4;
    const uint32_t slot = lane & (kPackedTreeDwords - 1);
    const size_t treeCount = treeEnd - treeBegin;
    const size_t firstDoc = block * kDocsPerBlock + wave * kWave;  // of the 64 documents this wave writes
    for (uint32_t group = treeBegin; group < treeEnd; group += kLeafIndexGroup) {
        __syncthreads();  // the tile is loaded; the previous group's indexes are written
        constexpr int kPerWave = kLeafIndexGroup / 4;
#pragma unroll 4
        for (int k = 0; k < kPerWave; ++k) {
            const uint32_t t = group + wave * kPerWave + k;
            if (t < treeEnd) {
                const uint32_t row = packedTrees[static_cast<size_t>(t) * kPackedTreeDwords + slot];
                stage[lane * kLeafIndexPitch + wave * kPerWave + k] = TreeIndexes<SEVEN_BIT, 8>(laneTile, row);
            }
        }
        __syncthreads();
        const uint32_t tree = group + lane;
        for (uint32_t d = 0; d < kWave; ++d) {
            const size_t doc = firstDoc + d;
            if (doc < docCount && tree < treeEnd) {
                out[doc * treeCount + (tree - treeBegin)] = (stage[d * kLeafIndexPitch + lane] >> (8 * wave)) & 0xffu;
            }
        }
    }
}

// Re-lays bins out as the reference does: blocks of 128 documents, [block][bucket][doc in block],
// the last block packed with its own document count (cpu/quantization.h:357-365).
__global__ __launch_bounds__(256) void ExportBinsKernel(const uint8_t* __restrict__ bins, size_t docCount,
                                                        uint32_t bucketCount, uint8_t* __restrict__ out) {
    const size_t doc = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (doc >= docCount) {
        return;
    }
    const size_t refBlockStart = doc / 128 * 128;
    const size_t inBlock = doc - refBlockStart;
    const size_t blockDocs = min(static_cast<size_t>(128), docCount - refBlockStart);
    for (uint32_t b = 0; b < bucketCount; ++b) {
        out[refBlockStart * bucketCount + b * blockDocs + inBlock] = BinOfDoc(bins, doc, bucketCount, b);
    }
}

// ---- prediction types on the device --------------------------------------------------------
// TEvalResultProcessor::PostprocessBlock (catboost/libs/model/eval_processing.h:174-240) over blocks of
// min(128, total documents) documents, with the reference's exponent (fmath::expd_v / fmath::expd,
// contrib/libs/fmath/fmath.hpp:474-512, 565-648). The library is compiled without contraction, so each
// operation rounds on its own like the CPU's.

struct TFastExpDev {
    const unsigned long long* Mantissa;  // 2048 mantissas of 2^(i / 2048)
    double Scale, InvScale;              // 2048 / ln 2 and its reciprocal
};

// the arithmetic both forms share; `indexBits`: table index in bits 0..10, binary exponent above
__device__ __forceinline__ double FastExpCore(const TFastExpDev& c, double x, double rounded, unsigned long long indexBits) {
    constexpr int kTableBits = 11;
    const double kMagic = static_cast<double>(3ull << 51);
    constexpr unsigned long long kAdjust = (1ull << (kTableBits + 10)) - (1ull << kTableBits);
    const unsigned long long mantissa = c.Mantissa[indexBits & ((1u << kTableBits) - 1)];
    const unsigned long long power = (((indexBits + kAdjust) >> kTableBits) << 52) | mantissa;
    double t = rounded - kMagic;
    t = t * c.InvScale;
    t = t - x;
    double y = 3.0000000027955394 - t;
    y = y * (t * t);
    y = y * 0.16666666685227835064;
    y = y - t;
    y = y + 1.0;
    return y * __longlong_as_double(static_cast<long long>(power));
}

// element `index` of a run of `count` values handed to the exponent at once: the first count & ~3 take
// the vector form (clamped argument, NaN -> upper clamp), the rest the scalar form (0 / +inf outside)
__device__ __forceinline__ double FastExpAt(const TFastExpDev& c, double v, size_t index, size_t count) {
    const double kMagic = static_cast<double>(3ull << 51);
    if (index < (count & ~size_t(3))) {
        v = v < 709.78272569338397 ? v : 709.78272569338397;
        v = v > -708.39641853226408 ? v : -708.39641853226408;
        double d = v * c.Scale;
        d = d + kMagic;
        return FastExpCore(c, v, d, static_cast<unsigned long long>(__double_as_longlong(d)));
    }
    if (v <= -708.39641853226408) {
        return 0.0;
    }
    if (v >= 709.78271289338397) {
        return __longlong_as_double(0x7ff0000000000000ll);
    }
    double d = v * c.Scale;
    d = d + kMagic;
    const long long low = static_cast<long long>(static_cast<int>(static_cast<unsigned int>(__double_as_longlong(d))));
    return FastExpCore(c, v, d, static_cast<unsigned long long>(low));
}

constexpr int kPredRaw = 0, kPredExponent = 1, kPredRmseWithUncertainty = 2, kPredProbability = 3, kPredClass = 4,
              kPredMultiProbability = 5;  // EApiPredictionType, catboost/libs/model_interface/c_api.h:50-57

// One thread per document of a chunk that starts at document `firstDoc` of `totalDocs`.
// raw[doc * dim + k] -> out (doc values for Class, doc * dim values otherwise). raw == out is allowed
// except for Class with dim > 1.
__global__ __launch_bounds__(256) void ApplyPredictionTypeKernel(int type, uint32_t dim, size_t firstDoc,
                                                                 size_t totalDocs, size_t docCount, TFastExpDev c,
                                                                 const double* raw, double* out) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= docCount) {
        return;
    }
    const size_t doc = firstDoc + i;
    const size_t blockSize = totalDocs < 128 ? totalDocs : 128;
    const size_t inBlock = doc % blockSize;
    const size_t blockDocs = min(blockSize, totalDocs - (doc - inBlock));  // documents of this document's block
    const double* r = raw + i * dim;
    if (type == kPredClass) {
        if (dim == 1) {
            out[i] = r[0] > 0.0 ? 1.0 : 0.0;
        } else {
            uint32_t best = 0;
            double top = r[0];
            for (uint32_t k = 1; k < dim; ++k) {
                const double v = r[k];
                if (top < v) {  // std::max_element: the first largest
                    top = v;
                    best = k;
                }
            }
            out[i] = static_cast<double>(best);
        }
        return;
    }
    double* o = out + i * dim;
    if (dim == 1) {
        const double v = r[0];
        if (type == kPredProbability) {
            o[0] = 1. / (1. + FastExpAt(c, -v, inBlock, blockDocs));
        } else if (type == kPredExponent) {
            o[0] = FastExpAt(c, v, inBlock, blockDocs);
        } else {
            o[0] = v;
        }
        return;
    }
    if (type == kPredRmseWithUncertainty) {
        for (uint32_t k = 0; k < dim; ++k) {
            double v = r[k];
            if (k == 1) {
                v = FastExpAt(c, v * 2.0, 0, 1);
            }
            o[k] = v;
        }
    } else if (type == kPredProbability) {  // CalcSoftmax, eval_processing.h:15-27
        double top = r[0];
        for (uint32_t k = 1; k < dim; ++k) {
            const double v = r[k];
            top = top < v ? v : top;
        }
        double sum = 0;
        for (uint32_t k = 0; k < dim; ++k) {
            const double e = FastExpAt(c, r[k] - top, k, dim);
            o[k] = e;
            sum += e;
        }
        for (uint32_t k = 0; k < dim; ++k) {
            o[k] = o[k] / sum;
        }
    } else if (type == kPredMultiProbability) {
        for (uint32_t k = 0; k < dim; ++k) {
            o[k] = 1. / (1. + FastExpAt(c, -r[k], inBlock * dim + k, blockDocs * dim));
        }
    } else {
        for (uint32_t k = 0; k < dim; ++k) {
            o[k] = r[k];
        }
    }
}

__global__ void FillBiasKernel(double* __restrict__ out, size_t count, const double* __restrict__ bias, int dim) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) {
        out[i] = bias[i % dim];
    }
}

// Clears `dwords` 32-bit words. A kernel rather than hipMemsetAsync, so that callers may capture the
// launch into a HIP graph.
__global__ void FillZeroKernel(uint32_t* __restrict__ out, size_t dwords) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < dwords; i += stride) {
        out[i] = 0;
    }
}

}  // namespace cbamd::dev
