// Host side of the HIP evaluator: model upload, kernel launches, host staging.
#include "hip_evaluator.h"
#include "fast_exp.h"
#include "kernels.hip.h"

#include <algorithm>
#include <cmath>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <string>
#include <thread>
#include <tuple>
#include <vector>

// Bin buffer of the entry point that allocates nothing (THipEvaluator::CalcDeviceNoAlloc): every GPU the
// library runs on holds one copy of this array, at its own address, until the process ends. In host code
// the name is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
static __device__ __align__(256) unsigned char scratch[cbamd::THipEvaluator::kNoAllocScratchBytes];

namespace cbamd {

namespace {

void HipCheck(hipError_t e, const char* what) {
    if (e != hipSuccess) {
        throw TModelError(std::string("HIP error in ") + what + ": " + hipGetErrorString(e));
    }
}
#define HIP_CHECK(expr) HipCheck((expr), #expr)

template <typename T>
class TDeviceVec {
public:
    TDeviceVec() = default;
    ~TDeviceVec() { Reset(); }
    TDeviceVec(const TDeviceVec&) = delete;
    TDeviceVec& operator=(const TDeviceVec&) = delete;

    void Reset() {
        if (Ptr) {
            (void)hipFree(Ptr);
            Ptr = nullptr;
            Cap = 0;
        }
    }
    void Upload(const std::vector<T>& host) {
        Reserve(std::max<size_t>(host.size(), 1));
        if (!host.empty()) {
            HIP_CHECK(hipMemcpy(Ptr, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
        }
    }
    // grow-only
    void Reserve(size_t count) {
        if (count > Cap) {
            Reset();
            HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&Ptr), count * sizeof(T)));
            Cap = count;
        }
    }
    T* Get() const { return Ptr; }
    size_t Capacity() const { return Cap; }

private:
    T* Ptr = nullptr;
    size_t Cap = 0;
};

template <typename T>
class TPinnedVec {
public:
    ~TPinnedVec() { Reset(); }
    void Reset() {
        if (Ptr) {
            (void)hipHostFree(Ptr);
            Ptr = nullptr;
            Cap = 0;
        }
    }
    void Reserve(size_t count) {
        if (count > Cap) {
            Reset();
            HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&Ptr), count * sizeof(T), hipHostMallocDefault));
            Cap = count;
        }
    }
    T* Get() const { return Ptr; }

private:
    T* Ptr = nullptr;
    size_t Cap = 0;
};

// A kernel that uses more than 64 KB of dynamic LDS has to be told so once (per device); the largest size asked
// for so far is remembered, so that the attribute is not set again on every launch.
// The code object of the assembly kernels, loaded once per device and kept for the life of the process: every
// evaluator of a device shares it (a few megabytes of code and some milliseconds of loading otherwise per model).
hipModule_t SharedRegModule(const void* image) {
    static std::mutex lock;
    static std::vector<std::pair<int, hipModule_t>> loaded;
    int device = 0;
    HIP_CHECK(hipGetDevice(&device));
    std::lock_guard<std::mutex> guard(lock);
    for (const auto& item : loaded) {
        if (item.first == device) {
            return item.second;
        }
    }
    hipModule_t module = nullptr;
    HIP_CHECK(hipModuleLoadData(&module, image));
    loaded.emplace_back(device, module);
    return module;
}

void EnsureDynamicLds(const void* kernel, size_t bytes) {
    if (bytes <= 64 * 1024) {
        return;
    }
    static std::mutex lock;
    static std::vector<std::pair<std::pair<int, const void*>, size_t>> granted;
    int device = 0;
    HIP_CHECK(hipGetDevice(&device));
    std::lock_guard<std::mutex> guard(lock);
    for (auto& item : granted) {
        if (item.first.first == device && item.first.second == kernel) {
            if (item.second >= bytes) {
                return;
            }
            HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
            item.second = bytes;
            return;
        }
    }
    HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    granted.push_back({{device, kernel}, bytes});
}

// Address of `scratch` on a device, asked for once per device, with that device current.
uint8_t* NoAllocScratchOfCurrentDevice(int deviceId) {
    static std::mutex lock;
    static std::vector<uint8_t*> perDevice;
    std::lock_guard<std::mutex> guard(lock);
    if (perDevice.size() <= static_cast<size_t>(deviceId)) {
        perDevice.resize(static_cast<size_t>(deviceId) + 1, nullptr);
    }
    if (perDevice[deviceId] == nullptr) {
        void* ptr = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        CBAMD_ENSURE(ptr != nullptr, "the device holds no copy of the no-allocation bin buffer");
        perDevice[deviceId] = static_cast<uint8_t*>(ptr);
    }
    return perDevice[deviceId];
}

// Code object of the register-resident evaluate kernels (assembled from the output of
// gen_eval_reg_kernel.py at build time).
alignas(4096) const unsigned char kEvalRegCodeObject[] = {
#include "eval_reg_kernel_co.inc"
};

// Must match gen_eval_reg_kernel.py: kernel arguments, variants, trees per LDS buffer.
struct TEvalRegArgs {
    const void* Bins;
    const void* Rows;
    const void* Leaves;
    void* Out;
    uint32_t DocCount;
    uint32_t BlockCount;
    uint32_t TreeBlocks;
    uint32_t Flags;
    double Scale;
    const double* Bias;
    uint32_t BucketCount;
    uint32_t Dim;
    uint32_t FirstDim;
    uint32_t StoreDims;
};
static_assert(sizeof(TEvalRegArgs) == 80, "kernel argument block shared by the register-resident and the fused kernels");

struct TEvalRegLaunchArgs {
    TEvalRegArgs Reg;
    uint32_t TreeBlocksPerSlice;  // grid.y slices of the trees; one slice: all tree blocks
    uint32_t Padding;
    const uint32_t* RegMap;       // read when Reg.Flags has kRegFlagMapped: where each bins register comes from
};
static_assert(sizeof(TEvalRegLaunchArgs) == 96, "kernel argument block of the register-resident kernels");
constexpr uint32_t kRegFlagMapped = 8;
// what a mapped bins register holds of its bucket's bins (bits 16.. of a map entry)
constexpr uint32_t kRegMapAsIs = 0, kRegMapLow = 1, kRegMapHigh = 2;  // bin, min(bin, 127), max(bin - 127, 0)

struct TEvalRegVariant {
    uint32_t Buckets;
    uint32_t Waves;
    uint32_t Pitch;   // dimensions per launch = doubles per leaf row
    uint32_t Leaves;  // leaf rows per tree (64: trees of depth <= 6)
    bool Mixed;       // 32-dword level tables, compare form chosen per tree
    bool Six;         // every bin below 64: even levels compare into bit 6, two levels share a merge
    const char* Name;
};
constexpr TEvalRegVariant kEvalRegVariants[] = {
    {96, 8, 1, 256, false, false, "cbamd_eval_reg_b96_w8_p1_l256"},
    {96, 8, 1, 64, false, false, "cbamd_eval_reg_b96_w8_p1_l64"},
    {200, 4, 1, 256, false, false, "cbamd_eval_reg_b200_w4_p1_l256"},
    {208, 4, 1, 256, false, false, "cbamd_eval_reg_b208_w4_p1_l256"},
    {224, 4, 1, 256, false, false, "cbamd_eval_reg_b224_w4_p1_l256"},
    {192, 4, 2, 64, false, false, "cbamd_eval_reg_b192_w4_p2_l64"},
    {160, 4, 4, 64, false, false, "cbamd_eval_reg_b160_w4_p4_l64"},
    {128, 4, 6, 64, false, false, "cbamd_eval_reg_b128_w4_p6_l64"},
    {192, 4, 2, 256, false, false, "cbamd_eval_reg_b192_w4_p2_l256"},
    {160, 4, 4, 256, false, false, "cbamd_eval_reg_b160_w4_p4_l256"},
    {128, 4, 6, 256, false, false, "cbamd_eval_reg_b128_w4_p6_l256"},
    {96, 8, 1, 256, true, false, "cbamd_eval_reg_b96_w8_p1_l256_m"},
    {96, 8, 1, 64, true, false, "cbamd_eval_reg_b96_w8_p1_l64_m"},
    {200, 4, 1, 256, true, false, "cbamd_eval_reg_b200_w4_p1_l256_m"},
    {208, 4, 1, 256, true, false, "cbamd_eval_reg_b208_w4_p1_l256_m"},
    {224, 4, 1, 256, true, false, "cbamd_eval_reg_b224_w4_p1_l256_m"},
    {192, 4, 2, 64, true, false, "cbamd_eval_reg_b192_w4_p2_l64_m"},
    {160, 4, 4, 64, true, false, "cbamd_eval_reg_b160_w4_p4_l64_m"},
    {128, 4, 6, 64, true, false, "cbamd_eval_reg_b128_w4_p6_l64_m"},
    {192, 4, 2, 256, true, false, "cbamd_eval_reg_b192_w4_p2_l256_m"},
    {160, 4, 4, 256, true, false, "cbamd_eval_reg_b160_w4_p4_l256_m"},
    {128, 4, 6, 256, true, false, "cbamd_eval_reg_b128_w4_p6_l256_m"},
    {96, 8, 1, 256, false, true, "cbamd_eval_reg_b96_w8_p1_l256_s"},
    {96, 8, 1, 64, false, true, "cbamd_eval_reg_b96_w8_p1_l64_s"},
    {200, 4, 1, 256, false, true, "cbamd_eval_reg_b200_w4_p1_l256_s"},
    {208, 4, 1, 256, false, true, "cbamd_eval_reg_b208_w4_p1_l256_s"},
    {224, 4, 1, 256, false, true, "cbamd_eval_reg_b224_w4_p1_l256_s"},
    {192, 4, 2, 64, false, true, "cbamd_eval_reg_b192_w4_p2_l64_s"},
    {160, 4, 4, 64, false, true, "cbamd_eval_reg_b160_w4_p4_l64_s"},
    {128, 4, 6, 64, false, true, "cbamd_eval_reg_b128_w4_p6_l64_s"},
    {192, 4, 2, 256, false, true, "cbamd_eval_reg_b192_w4_p2_l256_s"},
    {160, 4, 4, 256, false, true, "cbamd_eval_reg_b160_w4_p4_l256_s"},
    {128, 4, 6, 256, false, true, "cbamd_eval_reg_b128_w4_p6_l256_s"},
    // trees of depth 9 and 10 (one dimension, 1024 leaf rows; gen_eval_reg_kernel.py's DEEP_SHAPES)
    {96, 8, 1, 1024, false, false, "cbamd_eval_reg_b96_w8_p1_l1024"},
    {208, 4, 1, 1024, false, false, "cbamd_eval_reg_b208_w4_p1_l1024"},
    {96, 8, 1, 1024, false, true, "cbamd_eval_reg_b96_w8_p1_l1024_s"},
    {208, 4, 1, 1024, false, true, "cbamd_eval_reg_b208_w4_p1_l1024_s"},
};
constexpr int kRegMaxDepth = 10;  // deepest tree of the register kernels (one-dimensional models; 8 otherwise)

// Fused kernels (binarize + evaluate in one launch, bins only ever in registers): shapes of
// gen_eval_reg_kernel.py's FUSED_SHAPES, each in a plain and a six-bit form, and each of these in a form that
// walks six levels instead of eight (models of depth <= 6), listed before the eight-level form of its shape.
struct TFusedVariant {
    uint32_t Buckets;  // bins registers = 16 per unit of sixteen columns
    uint32_t Waves;
    bool Six;
    uint32_t Levels;
    const char* Name;
};
constexpr TFusedVariant kFusedVariants[] = {
    {64, 8, false, 6, "cbamd_fused_b64_w8_d6"},
    {64, 8, true, 6, "cbamd_fused_b64_w8_d6_s"},
    {64, 8, false, 8, "cbamd_fused_b64_w8"},
    {64, 8, true, 8, "cbamd_fused_b64_w8_s"},
    {80, 8, false, 6, "cbamd_fused_b80_w8_d6"},
    {80, 8, true, 6, "cbamd_fused_b80_w8_d6_s"},
    {80, 8, false, 8, "cbamd_fused_b80_w8"},
    {80, 8, true, 8, "cbamd_fused_b80_w8_s"},
    {208, 4, false, 6, "cbamd_fused_b208_w4_d6"},
    {208, 4, true, 6, "cbamd_fused_b208_w4_d6_s"},
    {208, 4, false, 8, "cbamd_fused_b208_w4"},
    {208, 4, true, 8, "cbamd_fused_b208_w4_s"},
};
constexpr uint32_t kFusedUnitColumns = 16;
constexpr uint32_t kFusedUnitDwords = 40;   // sixteen lo, sixteen scale, flags, padding
constexpr uint32_t kFusedMaxSteps = 4;
constexpr size_t kFusedImageBytes = 32 * 1024;
constexpr size_t kFusedLutOffset = 16 * 1024;

struct TEvalFusedArgs {
    TEvalRegArgs Reg;       // Bins unused; Leaves: the border table images, then the leaf table
    const void* Floats;
    const void* Units;
    uint32_t StrideBytes;
    uint32_t UnitCount;
};
static_assert(sizeof(TEvalFusedArgs) == 104, "kernel argument block of the fused kernels");

// Trees of a slice of a small batch: two of the kernels' tree blocks, and not fewer than 32 trees (kernels with
// large leaf tables have blocks of 2 or 4 trees, and a slice costs a partial sum per document)
uint32_t RegSliceTrees(uint32_t treeBlock) {
    return std::max(2 * treeBlock, 32u);
}

// trees per LDS buffer of a variant: a power of two, at most 16, buffer at most 32 KB
uint32_t RegTreeBlock(const TEvalRegVariant& v) {
    uint32_t block = 16;
    while (block > 1 && block * v.Leaves * v.Pitch * 8 > 32 * 1024) {
        block /= 2;
    }
    return block;
}

// The variant for a model: one-dimensional models take the smallest register file that holds
// their buckets; others the pitch that needs the fewest launches (then the smallest such pitch).
// mixed: the model has one-hot splits or bins above 127.
const TEvalRegVariant* PickRegVariant(uint32_t buckets, uint32_t dim, uint32_t maxDepth, bool mixed, bool six,
                                      uint32_t minVariantBuckets = 0) {
    const TEvalRegVariant* best = nullptr;
    uint32_t bestLaunches = 0;
    // A model of several dimensions with more buckets than the kernels of two and more dimensions hold (they
    // need registers for their sums) takes the one-dimensional kernels, a launch per dimension: every launch
    // walks the trees again, which still is several times faster than leaving the registers.
    for (int onePerLaunch = 0; onePerLaunch < 2 && !best; ++onePerLaunch) {
        if (onePerLaunch && dim == 1) {
            break;
        }
        for (const auto& v : kEvalRegVariants) {
            // trees of depth <= 6: 64 leaf rows and six levels. One-dimensional models only on the 96-register
            // shape: wider ones keep the eight-level kernels, whose fused forms they can take
            const bool shallow = maxDepth <= 6 && !onePerLaunch && (dim > 1 || (buckets <= 96 && minVariantBuckets <= 96));
            const uint32_t leaves = maxDepth > 8 ? 1024u : shallow ? 64u : 256u;
            if (buckets > v.Buckets || v.Buckets < minVariantBuckets || (dim == 1 || onePerLaunch) != (v.Pitch == 1) ||
                v.Leaves != leaves || v.Mixed != mixed || v.Six != six) {
                continue;
            }
            const uint32_t launches = (dim + v.Pitch - 1) / v.Pitch;
            if (!best || launches < bestLaunches || (launches == bestLaunches && dim > 1 && v.Pitch < best->Pitch)) {
                best = &v;
                bestLaunches = launches;
            }
        }
    }
    return best;
}

// Diagnostic switches, read from the environment when an evaluator is built (cb_hip_evaluator.h lists them) and
// only in a process that sets CATBOOST_AMD_TEST_SWITCHES=1: a production process that happens to have one of the
// names in its environment keeps the default kernels. They choose between kernels that give the same results;
// tests use them to reach every kernel with one model.
struct TKernelSwitches {
    bool RegKernel = true;        // CATBOOST_AMD_REG_KERNEL=0: no register-resident assembly kernels
    bool RegSix = true;           // CATBOOST_AMD_REG_SIX=0: no six-bit form of those kernels, nor of the pair-tile kernel
    bool CtrTile = true;          // CATBOOST_AMD_CTR_TILE=0: the plain CTR kernel instead of the tile kernel
    uint32_t RegMinBuckets = 0;   // CATBOOST_AMD_REG_MIN_BUCKETS=n: only register kernels that hold n buckets or more
    bool Fused = true;            // CATBOOST_AMD_FUSED=0: binarize and evaluate always as two launches
    bool SmallBatch = true;       // CATBOOST_AMD_SMALL_BATCH=0: small batches are not spread over slices of the trees
    bool LevelOrder = true;       // CATBOOST_AMD_LEVEL_ORDER=0: register kernels keep the model's order of a tree's levels
    bool PairTile = true;         // CATBOOST_AMD_PAIR_TILE=0: the half-tile kernel with one tree per wave
    bool RowTile = true;          // CATBOOST_AMD_ROW_TILE=0: the tile kernel that broadcasts a tree's levels from a lane
    bool RegSplit = true;         // CATBOOST_AMD_REG_SPLIT=0: buckets of more than 127 values send a model to the mixed kernels
    uint32_t NsWaves = 0;         // CATBOOST_AMD_NS_WAVES=4|6|8|12|16: that shape of the non-symmetric LDS kernel or none

    static TKernelSwitches FromEnvironment() {
        const auto off = [](const char* name) {
            const char* v = std::getenv(name);
            return v != nullptr && v[0] == '0';
        };
        TKernelSwitches k;
        const char* gate = std::getenv("CATBOOST_AMD_TEST_SWITCHES");
        if (gate == nullptr || gate[0] != '1') {
            return k;
        }
        k.RegKernel = !off("CATBOOST_AMD_REG_KERNEL");
        k.RegSix = !off("CATBOOST_AMD_REG_SIX");
        k.CtrTile = !off("CATBOOST_AMD_CTR_TILE");
        k.Fused = !off("CATBOOST_AMD_FUSED");
        k.LevelOrder = !off("CATBOOST_AMD_LEVEL_ORDER");
        k.SmallBatch = !off("CATBOOST_AMD_SMALL_BATCH");
        k.PairTile = !off("CATBOOST_AMD_PAIR_TILE");
        k.RowTile = !off("CATBOOST_AMD_ROW_TILE");
        k.RegSplit = !off("CATBOOST_AMD_REG_SPLIT");
        if (const char* v = std::getenv("CATBOOST_AMD_NS_WAVES")) {
            k.NsWaves = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
        }
        if (const char* v = std::getenv("CATBOOST_AMD_REG_MIN_BUCKETS")) {
            k.RegMinBuckets = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
        }
        return k;
    }
};

// log2 of the LDS slots per bucket of the row binarize kernel: the smallest count that still
// exceeds the largest bucket of the model
int BinarizeLog2Slots(uint32_t maxBucketValues) {
    return maxBucketValues < 32 ? 5 : maxBucketValues < 64 ? 6 : maxBucketValues < 128 ? 7 : 8;
}

// Host twin of dev::GridCell: the same two roundings and the same truncation.
uint32_t GridCell(float v, float lo, float scale) {
    volatile float d = v - lo;
    volatile float t = d * scale;
    const float tt = t;
    if (!(tt > 0.0f)) {
        return 0;
    }
    if (tt >= 4294967296.0f) {
        return dev::kLutCells - 1;
    }
    return std::min<uint32_t>(static_cast<uint32_t>(tt), dev::kLutCells - 1);
}

// The uniform grid over a float bucket's sorted borders that starts the border search: lowest border,
// cells per unit, the search steps that cover the tallest cell, and per cell the number of borders in
// lower cells (what a search in that cell may skip).
struct TBucketGrid {
    float Lo = 0.0f;
    float Scale = 0.0f;
    uint32_t Steps = 0;
    uint32_t Start[dev::kLutCells] = {};
};

TBucketGrid MakeBucketGrid(const std::vector<float>& borders) {
    TBucketGrid g;
    if (borders.empty()) {
        return g;
    }
    g.Lo = borders.front();
    const float span = borders.back() - g.Lo;
    if (std::isfinite(g.Lo) && std::isfinite(span) && span > 0.0f) {
        g.Scale = static_cast<float>(dev::kLutCells) / span;
        if (!std::isfinite(g.Scale)) {
            g.Scale = 0.0f;
        }
    } else {
        g.Lo = 0.0f;
    }
    uint32_t population[dev::kLutCells] = {};
    for (float x : borders) {
        ++population[GridCell(x, g.Lo, g.Scale)];
    }
    const uint32_t tallest = *std::max_element(population, population + dev::kLutCells);
    while ((1u << g.Steps) - 1 < tallest) {
        ++g.Steps;
    }
    uint32_t start = 0;
    for (int c = 0; c < dev::kLutCells; ++c) {
        g.Start[c] = start;
        start += population[c];
    }
    return g;
}

constexpr size_t kMaxTileLdsBytes = 160 * 1024;

// LDS of the tile kernel without leaf regions: the bins of 256 documents and the accumulator
size_t TileLdsBytes(uint32_t buckets, int dchunk) {
    return ((static_cast<size_t>(buckets) * dev::kDocsPerBlock + 7) & ~size_t(7)) +
           static_cast<size_t>(dev::kDocsPerBlock) * dchunk * sizeof(double);
}

// LDS of EvalNonSymmetricLdsKernel: 8 KB per wave (its entries, then rows of bins), the other rows of bins, the
// accumulator
size_t NsLdsKernelBytes(uint32_t buckets, uint32_t waves, uint32_t entries, uint32_t dims) {
    return static_cast<size_t>(dev::NsLdsTileRows(buckets, waves, entries)) * 256 + dev::kDocsPerBlock * sizeof(double) * dims;
}

// The shapes of EvalNonSymmetricLdsKernel, most waves first
// dimensions that one workgroup of EvalNonSymmetricLdsKernel sums (a model of more walks its trees once per slice)
uint32_t NsLdsDims(int dim) {
    return dim == 1 ? 1 : dim == 2 ? 2 : 4;
}

struct TNsLdsShape {
    uint32_t Waves;
    uint32_t Entries;
    double Speed;  // steps of a unit per unit of time, relative to the 8-wave shape
};
constexpr TNsLdsShape kNsLdsShapes[] = {{16, 1024, 1.45}, {12, 1536, 1.26}, {8, 2048, 1.0}, {6, 2048, 0.8}, {4, 2048, 0.55}};

// A unit of EvalNonSymmetricLdsKernel: up to three trees that a wave walks side by side out of its LDS region
struct TNsUnit {
    uint32_t Trees[dev::kNsUnitTrees];
    uint32_t TreeCount;
    uint32_t Entries;
    uint32_t Height;
};

// Groups the trees (rows: first entry, height, entry count, unused) into units of at most `limit` entries.
// A unit takes as many steps as its tallest tree, so the trees go in by falling height, and every tree joins
// the fullest of the recently opened units that still has room for it (trees need not be neighbours in the
// model: the kernel's sums are partial sums per wave anyway). False when a tree exceeds the limit.
bool PackNsUnits(const std::vector<uint32_t>& rows, size_t treeCount, uint32_t limit, std::vector<TNsUnit>* units) {
    std::vector<uint32_t> order(treeCount);
    for (size_t t = 0; t < treeCount; ++t) {
        if (rows[t * 4 + 2] > limit) {
            return false;
        }
        order[t] = static_cast<uint32_t>(t);
    }
    std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) {
        return rows[a * 4 + 1] != rows[b * 4 + 1] ? rows[a * 4 + 1] > rows[b * 4 + 1] : rows[a * 4 + 2] > rows[b * 4 + 2];
    });
    constexpr size_t kWindow = 64;  // open units looked at per tree
    std::vector<size_t> open;
    for (const uint32_t t : order) {
        const uint32_t size = rows[t * 4 + 2];
        size_t best = open.size();
        for (size_t i = open.size() > kWindow ? open.size() - kWindow : 0; i < open.size(); ++i) {
            const TNsUnit& unit = (*units)[open[i]];
            if (unit.Entries + size <= limit && (best == open.size() || unit.Entries > (*units)[open[best]].Entries)) {
                best = i;
            }
        }
        if (best == open.size()) {
            TNsUnit unit{};
            unit.Height = rows[t * 4 + 1];
            units->push_back(unit);
            open.push_back(units->size() - 1);
        }
        TNsUnit& unit = (*units)[open[best]];
        unit.Trees[unit.TreeCount++] = t;
        unit.Entries += size;
        if (unit.TreeCount == static_cast<uint32_t>(dev::kNsUnitTrees)) {
            open.erase(open.begin() + static_cast<std::ptrdiff_t>(best));
        }
    }
    return true;
}

// Dimensions that a workgroup of the row-tile kernel sums at a time. Two: the sums, the values in flight and three
// trees' worth of values fetched ahead then fit a wave's registers at sixteen waves. A walk for four dimensions takes
// 1.8 times as long (C3's trees over 300 features: 3.6 against 2.06 ms), so only models of three or four dimensions
// with 64 leaves per tree take it, for one walk instead of two.
uint32_t RowTileDims(uint32_t maxDepth, int dim) {
    return dim == 1 ? 1 : maxDepth <= 6 && (dim == 3 || dim == 4) ? 4 : 2;
}

// LDS of the row-tile kernel: 256 documents' bins, the accumulator, a tree's leaf values per wave
size_t RowTileLdsBytes(uint32_t buckets, uint32_t maxDepth, uint32_t dims, uint32_t waves) {
    const size_t leaves = maxDepth <= 6 ? 64 : 256;
    return ((static_cast<size_t>(buckets) * 256 + 15) & ~size_t(15)) + dev::kDocsPerBlock * dims * sizeof(double) +
           static_cast<size_t>(waves) * leaves * dims * sizeof(double);
}

// Waves per workgroup of the row-tile kernel: eight when two workgroups then share a CU, else sixteen if LDS
// has room for their regions, else eight; 0 when the tile leaves no room for eight regions.
uint32_t RowTileWaves(uint32_t buckets, uint32_t maxDepth, int dim) {
    const uint32_t dims = RowTileDims(maxDepth, dim);
    if (2 * RowTileLdsBytes(buckets, maxDepth, dims, dev::kTileWaves) <= kMaxTileLdsBytes) {
        return dev::kTileWaves;
    }
    if (RowTileLdsBytes(buckets, maxDepth, dims, dev::kWideTileWaves) <= kMaxTileLdsBytes) {
        return dev::kWideTileWaves;
    }
    return RowTileLdsBytes(buckets, maxDepth, dims, dev::kTileWaves) <= kMaxTileLdsBytes ? dev::kTileWaves : 0;
}

// LDS of the deep-tile kernel: 256 documents' bins and the accumulator
size_t DeepTileLdsBytes(uint32_t rows, int dims) {
    return ((static_cast<size_t>(rows) * 256 + 15) & ~size_t(15)) + static_cast<size_t>(dims) * dev::kDocsPerBlock * sizeof(double);
}

// dimensions that a workgroup of the deep-tile kernel sums per walk of the trees
int DeepTileDims(int dim) {
    return dim == 1 ? 1 : 2;
}

// LDS of the quad-tile kernel: 64 documents' bins, then per wave the leaf values of four trees (later the partial sums)
size_t QuadTileLdsBytes(uint32_t rows, int maxd, uint32_t waves) {
    return ((static_cast<size_t>(rows) * 64 + 15) & ~size_t(15)) +
           static_cast<size_t>(waves) * 4 * (size_t(1) << maxd) * sizeof(double);
}

// Waves per workgroup of the quad-tile kernel: eight, or four when the rows leave room for no more; 0: no room
uint32_t QuadTileWaves(uint32_t rows, int maxd) {
    return QuadTileLdsBytes(rows, maxd, 8) <= kMaxTileLdsBytes ? 8u : QuadTileLdsBytes(rows, maxd, 4) <= kMaxTileLdsBytes ? 4u : 0u;
}

// LDS of the pair-tile kernel: 128 documents' bins, then per wave the leaf values of two trees; the same area
// takes one partial sum per wave, lane group and document at the end
size_t PairTileLdsBytes(uint32_t buckets, int maxd) {
    return ((static_cast<size_t>(buckets) * 128 + 15) & ~size_t(15)) +
           static_cast<size_t>(dev::kTileWaves) * 2 * std::max<size_t>(size_t(1) << maxd, 128) * sizeof(double);
}

// dimensions the tile kernel accumulates per pass over the trees (and the pitch of its padded leaf rows)
int TileChunk(int dim) {
    return dim == 1 ? 1 : dim == 2 ? 2 : dim <= 4 ? 4 : dim <= 8 ? 8 : dim <= 12 ? 12 : 16;
}

// Level-order tables of non-symmetric trees for EvalNonSymmetricTileKernel (its comment has the
// entry format). The walk they encode is CalcIndexesNonSymmetric, cpu/evaluator_impl.cpp:462-493:
// from a node, the chosen side's diff leads to the next node and a zero diff ends the walk at the
// node's own leaf (NonSymmetricNodeIdToLeafId). A zero side becomes a terminal entry of its own.
// usable = false when a tree does not fit the 16-bit offsets of an entry.
// The compact tables (EvalNonSymmetricLdsKernel) are filled when the model is one-dimensional,
// has at most 1023 buckets and no tree above dev::kNsLdsEntries entries (one-hot splits count two).
void BuildLevelOrderTrees(const TModelTrees& trees, int dim, const std::vector<uint32_t>& firstLeaf,
                          TDeviceVec<uint32_t>* entriesOut, TDeviceVec<uint32_t>* rowsOut, bool* usable, bool* noXor,
                          std::vector<uint32_t>* compactEntries, std::vector<uint32_t>* compactRows,
                          std::vector<double>* valuesByEntry, bool* compactUsable) {
    struct TItem {
        uint32_t Node;        // model node, or the parent node of a synthetic terminal
        bool Terminal;
        bool Second = false;     // the second test of a one-hot split taken apart (see unfold)
        uint32_t LeftEntry = 0;  // of a second test: the entry of the split's left side
        int64_t CopyOf = -1;     // an entry that repeats an earlier one of the tree: same test, same children
    };
    struct TUnfolded {
        std::vector<TItem> Order;                                // breadth first, the two children of an entry side by side
        std::vector<uint32_t> Level;
        std::vector<std::pair<uint32_t, uint32_t>> Children;     // entry index of (false side, true side); terminals: unused
        uint32_t Height = 0;
        bool Fits = true;
    };
    // Breadth-first order of a tree's entries. A tree whose nodes share children (the loader only checks that
    // every step stays inside the tree) unfolds into more entries than it has nodes, up to 2^depth: the walk
    // stops as soon as the entries no longer fit the 16-bit offsets, and the model goes to the kernel that
    // follows the step nodes.
    // splitOneHot: the compact entries only know "bin >= splitIdx". A one-hot split, bin == v, becomes two of
    // them: "bin >= v" (false: the model's left side) and behind its true side "bin >= v + 1" (false: the
    // model's right side, the bins are equal; true: the left side again). The entry of the left side is
    // repeated there, not its subtree: the copy names the same pair of children.
    const auto unfold = [&](uint32_t root, bool splitOneHot) {
        TUnfolded u;
        u.Order.push_back({root, false});
        u.Level.push_back(0);
        for (size_t i = 0; i < u.Order.size() && u.Order.size() * 8 <= 0xffffu; ++i) {
            if (u.Order[i].CopyOf >= 0) {
                const size_t original = static_cast<size_t>(u.Order[i].CopyOf);  // an earlier index: already visited
                const int64_t keep = u.Order[i].CopyOf;
                u.Order[i] = u.Order[original];
                u.Order[i].CopyOf = keep;
                u.Children.push_back(u.Children[original]);
                if (u.Order[i].Terminal) {
                    u.Height = std::max(u.Height, u.Level[i]);
                }
                continue;
            }
            const TItem item = u.Order[i];
            const auto& st = trees.NonSymmetricStepNodes[item.Node];
            const bool terminal = item.Terminal || (!item.Second && st.LeftSubtreeDiff == 0 && st.RightSubtreeDiff == 0);
            u.Order[i].Terminal = terminal;
            if (terminal) {
                u.Height = std::max(u.Height, u.Level[i]);
                u.Children.emplace_back(0, 0);
                continue;
            }
            const uint32_t diffs[2] = {st.LeftSubtreeDiff, st.RightSubtreeDiff};
            const auto pushSide = [&](int side) {
                const uint32_t index = static_cast<uint32_t>(u.Order.size());
                if (diffs[side] == 0) {
                    u.Order.push_back({item.Node, true});
                } else {
                    u.Order.push_back({item.Node + diffs[side], false});
                }
                u.Level.push_back(u.Level[i] + 1);
                return index;
            };
            const bool oneHot = splitOneHot && trees.RepackedBins[item.Node].XorMask != 0;
            uint32_t child[2];
            if (!oneHot) {
                child[0] = pushSide(0);
                child[1] = pushSide(1);
            } else if (!item.Second) {
                child[0] = pushSide(0);
                child[1] = static_cast<uint32_t>(u.Order.size());
                TItem second{item.Node, false};
                second.Second = true;
                second.LeftEntry = child[0];
                u.Order.push_back(second);
                u.Level.push_back(u.Level[i] + 1);
            } else {
                child[0] = pushSide(1);
                child[1] = static_cast<uint32_t>(u.Order.size());
                TItem copy{item.Node, false};
                copy.CopyOf = item.LeftEntry;
                u.Order.push_back(copy);
                u.Level.push_back(u.Level[i] + 1);
            }
            u.Children.emplace_back(child[0], child[1]);
        }
        u.Fits = u.Order.size() * 8 <= 0xffffu;
        return u;
    };
    const size_t treeCount = trees.GetTreeCount();
    *noXor = true;
    for (const auto& rb : trees.RepackedBins) {
        *noXor = *noXor && rb.XorMask == 0;
    }
    std::vector<uint32_t> entries, rows(treeCount * 4, 0);
    *usable = true;
    *compactUsable = trees.EffectiveBinFeaturesBucketCount <= 1023;
    compactRows->assign(treeCount * 4, 0);
    for (size_t t = 0; t < treeCount && *usable; ++t) {
        const uint32_t root = static_cast<uint32_t>(trees.TreeStartOffsets[t]);
        const size_t firstEntry = entries.size() / 2;
        const TUnfolded plain = unfold(root, false);
        if (!plain.Fits) {
            *usable = false;
            break;
        }
        const std::vector<TItem>& order = plain.Order;
        const auto& children = plain.Children;
        for (size_t i = 0; i < order.size(); ++i) {
            const TItem item = order[i];
            uint32_t x, y;
            if (item.Terminal) {
                const uint32_t leafRel = (trees.NonSymmetricNodeIdToLeafId[item.Node] - firstLeaf[t]) / static_cast<uint32_t>(dim);
                if (leafRel > 0xffffu) {
                    *usable = false;
                    break;
                }
                x = 0;
                y = leafRel | (static_cast<uint32_t>(i * 8) << 16);
            } else {
                const auto& rb = trees.RepackedBins[item.Node];
                x = *noXor ? (static_cast<uint32_t>(rb.FeatureIndex) << 8) | (static_cast<uint32_t>(rb.SplitIdx) << 24)
                           : static_cast<uint32_t>(rb.FeatureIndex) | (static_cast<uint32_t>(rb.XorMask) << 16) |
                                 (static_cast<uint32_t>(rb.SplitIdx) << 24);
                y = (children[i].first * 8) | ((children[i].second * 8) << 16);
            }
            entries.push_back(x);
            entries.push_back(y);
        }
        rows[t * 4 + 0] = static_cast<uint32_t>(firstEntry);
        rows[t * 4 + 1] = plain.Height;
        rows[t * 4 + 2] = firstLeaf[t];
        // compact layout: root at 0, entry 1 unused, so that every pair of children starts even
        if (!*compactUsable || !*usable) {
            *compactUsable = false;
            continue;
        }
        const TUnfolded split = *noXor ? TUnfolded() : unfold(root, true);
        const TUnfolded& compact = *noXor ? plain : split;
        *compactUsable = compact.Fits && compact.Order.size() + 1 <= static_cast<size_t>(dev::kNsLdsEntries);
        if (*compactUsable) {
            const auto compactIndex = [](size_t i) { return static_cast<uint32_t>(i == 0 ? 0 : i + 1); };
            (*compactRows)[t * 4 + 0] = static_cast<uint32_t>(compactEntries->size());
            (*compactRows)[t * 4 + 1] = compact.Height;
            (*compactRows)[t * 4 + 2] = static_cast<uint32_t>(compact.Order.size() + 1);
            for (size_t i = 0; i < compact.Order.size(); ++i) {
                const TItem item = compact.Order[i];
                const uint32_t self = compactIndex(i);
                if (item.Terminal) {
                    const bool odd = (self & 1u) != 0;
                    compactEntries->push_back((odd ? 0u : 255u) | ((self & ~1u) << 21));
                    const double* leaf = trees.LeafValues.data() + trees.NonSymmetricNodeIdToLeafId[item.Node];
                    valuesByEntry->insert(valuesByEntry->end(), leaf, leaf + dim);
                } else {
                    const auto& rb = trees.RepackedBins[item.Node];
                    // a one-hot split holds ~value in its xor mask (and 255 as its split index)
                    uint32_t splitIdx = rb.SplitIdx;
                    if (rb.XorMask != 0) {
                        const uint32_t value = (~static_cast<uint32_t>(rb.XorMask)) & 0xffu;
                        splitIdx = item.Second ? value + 1 : value;
                        *compactUsable = *compactUsable && splitIdx <= 255;
                    }
                    // the true side always follows the false side in the order
                    compactEntries->push_back(splitIdx | (static_cast<uint32_t>(rb.FeatureIndex) << 8) |
                                              (compactIndex(compact.Children[i].first) << 21));
                    valuesByEntry->insert(valuesByEntry->end(), static_cast<size_t>(dim), 0.0);
                }
                if (i == 0) {
                    compactEntries->push_back(255u);  // the unused entry
                    valuesByEntry->insert(valuesByEntry->end(), static_cast<size_t>(dim), 0.0);
                }
            }
        }
    }
    *compactUsable = *compactUsable && *usable;
    if (*usable) {
        entriesOut->Upload(entries);
        rowsOut->Upload(rows);
    }
}

// Where the kernels read the model's features in a caller's data: the positions stored in the model, or
// those positions sent through a feature layout. The vector sizes a caller must provide follow the
// reference without a layout (the last feature of each list decides, model.h:494-541) and are the
// largest position read plus one with a layout.
struct TFeaturePositions {
    const TFeatureLayout* Layout = nullptr;
    size_t FlatVectorSize = 0;
    size_t MinFloatSize = 0;
    size_t MinCatSize = 0;

    TFeaturePosition Of(const TFloatFeature& f) const {
        return Layout ? Layout->Remap(f) : TFeaturePosition{f.Index, f.FlatIndex};
    }
    TFeaturePosition Of(const TCatFeature& c) const {
        return Layout ? Layout->Remap(c) : TFeaturePosition{c.Index, c.FlatIndex};
    }

    TFeaturePositions(const TModelTrees& trees, const TFeatureLayout* layout)
        : Layout(layout && layout->Defined() ? layout : nullptr)
    {
        if (!Layout) {
            FlatVectorSize = trees.GetFlatFeatureVectorExpectedSize();
            MinFloatSize = trees.MinimalSufficientFloatFeaturesVectorSize;
            MinCatSize = trees.MinimalSufficientCatFeaturesVectorSize;
            return;
        }
        for (const auto& f : trees.FloatFeatures) {
            if (f.UsedInModel() && f.Index >= 0 && f.FlatIndex >= 0) {
                const TFeaturePosition p = Of(f);
                FlatVectorSize = std::max(FlatVectorSize, static_cast<size_t>(p.FlatIndex) + 1);
                MinFloatSize = std::max(MinFloatSize, static_cast<size_t>(p.Index) + 1);
            }
        }
        for (const auto& c : trees.CatFeatures) {
            if (c.UsedInModel && c.Index >= 0 && c.FlatIndex >= 0) {
                const TFeaturePosition p = Of(c);
                FlatVectorSize = std::max(FlatVectorSize, static_cast<size_t>(p.FlatIndex) + 1);
                MinCatSize = std::max(MinCatSize, static_cast<size_t>(p.Index) + 1);
            }
        }
    }
};

// Device tables of the model's CTR features (TStaticCtrProvider, catboost/libs/model/static_ctr_provider.cpp):
// per feature a descriptor and its projection (SetupBinFeatureIndexes, :142-178, resolved to bucket
// numbers and input columns), all index buckets and all rows. Every row index and class index the kernel
// can reach is checked here, so a damaged model fails at load instead of reading out of bounds.
// Appends one bucket entry per 254 borders of a CTR feature to the binarize bucket tables.
void BuildCtrTables(const TModelTrees& trees, const TFeaturePositions& positions,
                    const std::vector<TCtrValueTable>& tables, std::vector<uint32_t>* srcFlat,
                    std::vector<uint32_t>* srcSplit, std::vector<uint32_t>* offsets, std::vector<uint32_t>* flags,
                    std::vector<uint32_t>* values, TDeviceVec<uint32_t>* featuresOut, TDeviceVec<uint32_t>* itemsOut,
                    TDeviceVec<uint32_t>* indexOut, TDeviceVec<uint32_t>* blobOut, TDeviceVec<uint32_t>* catColumnsFlatOut,
                    TDeviceVec<uint32_t>* catColumnsSplitOut, uint32_t* catColumnCountOut) {
    static_assert(sizeof(dev::TCtrFeatureDev) == 64 && sizeof(dev::TCtrItemDev) == 16, "device CTR records changed size");
    std::vector<dev::TCtrFeatureDev> features;
    std::vector<dev::TCtrItemDev> items;
    std::vector<uint32_t> index, blob;
    std::vector<uint32_t> catColumnsFlat, catColumnsSplit;  // distinct categorical columns of all projections
    std::vector<uint32_t> tableIndexBegin(tables.size(), 0), tableBlobBegin(tables.size(), 0), tableRows(tables.size(), 0);
    std::vector<bool> tableUploaded(tables.size(), false);

    // first bucket of every used float feature and of every one-hot feature
    std::vector<uint32_t> floatFirstBucket(trees.FloatFeatures.size(), 0), oneHotFirstBucket(trees.OneHotFeatures.size(), 0);
    uint32_t bucket = 0;
    for (size_t i = 0; i < trees.FloatFeatures.size(); ++i) {
        floatFirstBucket[i] = bucket;
        bucket += static_cast<uint32_t>((trees.FloatFeatures[i].Borders.size() + kMaxValuesPerBin - 1) / kMaxValuesPerBin);
    }
    for (size_t i = 0; i < trees.OneHotFeatures.size(); ++i) {
        oneHotFirstBucket[i] = bucket;
        bucket += static_cast<uint32_t>((trees.OneHotFeatures[i].Values.size() + kMaxValuesPerBin - 1) / kMaxValuesPerBin);
    }

    for (const auto& feature : trees.CtrFeatures) {
        const TModelCtr& ctr = feature.Ctr;
        size_t t = 0;
        while (t < tables.size() && !(tables[t].ModelCtrBase == ctr.Base)) {
            ++t;
        }
        CBAMD_ENSURE(t < tables.size(), "Model has a CTR feature without its table of learned statistics");
        const TCtrValueTable& table = tables[t];
        const size_t bucketCount = table.IndexHashRaw.size() / 12;
        CBAMD_ENSURE(table.IndexHashRaw.size() % 12 == 0 && bucketCount > 0 && (bucketCount & (bucketCount - 1)) == 0 &&
                         bucketCount <= (size_t(1) << 31),
                     "Dense hash view must have 2^k buckets");
        // bytes of one row and the class indexes the CTR reads (static_ctr_provider.cpp:52-126)
        size_t rowBytes = 0;
        switch (ctr.Base.CtrType) {
            case ECtrType::BinarizedTargetMeanValue:
            case ECtrType::FloatTargetMeanValue:
                rowBytes = 8;
                break;
            case ECtrType::Counter:
            case ECtrType::FeatureFreq:
                rowBytes = 4;
                break;
            case ECtrType::Buckets:
                CBAMD_ENSURE(table.TargetClassesCount > 0 && ctr.TargetBorderIdx >= 0 &&
                                 ctr.TargetBorderIdx < table.TargetClassesCount,
                             "CTR target border index out of range");
                rowBytes = 4 * static_cast<size_t>(table.TargetClassesCount);
                break;
            case ECtrType::Borders:
                if (table.TargetClassesCount > 2) {
                    CBAMD_ENSURE(ctr.TargetBorderIdx >= 0 && ctr.TargetBorderIdx < table.TargetClassesCount,
                                 "CTR target border index out of range");
                    rowBytes = 4 * static_cast<size_t>(table.TargetClassesCount);
                } else {
                    rowBytes = 8;
                }
                break;
        }
        if (!tableUploaded[t]) {
            tableUploaded[t] = true;
            tableIndexBegin[t] = static_cast<uint32_t>(index.size() / 3);
            tableBlobBegin[t] = static_cast<uint32_t>(blob.size());
            bool hasEmpty = false;
            uint32_t maxRow = 0;
            bool anyRow = false;
            for (size_t b = 0; b < bucketCount; ++b) {
                uint32_t w[3];
                std::memcpy(w, table.IndexHashRaw.data() + 12 * b, 12);
                index.insert(index.end(), w, w + 3);
                if ((w[0] & w[1]) == 0xffffffffu) {
                    hasEmpty = true;
                } else {
                    maxRow = std::max(maxRow, w[2]);
                    anyRow = true;
                }
            }
            CBAMD_ENSURE(hasEmpty, "CTR index hash table has no empty bucket");
            tableRows[t] = anyRow ? maxRow + 1 : 0;
            blob.resize(blob.size() + (table.CTRBlob.size() + 3) / 4, 0);
            if (!table.CTRBlob.empty()) {
                std::memcpy(blob.data() + tableBlobBegin[t], table.CTRBlob.data(), table.CTRBlob.size());
            }
            CBAMD_ENSURE(index.size() / 3 < (size_t(1) << 32) && blob.size() < (size_t(1) << 32), "CTR tables are too large");
        }
        CBAMD_ENSURE(static_cast<size_t>(tableRows[t]) * rowBytes <= table.CTRBlob.size(),
                     "CTR value table is shorter than its index");

        dev::TCtrFeatureDev f{};
        f.ItemBegin = static_cast<uint32_t>(items.size());
        for (int catIndex : ctr.Base.Projection.CatFeatures) {
            const TCatFeature* cat = nullptr;
            for (const auto& c : trees.CatFeatures) {
                if (c.Index == catIndex && c.UsedInModel) {
                    cat = &c;
                }
            }
            CBAMD_ENSURE(cat != nullptr && cat->FlatIndex >= 0 && cat->Index >= 0,
                         "CTR projection refers to an unknown or unused categorical feature");
            const TFeaturePosition at = positions.Of(*cat);
            CBAMD_ENSURE(static_cast<size_t>(at.FlatIndex) < positions.FlatVectorSize &&
                             static_cast<size_t>(at.Index) < positions.MinCatSize,
                         "categorical feature position exceeds the model's feature vector size");
            uint32_t tileRow = 0;
            while (tileRow < catColumnsSplit.size() && catColumnsSplit[tileRow] != static_cast<uint32_t>(at.Index)) {
                ++tileRow;
            }
            if (tileRow == catColumnsSplit.size()) {
                catColumnsFlat.push_back(static_cast<uint32_t>(at.FlatIndex));
                catColumnsSplit.push_back(static_cast<uint32_t>(at.Index));
            }
            items.push_back({dev::kCtrItemCat, static_cast<uint32_t>(at.FlatIndex), static_cast<uint32_t>(at.Index), tileRow});
        }
        for (const auto& split : ctr.Base.Projection.BinFeatures) {
            bool found = false;
            for (size_t i = 0; i < trees.FloatFeatures.size() && !found; ++i) {
                const auto& ff = trees.FloatFeatures[i];
                if (ff.Index != split.FloatFeature) {
                    continue;
                }
                for (size_t b = 0; b < ff.Borders.size(); ++b) {
                    if (ff.Borders[b] == split.Split) {
                        const uint32_t at = floatFirstBucket[i] + static_cast<uint32_t>(b / kMaxValuesPerBin);
                        items.push_back({dev::kCtrItemBinGe, at, at, static_cast<uint32_t>(b % kMaxValuesPerBin) + 1});
                        found = true;
                        break;
                    }
                }
            }
            CBAMD_ENSURE(found, "CTR projection refers to a float split the model does not have");
        }
        for (const auto& split : ctr.Base.Projection.OneHotFeatures) {
            bool found = false;
            for (size_t i = 0; i < trees.OneHotFeatures.size() && !found; ++i) {
                const auto& oh = trees.OneHotFeatures[i];
                if (oh.CatFeatureIndex != split.CatFeatureIdx) {
                    continue;
                }
                for (size_t v = 0; v < oh.Values.size(); ++v) {
                    if (oh.Values[v] == split.Value) {
                        const uint32_t at = oneHotFirstBucket[i] + static_cast<uint32_t>(v / kMaxValuesPerBin);
                        items.push_back({dev::kCtrItemBinEq, at, at, static_cast<uint32_t>(v % kMaxValuesPerBin) + 1});
                        found = true;
                        break;
                    }
                }
            }
            CBAMD_ENSURE(found, "CTR projection refers to a one-hot split the model does not have");
        }
        f.ItemEnd = static_cast<uint32_t>(items.size());
        f.HashBuckets = tableIndexBegin[t];
        f.HashMask = static_cast<uint32_t>(bucketCount - 1);
        f.BlobOffset = tableBlobBegin[t];
        f.Type = static_cast<uint32_t>(ctr.Base.CtrType);
        f.TargetBorderIdx = ctr.TargetBorderIdx;
        f.TargetClassesCount = table.TargetClassesCount;
        f.CounterDenominator = table.CounterDenominator;
        f.PriorNum = ctr.PriorNum;
        f.PriorDenom = ctr.PriorDenom;
        f.Shift = ctr.Shift;
        f.Scale = ctr.Scale;
        f.FirstBucket = static_cast<uint32_t>(srcFlat->size());
        for (size_t begin = 0; begin < feature.Borders.size(); begin += kMaxValuesPerBin) {
            const size_t end = std::min(begin + kMaxValuesPerBin, feature.Borders.size());
            std::vector<float> b;
            for (size_t i = begin; i < end; ++i) {
                if (!std::isnan(feature.Borders[i])) {
                    b.push_back(feature.Borders[i]);
                }
            }
            std::sort(b.begin(), b.end());
            for (float x : b) {
                uint32_t bits;
                std::memcpy(&bits, &x, 4);
                values->push_back(bits);
            }
            offsets->push_back(static_cast<uint32_t>(values->size()));
            srcFlat->push_back(0);
            srcSplit->push_back(0);
            flags->push_back(dev::kBucketFlagCtr);
        }
        f.BucketCount = static_cast<uint32_t>(srcFlat->size()) - f.FirstBucket;
        f.SameProjectionAsPrevious =
            !features.empty() && trees.CtrFeatures[features.size() - 1].Ctr.Base.Projection == ctr.Base.Projection ? 1u : 0u;
        features.push_back(f);
    }
    std::vector<uint32_t> raw(features.size() * (sizeof(dev::TCtrFeatureDev) / 4));
    std::memcpy(raw.data(), features.data(), raw.size() * 4);
    featuresOut->Upload(raw);
    raw.assign(std::max<size_t>(items.size(), 1) * (sizeof(dev::TCtrItemDev) / 4), 0);
    std::memcpy(raw.data(), items.data(), items.size() * sizeof(dev::TCtrItemDev));
    itemsOut->Upload(raw);
    indexOut->Upload(index);
    if (blob.empty()) {
        blob.push_back(0);
    }
    blobOut->Upload(blob);
    *catColumnCountOut = static_cast<uint32_t>(catColumnsFlat.size());
    catColumnsFlatOut->Upload(catColumnsFlat);
    catColumnsSplitOut->Upload(catColumnsSplit);
}

}  // namespace

int GetHipDeviceCount() {
    int n = 0;
    const hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        throw TModelError(std::string("HIP runtime reports no usable device: ") + hipGetErrorString(e));
    }
    return n;
}

struct THipEvaluator::TImpl {
    int DeviceId = 0;
    hipStream_t Stream = nullptr;
    uint8_t* NoAllocScratch = nullptr;  // this device's copy of the file-scope array `scratch`
    bool Oblivious = true;
    uint32_t RealBucketCount = 0;  // buckets of the model; the device layout uses max(1, this)
    uint32_t LayoutBuckets = 1;
    uint32_t BinarizeBuckets = 0;  // float and one-hot buckets: what the binarize kernels fill
    uint32_t CtrCount = 0;         // CTR features; their buckets follow and CtrBinarizeKernel fills them
    size_t FlatVectorSize = 0;
    size_t MinFloatSize = 0;
    size_t MinCatSize = 0;
    bool HasCats = false;
    uint32_t MaxBucketValues = 0;  // largest number of borders / one-hot values in one bucket
    uint32_t MaxDepth = 0;         // deepest oblivious tree
    bool HasOneHot = false;

    // binarize tables
    TDeviceVec<uint32_t> BucketSrcFlat, BucketSrcSplit, BucketOffset, BucketFlags, Values;
    TDeviceVec<uint32_t> BucketGrid;  // 4 dwords per bucket: lowest border, cells per unit, search steps, 0
    TDeviceVec<uint32_t> BucketLut;   // kLutCells bytes per bucket
    TDeviceVec<unsigned long long> ExpMantissa;  // the table of the prediction types' exponent
    // CTR tables: feature descriptors, projection items, the index buckets and the rows of all tables
    TDeviceVec<uint32_t> CtrFeatures, CtrItems, CtrIndexBuckets, CtrBlob, CtrCatColumnsFlat, CtrCatColumnsSplit;
    uint32_t CtrCatColumnCount = 0;
    bool CtrTileUsable = false;  // the projections' categorical columns fit the LDS tile of CtrBinarizeTileKernel
    // tree tables
    TDeviceVec<uint32_t> Splits, TreeStart, TreeSize, FirstLeaf, StepNodes, NodeToLeaf;
    TDeviceVec<double> Leaves, Bias;
    TDeviceVec<uint32_t> PackedTrees;  // tile kernel: 16 dwords per oblivious tree of depth <= 8
    TDeviceVec<uint32_t> PackedMixed;  // half-tile kernel: packed rows in the form chosen per tree
    TDeviceVec<double> HalfTileLeaves; // half-tile kernel: 64 or 256 leaf values per tree at a fixed pitch
    TDeviceVec<uint32_t> PairRows;     // pair-tile kernel: 8 dwords per tree, empty when the model does not qualify
    bool PairSix = false;              // ... in the six-bit form (every bin below 64)
    TDeviceVec<uint32_t> QuadRows;     // quad-tile kernel: the same with 64 bytes per row of the tile
    TDeviceVec<uint32_t> TileRows;     // row-tile kernel (whole tile, one tree per wave): the same with 256 bytes per bucket
    TDeviceVec<double> TileLeaves;     // its leaf values: [slice of the dimensions][tree][pair of dimensions][leaf][2]
    size_t TileSliceStride = 0;        // 16-byte pairs of TileLeaves per slice
    TDeviceVec<uint32_t> DeepRows;     // deep-tile kernel (depth 9 to 16): 32 dwords per tree, two halves of the row-tile form
    TDeviceVec<uint32_t> DeepFirstLeaf;  // and the trees' first leaf values in Leaves (one dimension) or first leaves in DeepLeaves
    TDeviceVec<double> DeepLeaves;       // several dimensions: [slice of two][tree][leaf][2]
    uint32_t DeepSliceLeaves = 0;        // leaves of all trees
    TDeviceVec<uint32_t> TileMap;      // rows of the tile of the row-tile or pair-tile kernel when buckets of more than
                                       // 127 values take two; empty: a row per bucket
    uint32_t TileRowCount = 0;
    TDeviceVec<double> LeavesPadded;   // tile kernel, multi-dimensional: [tree][chunk][leaf][TileChunk(dim)]
    bool PackedSevenBit = false;
    bool LeavesPairAligned = false;  // every tree's first leaf value sits at an even index
    double Scale = 1.0;
    int Dim = 1;
    std::vector<double> HostBias;

    // non-symmetric trees re-laid level by level for the tile kernel
    bool NsTileUsable = false;
    bool NsNoXor = false;
    TDeviceVec<uint32_t> NsEntries;  // pairs of dwords
    TDeviceVec<uint32_t> NsRows;     // 4 dwords per tree
    bool NsLdsUsable = false;        // compact entries walked out of LDS (one-dimensional, no xor)
    TDeviceVec<uint32_t> NsCompactEntries;
    TDeviceVec<uint32_t> NsCompactRows;  // 8 dwords per unit of trees
    uint32_t NsUnitCount = 0;
    uint32_t NsEntryCount = 0;       // entries of all units: rows of NsValuesByEntry per slice of the dimensions
    TNsLdsShape NsLdsShape{0, 0};    // waves and entries per region of EvalNonSymmetricLdsKernel for this model
    TDeviceVec<double> NsValuesByEntry;

    // register-resident kernels (one-dimensional 7-bit oblivious models of depth <= 8 whose
    // buckets fit the register file): level rows and leaf values at a fixed pitch per tree
    bool RegKernelUsable = false;
    bool SmallBatchSlices = true;  // small batches: slices of the trees on workgroups of their own
    hipModule_t RegModule = nullptr;  // the device's shared module (SharedRegModule), not owned
    hipFunction_t RegFunction = nullptr;
    uint32_t RegWaves = 0;
    uint32_t RegTreeBlocks = 0;
    uint32_t RegTreeBlockSize = 16;   // trees per LDS buffer of the chosen kernel
    uint32_t RegRowDwords = 16;       // dwords of a tree's level table
    size_t RegLaunchLeaves = 0;  // doubles of the leaf table of one launch
    TDeviceVec<uint32_t> RegRows;
    TDeviceVec<double> RegLeaves;  // [launch][tree][leaf row][pitch]
    TDeviceVec<double> RegBias;    // the bias, readable for a whole pitch behind every dimension
    // The launches of a pass over the trees: the kernel's pitch in dimensions each, the last one with the narrowest kernel that
    // holds what is left (ten dimensions: six, then four instead of six of which two are padding).
    struct TRegLaunch {
        hipFunction_t Function = nullptr;
        const char* Name = "";
        uint32_t Waves = 0;
        uint32_t FirstDim = 0;
        uint32_t StoreDims = 1;
        uint32_t TreeBlock = 16;         // trees per LDS buffer of this kernel
        size_t TreeLeafDoubles = 0;      // doubles of a tree in Leaves
        const double* Leaves = nullptr;  // the launch's leaf table
    };
    std::vector<TRegLaunch> RegLaunches;
    TDeviceVec<double> RegTailLeaves;  // leaf table of a last launch that uses another kernel
    // Models without xor masks whose buckets hold more than 127 values: such a bucket takes two bins registers,
    // min(bin, 127) and max(bin - 127, 0), so that every level is a 7-bit compare (the kernels' register map)
    TDeviceVec<uint32_t> RegMap;

    // fused kernels, per row layout (0: flat rows, 1: split rows of a model without categorical features)
    struct TFused {
        bool Usable = false;
        uint32_t UnitCount = 0;
        TDeviceVec<uint32_t> Rows;    // level rows that name bins registers of the fused layout
        TDeviceVec<uint32_t> Units;   // unit records
        TDeviceVec<uint8_t> Table;    // border table images, then a copy of the leaf table
    };
    TFused Fused[2];
    hipFunction_t FusedFunction = nullptr;
    uint32_t FusedWaves = 0;
    // Below about one wave per SIMD a fused launch lasts as long as one wave's binarize phase and tree walk,
    // and two launches (the binarize kernel spreads a block over many waves) are shorter.
    size_t FusedMinDocs() const {
        return SmallBatchSlices ? size_t(1024) * dev::kDocsPerBlock : 0;
    }
    const char* RegKernelName = "";
    const char* FusedKernelName = "";

    // Staging of the calls that own their buffers (CalcDevice and the host entry points): a call borrows a
    // context - a stream, a bin buffer and two slots of pinned and device staging memory - from a small pool,
    // so that a few callers of one evaluator run side by side and later ones wait for a free context.
    struct THostSlot {
        TPinnedVec<float> PinnedFloats;
        TPinnedVec<int32_t> PinnedCats;
        TPinnedVec<double> PinnedResults;
        TPinnedVec<uint32_t> PinnedIndexes;
        TPinnedVec<uint8_t> PinnedExport;
        TDeviceVec<float> StageFloats;
        TDeviceVec<int32_t> StageCats;
        TDeviceVec<double> StageResults;
        TDeviceVec<uint32_t> StageIndexes;
        TDeviceVec<uint8_t> StageExport;
        // binarize start, binarize end, evaluate end, results on the host
        hipEvent_t Ev[4] = {nullptr, nullptr, nullptr, nullptr};
    };
    struct THostContext {
        hipStream_t Stream = nullptr;
        TDeviceVec<uint8_t> ScratchBins;
        TDeviceVec<double> SlicePartials;  // raw sums per slice of the trees (small batches)
        THostSlot Slots[2];
        hipEvent_t Ev[3] = {nullptr, nullptr, nullptr};
        bool Busy = false;

        THostContext() {
            try {
                HIP_CHECK(hipStreamCreateWithFlags(&Stream, hipStreamNonBlocking));
                for (auto& e : Ev) {
                    HIP_CHECK(hipEventCreate(&e));
                }
                for (auto& slot : Slots) {
                    for (auto& e : slot.Ev) {
                        HIP_CHECK(hipEventCreate(&e));
                    }
                }
            } catch (...) {
                Release();  // the destructor does not run for a constructor that throws
                throw;
            }
        }
        ~THostContext() {
            Release();
        }
        void Release() {
            if (Stream) {
                (void)hipStreamSynchronize(Stream);
            }
            for (auto& e : Ev) {
                if (e) {
                    (void)hipEventDestroy(e);
                }
            }
            for (auto& slot : Slots) {
                for (auto& e : slot.Ev) {
                    if (e) {
                        (void)hipEventDestroy(e);
                    }
                }
            }
            if (Stream) {
                (void)hipStreamDestroy(Stream);
                Stream = nullptr;
            }
        }
        THostContext(const THostContext&) = delete;
        THostContext& operator=(const THostContext&) = delete;
    };
    static constexpr size_t kMaxHostContexts = 4;
    std::mutex ContextLock;
    std::condition_variable ContextFree;
    std::vector<std::unique_ptr<THostContext>> Contexts;

    // A context of the pool for the time of one call.
    class TContextLease {
    public:
        explicit TContextLease(TImpl& impl)
            : Impl(impl)
        {
            std::unique_lock<std::mutex> guard(Impl.ContextLock);
            for (;;) {
                for (auto& c : Impl.Contexts) {
                    if (!c->Busy) {
                        Context = c.get();
                        break;
                    }
                }
                if (!Context && Impl.Contexts.size() < kMaxHostContexts) {
                    Impl.Contexts.emplace_back(new THostContext);
                    Context = Impl.Contexts.back().get();
                }
                if (Context) {
                    Context->Busy = true;
                    return;
                }
                Impl.ContextFree.wait(guard);
            }
        }
        ~TContextLease() {
            {
                std::lock_guard<std::mutex> guard(Impl.ContextLock);
                Context->Busy = false;
            }
            Impl.ContextFree.notify_one();
        }
        THostContext& operator*() const { return *Context; }
        THostContext* operator->() const { return Context; }

    private:
        TImpl& Impl;
        THostContext* Context = nullptr;
    };

    dev::TBinarizeTables BinarizeTables(bool flat) const {
        dev::TBinarizeTables t;
        t.BucketCount = BinarizeBuckets;
        t.BucketPitch = LayoutBuckets;
        t.BucketSrc = flat ? BucketSrcFlat.Get() : BucketSrcSplit.Get();
        t.BucketOffset = BucketOffset.Get();
        t.BucketFlags = BucketFlags.Get();
        t.Values = Values.Get();
        t.Grid = reinterpret_cast<const uint4*>(BucketGrid.Get());
        t.Lut = BucketLut.Get();
        return t;
    }
    dev::TCtrTablesDev CtrTables() const {
        dev::TCtrTablesDev t;
        t.Features = reinterpret_cast<const dev::TCtrFeatureDev*>(CtrFeatures.Get());
        t.Items = reinterpret_cast<const dev::TCtrItemDev*>(CtrItems.Get());
        t.IndexBuckets = CtrIndexBuckets.Get();
        t.Blob = CtrBlob.Get();
        t.CatColumnsFlat = CtrCatColumnsFlat.Get();
        t.CatColumnsSplit = CtrCatColumnsSplit.Get();
        t.CatColumnCount = CtrCatColumnCount;
        t.FeatureCount = CtrCount;
        return t;
    }
    dev::TTreeTables TreeTables() const {
        dev::TTreeTables t;
        t.Splits = Splits.Get();
        t.TreeStart = TreeStart.Get();
        t.TreeSize = TreeSize.Get();
        t.FirstLeaf = FirstLeaf.Get();
        t.StepNodes = StepNodes.Get();
        t.NodeToLeaf = NodeToLeaf.Get();
        t.Leaves = Leaves.Get();
        t.Bias = Bias.Get();
        t.Scale = Scale;
        t.Dim = Dim;
        return t;
    }
    hipStream_t Pick(void* stream) const { return stream ? static_cast<hipStream_t>(stream) : Stream; }

    // Also runs when the evaluator's constructor throws half way (a refused model), so that the
    // stream, the events and the code object of a partly built evaluator are released.
    ~TImpl() {
        (void)hipSetDevice(DeviceId);
        if (Stream) {
            (void)hipStreamSynchronize(Stream);
        }
        Contexts.clear();
        if (Stream) {
            (void)hipStreamDestroy(Stream);
        }
    }
};

THipEvaluator::THipEvaluator(const TModelTrees& trees, int deviceId, const std::vector<TCtrValueTable>* ctrTables,
                             const TFeatureLayout* layout)
    : Impl(new TImpl)
{
    const TFeaturePositions positions(trees, layout);
    const TKernelSwitches switches = TKernelSwitches::FromEnvironment();
    const int deviceCount = GetHipDeviceCount();
    CBAMD_ENSURE(deviceCount > 0, "no HIP device found: the HIP evaluator needs an AMD GPU");
    CBAMD_ENSURE(deviceId >= 0 && deviceId < deviceCount, "HIP device id out of range");
    HIP_CHECK(hipSetDevice(deviceId));
    TImpl& m = *Impl;
    m.DeviceId = deviceId;
    m.SmallBatchSlices = switches.SmallBatch;
    m.NoAllocScratch = NoAllocScratchOfCurrentDevice(deviceId);
    HIP_CHECK(hipStreamCreateWithFlags(&m.Stream, hipStreamNonBlocking));
    TreeCount = trees.GetTreeCount();
    ApproxDimension = trees.ApproxDimension;
    BucketCount = trees.EffectiveBinFeaturesBucketCount;
    m.Oblivious = trees.IsOblivious();
    m.RealBucketCount = BucketCount;
    m.LayoutBuckets = std::max<uint32_t>(1, BucketCount);
    m.FlatVectorSize = positions.FlatVectorSize;
    m.MinFloatSize = positions.MinFloatSize;
    m.MinCatSize = positions.MinCatSize;
    m.HasCats = trees.UsedCatFeaturesCount > 0;
    m.Dim = trees.ApproxDimension;
    m.Scale = trees.Scale;
    m.HostBias = trees.Bias;
    {
        const TFastExpConstants constants = FastExpConstants();
        m.ExpMantissa.Upload(std::vector<unsigned long long>(constants.Mantissa, constants.Mantissa + 2048));
    }

    // ---- binarize tables: one entry per bucket, float buckets first, then one-hot buckets, in
    // the order of BinarizeFeatures (cpu/quantization.h:366-409, 54-79). Borders are sorted inside
    // each bucket (the bin is a count, so order does not matter) and NaN borders, which never
    // compare below anything, are dropped.
    std::vector<uint32_t> srcFlat, srcSplit, offsets, flags, values;
    offsets.push_back(0);
    for (const auto& f : trees.FloatFeatures) {
        if (!f.UsedInModel()) {
            continue;
        }
        CBAMD_ENSURE(f.FlatIndex >= 0 && f.Index >= 0, "float feature without a position");
        // the vector sizes come from the last feature of each list (as in the reference); a feature
        // that points past them would make the kernels read behind a caller's row
        const TFeaturePosition at = positions.Of(f);
        CBAMD_ENSURE(static_cast<size_t>(at.FlatIndex) < m.FlatVectorSize && static_cast<size_t>(at.Index) < m.MinFloatSize,
                     "float feature position exceeds the model's feature vector size");
        for (size_t begin = 0; begin < f.Borders.size(); begin += kMaxValuesPerBin) {
            const size_t end = std::min(begin + kMaxValuesPerBin, f.Borders.size());
            std::vector<float> b;
            for (size_t i = begin; i < end; ++i) {
                if (!std::isnan(f.Borders[i])) {
                    b.push_back(f.Borders[i]);
                }
            }
            std::sort(b.begin(), b.end());
            for (float x : b) {
                uint32_t bits;
                std::memcpy(&bits, &x, 4);
                values.push_back(bits);
            }
            offsets.push_back(static_cast<uint32_t>(values.size()));
            srcFlat.push_back(static_cast<uint32_t>(at.FlatIndex));
            srcSplit.push_back(static_cast<uint32_t>(at.Index));
            const bool nanToInf = f.HasNans && f.NanValueTreatment == ENanValueTreatment::AsTrue;
            flags.push_back(nanToInf ? dev::kBucketFlagNanToInf : 0);
        }
    }
    for (const auto& oh : trees.OneHotFeatures) {
        const TCatFeature* cat = nullptr;
        for (const auto& c : trees.CatFeatures) {
            if (c.Index == oh.CatFeatureIndex && c.UsedInModel) {
                cat = &c;
            }
        }
        CBAMD_ENSURE(cat != nullptr, "one-hot feature refers to an unknown or unused categorical feature");
        CBAMD_ENSURE(cat->FlatIndex >= 0 && cat->Index >= 0, "categorical feature without a position");
        const TFeaturePosition at = positions.Of(*cat);
        CBAMD_ENSURE(static_cast<size_t>(at.FlatIndex) < m.FlatVectorSize && static_cast<size_t>(at.Index) < m.MinCatSize,
                     "categorical feature position exceeds the model's feature vector size");
        for (size_t begin = 0; begin < oh.Values.size(); begin += kMaxValuesPerBin) {
            const size_t end = std::min(begin + kMaxValuesPerBin, oh.Values.size());
            for (size_t i = begin; i < end; ++i) {
                values.push_back(static_cast<uint32_t>(oh.Values[i]));
            }
            offsets.push_back(static_cast<uint32_t>(values.size()));
            srcFlat.push_back(static_cast<uint32_t>(at.FlatIndex));
            srcSplit.push_back(static_cast<uint32_t>(at.Index));
            flags.push_back(dev::kBucketFlagOneHot);
        }
    }
    m.BinarizeBuckets = static_cast<uint32_t>(srcFlat.size());
    CBAMD_ENSURE(m.BinarizeBuckets == trees.CtrFirstBucket, "internal error: bucket count mismatch");
    if (!trees.CtrFeatures.empty()) {
        CBAMD_ENSURE(ctrTables != nullptr, "Model has CTR features but no tables of learned statistics");
        BuildCtrTables(trees, positions, *ctrTables, &srcFlat, &srcSplit, &offsets, &flags, &values, &m.CtrFeatures, &m.CtrItems,
                       &m.CtrIndexBuckets, &m.CtrBlob, &m.CtrCatColumnsFlat, &m.CtrCatColumnsSplit, &m.CtrCatColumnCount);
        m.CtrCount = static_cast<uint32_t>(trees.CtrFeatures.size());
        m.CtrTileUsable = m.CtrCatColumnCount <= dev::kCtrMaxTileColumns && switches.CtrTile;
    }
    CBAMD_ENSURE(srcFlat.size() == BucketCount, "internal error: bucket count mismatch");
    for (size_t b = 0; b + 1 < offsets.size(); ++b) {
        m.MaxBucketValues = std::max(m.MaxBucketValues, offsets[b + 1] - offsets[b]);
    }
    m.HasOneHot = !trees.OneHotFeatures.empty();
    if (m.Oblivious) {
        for (int d : trees.TreeSizes) {
            m.MaxDepth = std::max<uint32_t>(m.MaxDepth, static_cast<uint32_t>(d));
        }
    }
    if (BucketCount == 0) {  // keep the device tables non-empty; the binarize kernel is skipped
        srcFlat.push_back(0);
        srcSplit.push_back(0);
        offsets.push_back(0);
        flags.push_back(0);
    }
    // grid and search window of every float bucket (dev::CountBelowInCell)
    {
        const uint32_t slots = 1u << BinarizeLog2Slots(m.MaxBucketValues);
        const size_t bucketRows = offsets.size() - 1;
        std::vector<uint32_t> grid(bucketRows * 4, 0), lut(bucketRows * (dev::kLutCells / 4), 0);
        for (size_t b = 0; b < bucketRows; ++b) {
            const uint32_t n = offsets[b + 1] - offsets[b];
            if ((flags[b] & dev::kBucketFlagOneHot) || n == 0) {
                continue;
            }
            std::vector<float> borders(n);
            std::memcpy(borders.data(), values.data() + offsets[b], n * sizeof(float));
            const TBucketGrid g = MakeBucketGrid(borders);
            const float lo = g.Lo, scale = g.Scale;
            const uint32_t steps = g.Steps;
            CBAMD_ENSURE((1u << steps) <= slots, "internal error: search window exceeds the bucket's slots");
            uint8_t* cells = reinterpret_cast<uint8_t*>(lut.data() + b * (dev::kLutCells / 4));
            for (int c = 0; c < dev::kLutCells; ++c) {
                // a lower start only adds borders known to be below the value; it keeps the window inside the slots
                cells[c] = static_cast<uint8_t>(std::min(g.Start[c], slots - (1u << steps)));
            }
            std::memcpy(&grid[b * 4 + 0], &lo, 4);
            std::memcpy(&grid[b * 4 + 1], &scale, 4);
            grid[b * 4 + 2] = steps;
        }
        m.BucketGrid.Upload(grid);
        m.BucketLut.Upload(lut);
    }
    m.BucketSrcFlat.Upload(srcFlat);
    m.BucketSrcSplit.Upload(srcSplit);
    m.BucketOffset.Upload(offsets);
    m.BucketFlags.Upload(flags);
    m.Values.Upload(values);

    // ---- tree tables
    std::vector<uint32_t> splits(trees.RepackedBins.size());
    for (size_t i = 0; i < splits.size(); ++i) {
        const auto& rb = trees.RepackedBins[i];
        CBAMD_ENSURE(rb.FeatureIndex < m.LayoutBuckets, "internal error: split refers to a missing bucket");
        splits[i] = static_cast<uint32_t>(rb.FeatureIndex) | (static_cast<uint32_t>(rb.XorMask) << 16) |
                    (static_cast<uint32_t>(rb.SplitIdx) << 24);
    }
    std::vector<uint32_t> treeStart(trees.TreeStartOffsets.begin(), trees.TreeStartOffsets.end());
    std::vector<uint32_t> treeSize(trees.TreeSizes.begin(), trees.TreeSizes.end());
    std::vector<uint32_t> firstLeaf(trees.TreeFirstLeafOffsets.size());
    for (size_t t = 0; t < firstLeaf.size(); ++t) {
        CBAMD_ENSURE(trees.TreeFirstLeafOffsets[t] <= std::numeric_limits<uint32_t>::max(), "model has too many leaf values");
        firstLeaf[t] = static_cast<uint32_t>(trees.TreeFirstLeafOffsets[t]);
    }
    std::vector<uint32_t> steps(trees.NonSymmetricStepNodes.size());
    for (size_t i = 0; i < steps.size(); ++i) {
        steps[i] = static_cast<uint32_t>(trees.NonSymmetricStepNodes[i].LeftSubtreeDiff) |
                   (static_cast<uint32_t>(trees.NonSymmetricStepNodes[i].RightSubtreeDiff) << 16);
    }
    m.Splits.Upload(splits);
    m.TreeStart.Upload(treeStart);
    m.TreeSize.Upload(treeSize);
    m.FirstLeaf.Upload(firstLeaf);
    m.StepNodes.Upload(steps);
    m.NodeToLeaf.Upload(trees.NonSymmetricNodeIdToLeafId);
    {
        // the tile kernel copies (1 << 8) * dim doubles per tree: keep that much readable behind the end
        std::vector<double> padded = trees.LeafValues;
        padded.resize(padded.size() + 256 * static_cast<size_t>(trees.ApproxDimension), 0.0);
        m.Leaves.Upload(padded);
    }
    m.Bias.Upload(trees.Bias);

    // The kernels that keep a tree's row in registers (two trees per wave on half a tile, one on a whole tile)
    // compare 7 bits. Their tile has a row per bucket, and two for a bucket of more than 127 values, which the
    // kernel makes while it copies the bins to LDS (tileMap): min(bin, 127) and max(bin - 127, 0) for a float
    // bucket, the bins up to 127 (0 for the others) and bin - 127 from 128 on (0 for the others) for a one-hot bucket.
    std::vector<uint32_t> tileRowOfBucket(offsets.size(), 0), tileMap;
    const bool tileRowsUsable = true;
    bool tileRowsSplit = false;
    for (size_t b = 0; b + 1 < offsets.size(); ++b) {
        tileRowOfBucket[b] = static_cast<uint32_t>(tileMap.size());
        if (offsets[b + 1] - offsets[b] <= 127) {
            tileMap.push_back(static_cast<uint32_t>(b));
        } else {
            const bool oneHot = (flags[b] & dev::kBucketFlagOneHot) != 0;
            tileMap.push_back(static_cast<uint32_t>(b) | ((oneHot ? dev::kTileMapOneHotLow : dev::kTileMapLow) << 16));
            tileMap.push_back(static_cast<uint32_t>(b) | (dev::kTileMapHigh << 16));
            tileRowsSplit = true;
        }
    }
    const uint32_t tileRowCount = static_cast<uint32_t>(tileMap.size());
    // A level of a tree in those kernels' rows: (row of the tile, xor byte, value added to the four bins, xors)
    struct TTileLevel {
        uint32_t Row, Xor, Add;
        bool IsXor;
    };
    const auto tileLevelOf = [&](const TRepackedBin& rb) {
        TTileLevel level = {tileRowOfBucket[rb.FeatureIndex], 0, 0, false};
        if (rb.XorMask != 0 || rb.SplitIdx == 0xff) {
            // one-hot: bin == value, value = ~XorMask; below 128 seven bits of it are enough, a value from 128 on
            // is looked for as value - 127 in the bucket's second row
            uint32_t value = ~static_cast<uint32_t>(rb.XorMask) & 0xffu;
            if (value > 127 && offsets[rb.FeatureIndex + 1] - offsets[rb.FeatureIndex] > 127) {
                level.Row += 1;
                value -= 127;
            }
            level.Xor = ~value & 0x7fu;
            level.Add = 0x01010101u;
            level.IsXor = true;
        } else if (rb.SplitIdx > 127) {
            level.Row += 1;  // the bucket's second row holds max(bin - 127, 0)
            level.Add = (128u - (rb.SplitIdx - 127u)) * 0x01010101u;
        } else {
            level.Add = (128u - rb.SplitIdx) * 0x01010101u;
        }
        return level;
    };
    // Their rows: 16 dwords per tree, slot d the byte offset of level d's row in the tile | xor byte << 24, slot
    // 8 + d the value added to the four bins of a dword.
    const auto rowsInRegisters = [&](uint32_t bucketBytes) {
        std::vector<uint32_t> rows((trees.GetTreeCount() + dev::kQuadTreePadding) * dev::kPackedTreeDwords, 0);
        for (size_t t = 0; t < trees.GetTreeCount(); ++t) {
            uint32_t* row = rows.data() + t * dev::kPackedTreeDwords;
            bool anyXor = false;
            for (int d = 0; d < trees.TreeSizes[t]; ++d) {
                const TTileLevel level = tileLevelOf(trees.RepackedBins[trees.TreeStartOffsets[t] + d]);
                row[d] = level.Row * bucketBytes | level.Xor << 24;
                row[8 + d] = level.Add;
                anyXor = anyXor || level.IsXor;
            }
            if (anyXor) {
                row[0] |= dev::kPairRowXorFlag;
            }
        }
        return rows;
    };

    // The pair-tile kernel's rows: 8 dwords per tree, a level's row offset (128-byte rows), xor byte (bits 0-6) and
    // the byte added to the bins (bits 24-31) in one dword
    const auto packedPairRows = [&](bool six) {
        constexpr uint32_t kDwords = 8;
        std::vector<uint32_t> rows((trees.GetTreeCount() + dev::kQuadTreePadding) * kDwords, 0);
        for (size_t t = 0; t < trees.GetTreeCount(); ++t) {
            uint32_t* row = rows.data() + t * kDwords;
            bool anyXor = false;
            for (int d = 0; d < trees.TreeSizes[t]; ++d) {
                const TTileLevel level = tileLevelOf(trees.RepackedBins[trees.TreeStartOffsets[t] + d]);
                CBAMD_ENSURE(level.Row < 1024 && level.Xor < 128 && (level.Add & 0xffu) <= 128, "level does not fit the packed row");
                uint32_t xorByte = level.Xor, addByte = level.Add & 0xffu;
                if (six && d % 2 == 0) {
                    // the six-bit form of an even level: its result goes to bit 6 of the byte
                    if (level.IsXor) {
                        xorByte &= 0x3fu;
                    } else {
                        CBAMD_ENSURE(addByte > 64, "split index beyond the six-bit form");
                        addByte -= 64;
                    }
                }
                row[d] = level.Row * 128u | xorByte | addByte << 24;
                anyXor = anyXor || level.IsXor;
            }
            if (anyXor) {
                row[0] |= dev::kPairRowXorFlag;
            }
        }
        return rows;
    };

    // 7-bit compares need every bin and split index to fit 7 bits and no xor mask
    m.PackedSevenBit = m.Oblivious && !m.HasOneHot && m.MaxBucketValues <= 127;
    if (m.Oblivious && m.MaxDepth <= 8) {
        std::vector<uint32_t> packed(trees.GetTreeCount() * dev::kPackedTreeDwords, 0);
        for (size_t t = 0; t < trees.GetTreeCount(); ++t) {
            uint32_t* row = packed.data() + t * dev::kPackedTreeDwords;
            for (int d = 0; d < 8; ++d) {
                if (d < trees.TreeSizes[t]) {
                    const auto& rb = trees.RepackedBins[trees.TreeStartOffsets[t] + d];
                    row[d] = m.PackedSevenBit
                                 ? (static_cast<uint32_t>(rb.FeatureIndex) << 8) | (128u - rb.SplitIdx)
                                 : (static_cast<uint32_t>(rb.FeatureIndex) << 16) |
                                       (static_cast<uint32_t>(rb.XorMask) << 8) | rb.SplitIdx;
                } else {
                    row[d] = m.PackedSevenBit ? 0u : 0xffu;  // a level that is false for every bin
                }
            }
            row[dev::kPackedFirstLeafSlot] = firstLeaf[t];
        }
        if (m.Dim > 1) {
            const size_t pitch = static_cast<size_t>(TileChunk(m.Dim));
            const size_t chunks = (static_cast<size_t>(m.Dim) + pitch - 1) / pitch;
            std::vector<double> padded;
            for (size_t t = 0; t < trees.GetTreeCount(); ++t) {
                const size_t leafCount = size_t(1) << trees.TreeSizes[t];
                CBAMD_ENSURE(padded.size() <= std::numeric_limits<uint32_t>::max(), "model has too many leaf values");
                packed[t * dev::kPackedTreeDwords + dev::kPackedPaddedLeafSlot] = static_cast<uint32_t>(padded.size());
                packed[t * dev::kPackedTreeDwords + dev::kPackedLeafCountSlot] = static_cast<uint32_t>(leafCount);
                const double* values = trees.LeafValues.data() + trees.TreeFirstLeafOffsets[t];
                for (size_t c = 0; c < chunks; ++c) {
                    for (size_t leaf = 0; leaf < leafCount; ++leaf) {
                        for (size_t k = 0; k < pitch; ++k) {
                            const size_t d = c * pitch + k;
                            padded.push_back(d < static_cast<size_t>(m.Dim) ? values[leaf * m.Dim + d] : 0.0);
                        }
                    }
                }
            }
            padded.resize(padded.size() + 256 * pitch, 0.0);  // the kernel copies 256 leaves' worth per tree
            m.LeavesPadded.Upload(padded);
        }
        m.PackedTrees.Upload(packed);
        if (m.Dim == 1) {
            // per-tree form: 7-bit when the tree has no one-hot split and every float bin fits 7 bits
            uint32_t maxFloatValues = 0;
            for (size_t b = 0; b + 1 < offsets.size(); ++b) {
                if (!(flags[b] & dev::kBucketFlagOneHot)) {
                    maxFloatValues = std::max(maxFloatValues, offsets[b + 1] - offsets[b]);
                }
            }
            std::vector<uint32_t> mixed(packed.size(), 0);
            for (size_t t = 0; t < trees.GetTreeCount(); ++t) {
                bool sevenBit = maxFloatValues <= 127;
                for (int d = 0; d < trees.TreeSizes[t]; ++d) {
                    sevenBit = sevenBit && trees.RepackedBins[trees.TreeStartOffsets[t] + d].XorMask == 0;
                }
                uint32_t* row = mixed.data() + t * dev::kPackedTreeDwords;
                for (int d = 0; d < 8; ++d) {
                    if (d < trees.TreeSizes[t]) {
                        const auto& rb = trees.RepackedBins[trees.TreeStartOffsets[t] + d];
                        if (sevenBit) {
                            // ready for use: byte offset of the bucket's row in the half tile, compare constant
                            row[d] = static_cast<uint32_t>(rb.FeatureIndex) * 128u;
                            row[8 + d] = (128u - rb.SplitIdx) * 0x0101u;
                        } else {
                            row[d] = (static_cast<uint32_t>(rb.FeatureIndex) << 16) |
                                     (static_cast<uint32_t>(rb.XorMask) << 8) | rb.SplitIdx;
                        }
                    } else {
                        row[d] = sevenBit ? 0u : 0xffu;  // a split that no bin passes
                    }
                }
                if (!sevenBit) {
                    row[dev::kPackedFormSlot] |= 0x80000000u;
                }
            }
            m.PackedMixed.Upload(mixed);
            if (TileLdsBytes(m.LayoutBuckets, 1) > kMaxTileLdsBytes) {
                const size_t pitch = m.MaxDepth <= 6 ? 64 : 256;
                // zeros at the end: the pair-tile and quad-tile kernels fetch ahead of their trees without a bound
                std::vector<double> fixed((trees.GetTreeCount() + dev::kQuadTreePadding) * pitch, 0.0);
                for (size_t t = 0; t < trees.GetTreeCount(); ++t) {
                    std::copy_n(trees.LeafValues.begin() + trees.TreeFirstLeafOffsets[t], size_t(1) << trees.TreeSizes[t],
                                fixed.begin() + t * pitch);
                }
                m.HalfTileLeaves.Upload(fixed);
                // two trees per wave: every bin of the tile's rows below 128 (the one-hot test then fits 7 bits too)
                const int maxd = m.MaxDepth <= 6 ? 6 : 8;
                const bool pairFits = PairTileLdsBytes(tileRowCount, 8) <= kMaxTileLdsBytes;
                // four trees per wave on a quarter of a block when the rows do not fit the half tile
                const bool quadFits = !pairFits && QuadTileWaves(tileRowCount, maxd) != 0;
                if (switches.PairTile && tileRowsUsable && (pairFits || quadFits)) {
                    if (pairFits) {
                        // every bin below 64: the walk joins two levels at a time
                        m.PairSix = m.MaxBucketValues <= 63 && !tileRowsSplit && switches.RegSix;
                        m.PairRows.Upload(packedPairRows(m.PairSix));
                    } else {
                        m.QuadRows.Upload(rowsInRegisters(64));
                    }
                    m.TileRowCount = tileRowsSplit ? tileRowCount : m.LayoutBuckets;  // (a model without splits: its one zero bucket)
                    if (tileRowsSplit) {
                        m.TileMap.Upload(tileMap);
                    }
                }
            }
        }
        m.LeavesPairAligned = true;
        for (uint32_t f : firstLeaf) {
            m.LeavesPairAligned = m.LeavesPairAligned && (f % 2 == 0);
        }
    }

    if (!m.Oblivious) {
        std::vector<uint32_t> compactEntries, compactRows;
        std::vector<double> valuesByEntry;
        BuildLevelOrderTrees(trees, m.Dim, firstLeaf, &m.NsEntries, &m.NsRows, &m.NsTileUsable, &m.NsNoXor,
                             &compactEntries, &compactRows, &valuesByEntry, &m.NsLdsUsable);
        if (m.NsLdsUsable) {
            // the shape whose units take the least time: more waves hide more of the walk's latency (steps per
            // unit of time relative to 8 waves, measured on 500 trees of about 430 entries: 12 waves 1.26), smaller
            // regions hold fewer trees per unit
            m.NsLdsUsable = false;
            double bestCost = 0.0;
            std::vector<TNsUnit> bestUnits;
            for (const TNsLdsShape& shape : kNsLdsShapes) {
                if ((switches.NsWaves != 0 && switches.NsWaves != shape.Waves) ||
                    NsLdsKernelBytes(m.LayoutBuckets, shape.Waves, shape.Entries, NsLdsDims(m.Dim)) > kMaxTileLdsBytes) {
                    continue;
                }
                std::vector<TNsUnit> plan;
                if (!PackNsUnits(compactRows, TreeCount, shape.Entries, &plan)) {
                    continue;  // a tree larger than a region
                }
                uint64_t steps = 0;
                for (const TNsUnit& unit : plan) {
                    steps += unit.Height;
                }
                const double cost = static_cast<double>(steps) / shape.Speed;
                if (!m.NsLdsUsable || cost < bestCost) {
                    m.NsLdsUsable = true;
                    m.NsLdsShape = shape;
                    bestCost = cost;
                    bestUnits.swap(plan);
                }
            }
            if (m.NsLdsUsable) {
                // the entries in the order of the units; child indexes (bits 21-31) count from the unit's first entry
                std::vector<uint32_t> entries, units;
                std::vector<double> values;
                entries.reserve(compactEntries.size());
                values.reserve(valuesByEntry.size());
                for (const TNsUnit& unit : bestUnits) {
                    // a wave copies a unit sixteen bytes per lane: every unit starts at a multiple of four entries
                    while (entries.size() % 4 != 0) {
                        entries.push_back(255u);
                        values.insert(values.end(), static_cast<size_t>(m.Dim), 0.0);
                    }
                    const uint32_t first = static_cast<uint32_t>(entries.size());
                    uint32_t start[dev::kNsUnitTrees] = {};
                    uint32_t count = 0;
                    for (uint32_t i = 0; i < unit.TreeCount; ++i) {
                        const uint32_t t = unit.Trees[i];
                        const uint32_t treeFirst = compactRows[t * 4], treeEntries = compactRows[t * 4 + 2];
                        start[i] = count;
                        for (uint32_t e = 0; e < treeEntries; ++e) {
                            // the bucket (bits 8-17) becomes the LDS row of its bins in this shape
                            const uint32_t entry = compactEntries[treeFirst + e];
                            const uint32_t tileRow = dev::NsLdsTileRow((entry >> 8) & 0x3ffu, m.NsLdsShape.Waves, m.NsLdsShape.Entries);
                            entries.push_back((entry & ~0x3ff00u) + (tileRow << 8) + (count << 21));
                            const double* value = valuesByEntry.data() + static_cast<size_t>(treeFirst + e) * m.Dim;
                            values.insert(values.end(), value, value + m.Dim);
                        }
                        count += treeEntries;
                    }
                    const uint32_t row[8] = {first, unit.Height, count, start[1], start[2] | (unit.TreeCount << 16),
                                             unit.Trees[0], unit.Trees[1], unit.Trees[2]};
                    units.insert(units.end(), row, row + 8);
                }
                m.NsUnitCount = static_cast<uint32_t>(bestUnits.size());
                m.NsEntryCount = static_cast<uint32_t>(entries.size());
                {
                    // ... in whole regions, whatever the unit's size: spare entries behind the last unit
                    std::vector<uint32_t> padded(entries);
                    padded.resize(entries.size() + m.NsLdsShape.Entries, 255u);
                    m.NsCompactEntries.Upload(padded);
                }
                m.NsCompactRows.Upload(units);
                if (m.Dim > 1) {
                    // [slice of the dimensions][entry][dimension of the slice], zeros past the last dimension
                    const uint32_t dims = NsLdsDims(m.Dim), slices = (static_cast<uint32_t>(m.Dim) + dims - 1) / dims;
                    std::vector<double> bySlice(static_cast<size_t>(slices) * entries.size() * dims, 0.0);
                    for (uint32_t slice = 0; slice < slices; ++slice) {
                        for (size_t e = 0; e < entries.size(); ++e) {
                            for (uint32_t k = 0; k < dims && slice * dims + k < static_cast<uint32_t>(m.Dim); ++k) {
                                bySlice[(slice * entries.size() + e) * dims + k] = values[e * m.Dim + slice * dims + k];
                            }
                        }
                    }
                    values.swap(bySlice);
                }
                m.NsValuesByEntry.Upload(values);
            }
        }
    }

    const bool regEnabled = switches.RegKernel;
    // six-bit form: no one-hot split and no bucket with more than 63 values, so that every bin is below 64
    const bool six = m.PackedSevenBit && m.MaxBucketValues <= 63 && switches.RegSix;
    const TEvalRegVariant* variant =
        m.Oblivious && m.MaxDepth <= kRegMaxDepth && TreeCount > 0
            ? PickRegVariant(m.LayoutBuckets, static_cast<uint32_t>(m.Dim), m.MaxDepth, !m.PackedSevenBit, six,
                             switches.RegMinBuckets)
            : nullptr;
    // bins registers: one per bucket, or two for the buckets of more than 127 values when that keeps a model
    // without xor masks off the 8-bit compare
    std::vector<uint32_t> firstRegOfBucket(offsets.size(), 0), regMap;
    bool regMapped = false;
    uint32_t maxFloatBucketValues = 0;
    for (size_t b = 0; b + 1 < offsets.size(); ++b) {
        if (!(flags[b] & dev::kBucketFlagOneHot)) {
            maxFloatBucketValues = std::max(maxFloatBucketValues, offsets[b + 1] - offsets[b]);
        }
    }
    if (m.Oblivious && m.MaxDepth <= kRegMaxDepth && TreeCount > 0 && maxFloatBucketValues > 127 && switches.RegSplit) {
        for (size_t b = 0; b + 1 < offsets.size(); ++b) {
            firstRegOfBucket[b] = static_cast<uint32_t>(regMap.size());
            if ((flags[b] & dev::kBucketFlagOneHot) || offsets[b + 1] - offsets[b] <= 127) {
                regMap.push_back(static_cast<uint32_t>(b) | (kRegMapAsIs << 16));
            } else {
                regMap.push_back(static_cast<uint32_t>(b) | (kRegMapLow << 16));
                regMap.push_back(static_cast<uint32_t>(b) | (kRegMapHigh << 16));
            }
        }
        // without one-hot splits the model is all 7-bit now; with them the trees that have none are
        const TEvalRegVariant* splitVariant = PickRegVariant(static_cast<uint32_t>(regMap.size()), static_cast<uint32_t>(m.Dim),
                                                             m.MaxDepth, m.HasOneHot, false, switches.RegMinBuckets);
        if (splitVariant != nullptr) {
            variant = splitVariant;
            regMapped = true;
        }
    }
    const uint32_t regCount = regMapped ? static_cast<uint32_t>(regMap.size()) : m.LayoutBuckets;
    // a thread's 32-bit offset walks through the leaf table of a launch while it is copied to LDS
    const bool regTableAddressable =
        variant && (TreeCount / RegTreeBlock(*variant) + 3) * RegTreeBlock(*variant) * variant->Leaves * variant->Pitch * 8 <
                       (uint64_t(1) << 32) - (1u << 20);
    if (regEnabled && variant && regTableAddressable) {
        m.RegModule = SharedRegModule(kEvalRegCodeObject);
        HIP_CHECK(hipModuleGetFunction(&m.RegFunction, m.RegModule, variant->Name));
        m.RegKernelName = variant->Name;
        const uint32_t block = RegTreeBlock(*variant);
        const size_t pitch = variant->Pitch, rowsPerTree = variant->Leaves;
        const size_t rowDwords = variant->Mixed || variant->Leaves > 256 ? 32 : 16;
        const int rowLevels = variant->Leaves > 256 ? 10 : 8;
        m.RegWaves = variant->Waves;
        m.RegRowDwords = static_cast<uint32_t>(rowDwords);
        m.RegTreeBlocks = static_cast<uint32_t>((TreeCount + block - 1) / block);
        // two blocks of null trees behind the last one: the kernels prefetch that far
        const size_t tableTrees = (static_cast<size_t>(m.RegTreeBlocks) + 2) * block;
        const size_t launches = (static_cast<size_t>(m.Dim) + pitch - 1) / pitch;
        m.RegLaunchLeaves = tableTrees * rowsPerTree * pitch;
        // the last launch: the kernel of the same form with the smallest pitch that holds the dimensions left
        const size_t tailFirst = (launches - 1) * pitch, tailDims = static_cast<size_t>(m.Dim) - tailFirst;
        const TEvalRegVariant* tailVariant = nullptr;
        for (const auto& v : kEvalRegVariants) {
            if (m.Dim > 1 && v.Pitch > 1 && v.Pitch >= tailDims && v.Pitch < pitch && v.Leaves == variant->Leaves &&
                v.Mixed == variant->Mixed && v.Six == variant->Six && v.Waves == variant->Waves &&
                regCount <= v.Buckets && (!tailVariant || v.Pitch < tailVariant->Pitch)) {
                tailVariant = &v;
            }
        }
        const uint32_t tailBlock = tailVariant ? RegTreeBlock(*tailVariant) : block;
        const size_t tailPitch = tailVariant ? tailVariant->Pitch : pitch;
        const size_t tailTableTrees = ((TreeCount + tailBlock - 1) / tailBlock + 2) * tailBlock;
        // tree ranges are cut at blocks of the kernel with the larger block (both are powers of two)
        m.RegTreeBlockSize = std::max(block, tailBlock);
        std::vector<uint32_t> rows(std::max(tableTrees, tailTableTrees) * rowDwords, 0);  // 7-bit form (bucket 0, add 0): false for every bin
        std::vector<double> leaves((tailVariant ? launches - 1 : launches) * m.RegLaunchLeaves, 0.0);
        std::vector<double> tailLeaves(tailVariant ? tailTableTrees * rowsPerTree * tailPitch : 0, 0.0);
        // Order of a tree's levels in these tables (levelOrder[t][position] = level of the model). The leaf
        // gathers of a wave meet in the LDS banks that the low bits of the leaf indexes choose; lanes with the
        // same index share one access, lanes that differ only in high bits wait for each other. So the levels
        // that split the documents most evenly go to the low bits and the lopsided ones, on which most lanes
        // agree, to the high bits: fewer lanes of a bank then differ. How evenly a level splits is estimated
        // from the rank of its border among the feature's borders (borders are quantiles of the training data).
        // The leaf tables are permuted to match; the sums and their order do not change.
        std::vector<std::vector<int>> levelOrder(TreeCount);
        for (size_t t = 0; t < TreeCount; ++t) {
            const int depth = trees.TreeSizes[t];
            std::vector<std::pair<double, int>> lopsided;
            for (int d = 0; d < depth; ++d) {
                const auto& rb = trees.RepackedBins[trees.TreeStartOffsets[t] + d];
                const uint32_t n = offsets[rb.FeatureIndex + 1] - offsets[rb.FeatureIndex];
                const bool oneHot = (flags[rb.FeatureIndex] & dev::kBucketFlagOneHot) != 0 || rb.XorMask != 0;
                const double share = oneHot ? 0.05 : static_cast<double>(rb.SplitIdx) / (n + 1.0);
                lopsided.emplace_back(switches.LevelOrder ? std::fabs(share - 0.5) : 0.0, d);
            }
            std::stable_sort(lopsided.begin(), lopsided.end(),
                             [](const auto& a, const auto& b) { return a.first < b.first; });
            for (const auto& item : lopsided) {
                levelOrder[t].push_back(item.second);
            }
        }
        // The register of a level's bins and the split index there: a float bucket that takes two registers answers
        // "bin >= s" in the first for s <= 127 and as "bin - 127 >= s - 127" in the second.
        const auto registerOf = [&](const TRepackedBin& rb) -> std::pair<uint32_t, uint32_t> {
            uint32_t reg = rb.FeatureIndex, splitIdx = rb.SplitIdx;
            if (regMapped) {
                reg = firstRegOfBucket[rb.FeatureIndex];
                if (rb.XorMask == 0 && splitIdx > 127 && !(flags[rb.FeatureIndex] & dev::kBucketFlagOneHot)) {
                    reg += 1;
                    splitIdx -= 127;
                }
            }
            return {reg, splitIdx};
        };
        for (size_t t = 0; t < TreeCount; ++t) {
            const int depth = trees.TreeSizes[t];
            const auto levelAt = [&](int position) -> const TRepackedBin& {
                return trees.RepackedBins[trees.TreeStartOffsets[t] + levelOrder[t][position]];
            };
            // 7-bit form: no xor mask in the tree and every bin of its buckets below 128
            bool sevenBit = true;
            for (int d = 0; d < depth; ++d) {
                const auto& rb = levelAt(d);
                sevenBit = sevenBit && rb.XorMask == 0 &&
                           (regMapped || offsets[rb.FeatureIndex + 1] - offsets[rb.FeatureIndex] <= 127);
            }
            CBAMD_ENSURE(sevenBit || variant->Mixed, "internal error: tree needs the 8-bit compare");
            // a mixed model's bucket 0 may hold bins above 127, which the 7-bit padding level
            // (bucket 0, add 0) would take for true: a tree without levels goes the 8-bit way and
            // the padding levels of the others use the tree's own first bucket
            sevenBit = sevenBit && (depth > 0 || !variant->Mixed);
            uint32_t* row = rows.data() + t * rowDwords;
            if (sevenBit) {
                for (int d = 0; d < depth; ++d) {
                    const auto& rb = levelAt(d);
                    const auto [reg, splitIdx] = registerOf(rb);
                    row[2 * d] = reg;
                    // the level's bit is the carry into bit 7; six-bit kernels want the even levels' in bit 6
                    // (of the first eight levels: levels 8 and 9 of a deep tree are read from bit 7 in every form)
                    row[2 * d + 1] = ((variant->Six && d % 2 == 0 && d < 8 ? 64u : 128u) - splitIdx) * 0x01010101u;
                }
                for (int d = depth; d < rowLevels && depth > 0; ++d) {
                    row[2 * d] = row[0];
                }
            } else {
                for (int d = 0; d < 8; ++d) {
                    // levels past the tree's depth: splitIdx 255, false for every bin (bins are at most 254)
                    uint32_t bucket = 0, xorMask = 0, splitIdx = 255;
                    if (d < depth) {
                        const auto& rb = levelAt(d);
                        std::tie(bucket, splitIdx) = registerOf(rb);
                        xorMask = rb.XorMask;
                    }
                    row[4 * d] = bucket;
                    row[4 * d + 1] = xorMask * 0x01010101u;
                    row[4 * d + 2] = (splitIdx & 0x7fu) * 0x01010101u;
                    row[4 * d + 3] = splitIdx < 128 ? 0x80808080u : 0u;
                }
                row[0] |= 0x80000000u;
            }
            const double* values = trees.LeafValues.data() + trees.TreeFirstLeafOffsets[t];
            for (size_t launch = 0; launch < launches; ++launch) {
                const bool tailTable = tailVariant && launch + 1 == launches;
                const size_t launchPitch = tailTable ? tailPitch : pitch;
                double* table = tailTable ? tailLeaves.data() + t * rowsPerTree * tailPitch
                                          : leaves.data() + launch * m.RegLaunchLeaves + t * rowsPerTree * pitch;
                for (size_t leaf = 0; leaf < (size_t(1) << depth); ++leaf) {
                    // the leaf of the model whose level bits are this table row's position bits
                    size_t modelLeaf = 0;
                    for (int d = 0; d < depth; ++d) {
                        modelLeaf |= ((leaf >> d) & 1) << levelOrder[t][d];
                    }
                    // one-dimensional: a value per leaf; else pieces of two dimensions, 16 bytes per leaf and piece
                    for (size_t k = 0; k < launchPitch && launch * pitch + k < static_cast<size_t>(m.Dim); ++k) {
                        const size_t slot = launchPitch == 1 ? leaf : (k / 2) * rowsPerTree * 2 + leaf * 2 + k % 2;
                        table[slot] = values[modelLeaf * m.Dim + launch * pitch + k];
                    }
                }
            }
        }
        std::vector<double> biasPadded(static_cast<size_t>(m.Dim) + pitch, 0.0);
        std::copy(m.HostBias.begin(), m.HostBias.end(), biasPadded.begin());
        m.RegRows.Upload(rows);
        m.RegLeaves.Upload(leaves);
        m.RegBias.Upload(biasPadded);
        if (tailVariant) {
            m.RegTailLeaves.Upload(tailLeaves);
        }
        if (regMapped) {
            // an entry per register of the largest kernel, in whole batches of sixteen; the spare ones load bucket 0
            regMap.resize((224 + 15) / 16 * 16, 0);
            m.RegMap.Upload(regMap);
        }
        for (size_t launch = 0; launch < launches; ++launch) {
            TImpl::TRegLaunch l;
            l.FirstDim = static_cast<uint32_t>(launch * pitch);
            l.StoreDims = static_cast<uint32_t>(std::min(pitch, static_cast<size_t>(m.Dim) - launch * pitch));
            l.Waves = variant->Waves;
            if (tailVariant && launch + 1 == launches) {
                HIP_CHECK(hipModuleGetFunction(&l.Function, m.RegModule, tailVariant->Name));
                l.Name = tailVariant->Name;
                l.TreeBlock = tailBlock;
                l.TreeLeafDoubles = rowsPerTree * tailPitch;
                l.Leaves = m.RegTailLeaves.Get();
            } else {
                l.Function = m.RegFunction;
                l.Name = variant->Name;
                l.TreeBlock = block;
                l.TreeLeafDoubles = rowsPerTree * pitch;
                l.Leaves = m.RegLeaves.Get() + launch * m.RegLaunchLeaves;
            }
            m.RegLaunches.push_back(l);
        }
        m.RegKernelUsable = true;

        // ---- fused kernels: float-only one-dimensional models in the 7-bit or six-bit form whose rows are
        // at least sixteen columns wide. The bins registers follow the columns of the rows (a unit = sixteen
        // consecutive columns = sixteen registers), so the level rows are rewritten per row layout.
        // Models of the 96-register shape take the fused kernel of 64 or 80 bins registers when their units fit it (112
        // and 128 registers: four waves per SIMD like their evaluate kernel); with more units they stay on two launches
        // (a fused kernel of 96 bins registers would run at three waves per SIMD and is the slower - measured on
        // 50 and 90 buckets). The fused kernels copy 256 leaf rows per tree: a model on the six-level kernel gets
        // a leaf table of that pitch for them (its level rows have the eight slots anyway) and the form of the
        // fused kernel that walks six levels (4M documents x 1000 trees of depth 6 over 70 features: 1.06 ms
        // against 1.15 on two launches; with the eight-level walk 1.19).
        const bool fusedCandidate = switches.Fused && !regMapped && !variant->Mixed && variant->Pitch == 1 && variant->Leaves <= 256 && m.Dim == 1 && !m.HasCats &&
                                    m.CtrCount == 0 && m.BinarizeBuckets == BucketCount && BucketCount > 0 &&
                                    (TreeCount / block + 3) * block * 256 * 8 + 16 * kFusedImageBytes < (uint64_t(1) << 32) - (1u << 20);
        std::vector<double> fusedLeaves;  // 256 rows per tree
        if (fusedCandidate && variant->Leaves == 64) {
            fusedLeaves.assign(tableTrees * 256, 0.0);
            for (size_t t = 0; t < TreeCount; ++t) {
                std::copy(leaves.begin() + t * 64, leaves.begin() + (t + 1) * 64, fusedLeaves.begin() + t * 256);
            }
        }
        const std::vector<double>& fusedLeafTable = variant->Leaves == 64 ? fusedLeaves : leaves;
        for (int layoutIndex = 0; layoutIndex < 2 && fusedCandidate; ++layoutIndex) {
            const std::vector<uint32_t>& columns = layoutIndex == 0 ? srcFlat : srcSplit;
            const size_t rowWidth = layoutIndex == 0 ? m.FlatVectorSize : m.MinFloatSize;
            if (rowWidth < kFusedUnitColumns) {
                continue;
            }
            std::vector<std::pair<uint32_t, uint32_t>> byColumn;  // (column, bucket)
            for (uint32_t b = 0; b < BucketCount; ++b) {
                byColumn.emplace_back(columns[b], b);
            }
            std::sort(byColumn.begin(), byColumn.end());
            bool distinct = true;
            for (size_t i = 1; i < byColumn.size(); ++i) {
                distinct = distinct && byColumn[i].first != byColumn[i - 1].first;
            }
            if (!distinct) {
                continue;
            }
            // units: sixteen columns from a used column on, moved back where they would leave the row
            std::vector<uint32_t> unitStart, slotOfBucket(BucketCount, 0);
            for (size_t i = 0; i < byColumn.size();) {
                const uint32_t start = static_cast<uint32_t>(std::min<size_t>(byColumn[i].first, rowWidth - kFusedUnitColumns));
                const uint32_t unit = static_cast<uint32_t>(unitStart.size());
                unitStart.push_back(start);
                while (i < byColumn.size() && byColumn[i].first < start + kFusedUnitColumns) {
                    slotOfBucket[byColumn[i].second] = unit * kFusedUnitColumns + (byColumn[i].first - start);
                    ++i;
                }
            }
            const TFusedVariant* fused = nullptr;
            for (const auto& v : kFusedVariants) {
                // (the wide fused shape is for the models of the wide evaluate kernels)
                if (v.Six == variant->Six && unitStart.size() * kFusedUnitColumns <= v.Buckets && !fused &&
                    (variant->Waves == 4 || v.Buckets <= 80) && m.MaxDepth <= v.Levels) {
                    fused = &v;
                }
            }
            if (!fused || (m.FusedFunction && m.FusedWaves != fused->Waves)) {
                continue;
            }
            const uint32_t slots = fused->Six ? 64 : 128;           // border slots of a bucket in an image
            const uint32_t bucketsPerImage = fused->Six ? 64 : 32;
            const uint32_t unitsPerImage = bucketsPerImage / kFusedUnitColumns;
            const uint32_t maxUnits = fused->Buckets / kFusedUnitColumns;
            uint32_t images = (fused->Buckets + bucketsPerImage - 1) / bucketsPerImage;
            images += images % 2;
            std::vector<uint32_t> bucketOfSlot(fused->Buckets, UINT32_MAX);
            for (uint32_t b = 0; b < BucketCount; ++b) {
                bucketOfSlot[slotOfBucket[b]] = b;
            }
            // grids first: the four columns of a load share their number of search steps
            std::vector<TBucketGrid> grids(fused->Buckets);
            std::vector<std::vector<float>> bordersOfSlot(fused->Buckets);
            std::vector<uint32_t> groupSteps(fused->Buckets / 4, 1);
            bool fits = true;
            for (uint32_t slot = 0; slot < fused->Buckets; ++slot) {
                const uint32_t b = bucketOfSlot[slot];
                if (b == UINT32_MAX) {
                    continue;
                }
                const uint32_t n = offsets[b + 1] - offsets[b];
                bordersOfSlot[slot].resize(n);
                std::memcpy(bordersOfSlot[slot].data(), values.data() + offsets[b], n * sizeof(float));
                grids[slot] = MakeBucketGrid(bordersOfSlot[slot]);
                groupSteps[slot / 4] = std::max(groupSteps[slot / 4], grids[slot].Steps);
                fits = fits && n < slots;
            }
            for (uint32_t steps : groupSteps) {
                fits = fits && steps <= kFusedMaxSteps && (1u << steps) <= slots;
            }
            if (!fits) {
                continue;
            }
            // the records of all units the kernel has code for, one more, and the units' byte offsets in a row
            std::vector<uint32_t> units((static_cast<size_t>(maxUnits) + 1) * kFusedUnitDwords + 16, 0);
            for (size_t u = 0; u < unitStart.size(); ++u) {
                units[(static_cast<size_t>(maxUnits) + 1) * kFusedUnitDwords + u] = unitStart[u] * 4;
            }
            std::vector<uint8_t> table(images * kFusedImageBytes + fusedLeafTable.size() * sizeof(double), 0);
            for (uint32_t slot = 0; slot < fused->Buckets; ++slot) {
                const uint32_t unit = slot / kFusedUnitColumns, column = slot % kFusedUnitColumns;
                uint32_t* record = units.data() + static_cast<size_t>(unit) * kFusedUnitDwords;
                const uint32_t steps = groupSteps[slot / 4], group = column / 4;
                record[32] |= (steps >= 4 ? 1u << group : 0u) | (steps >= 3 ? 16u << group : 0u) | (steps >= 2 ? 256u << group : 0u);
                const uint32_t b = bucketOfSlot[slot];
                if (b == UINT32_MAX) {
                    continue;  // a column no split reads: all-zero record and tables, its register is never indexed
                }
                std::memcpy(&record[column], &grids[slot].Lo, 4);
                std::memcpy(&record[16 + column], &grids[slot].Scale, 4);
                if (flags[b] & dev::kBucketFlagNanToInf) {
                    record[32] |= 0x10000u << column;
                }
                uint8_t* image = table.data() + (unit / unitsPerImage) * kFusedImageBytes;
                const uint32_t local = (unit % unitsPerImage) * kFusedUnitColumns + column;
                uint32_t* borders = reinterpret_cast<uint32_t*>(image + static_cast<size_t>(local) * slots * 4);
                for (uint32_t k = 0; k < slots; ++k) {
                    uint32_t bits = 0x7f800000u;  // +inf behind the real borders
                    if (k < bordersOfSlot[slot].size()) {
                        std::memcpy(&bits, &bordersOfSlot[slot][k], 4);
                    }
                    borders[k] = bits;
                }
                uint8_t* lut = image + kFusedLutOffset + static_cast<size_t>(local) * dev::kLutCells;
                for (int c = 0; c < dev::kLutCells; ++c) {
                    const uint32_t start = std::min(grids[slot].Start[c], slots - (1u << steps));
                    lut[c] = static_cast<uint8_t>(fused->Six ? start * 4 : start);  // the six-bit form stores byte offsets
                }
            }
            std::memcpy(table.data() + images * kFusedImageBytes, fusedLeafTable.data(), fusedLeafTable.size() * sizeof(double));
            // level rows of the same form as the register kernel's, naming bins registers of this layout
            std::vector<uint32_t> fusedRows(rows);
            for (size_t t = 0; t < TreeCount; ++t) {
                const int depth = trees.TreeSizes[t];
                uint32_t* row = fusedRows.data() + t * rowDwords;
                for (int d = 0; d < depth; ++d) {
                    row[2 * d] = slotOfBucket[trees.RepackedBins[trees.TreeStartOffsets[t] + levelOrder[t][d]].FeatureIndex];
                }
                for (int d = depth; d < 8 && depth > 0; ++d) {
                    row[2 * d] = row[0];
                }
            }
            if (!m.FusedFunction) {
                HIP_CHECK(hipModuleGetFunction(&m.FusedFunction, m.RegModule, fused->Name));
                m.FusedWaves = fused->Waves;
                m.FusedKernelName = fused->Name;
            }
            TImpl::TFused& f = m.Fused[layoutIndex];
            f.UnitCount = static_cast<uint32_t>(unitStart.size());
            f.Rows.Upload(fusedRows);
            f.Units.Upload(units);
            f.Table.Upload(table);
            f.Usable = true;
        }
    }

    // Models that the register kernels do not take, every bin of the tile's rows below 128, the 256-document tile and the leaf
    // regions of eight waves in LDS: a tree's row in registers (EvalObliviousRowTileKernel).
    if (!m.RegKernelUsable && m.Oblivious && m.MaxDepth <= 8 && TreeCount > 0 && switches.RowTile && tileRowsUsable &&
        RowTileWaves(tileRowCount, m.MaxDepth, m.Dim) != 0) {
        const size_t leavesPerTree = m.MaxDepth <= 6 ? 64 : 256;
        const size_t dims = RowTileDims(m.MaxDepth, m.Dim), slices = (static_cast<size_t>(m.Dim) + dims - 1) / dims;
        const size_t tableTrees = TreeCount + dev::kPairTreePadding;  // zeros at the end: the kernel fetches ahead of its trees
        std::vector<double> values(slices * tableTrees * leavesPerTree * dims, 0.0);
        for (size_t t = 0; t < TreeCount; ++t) {
            const double* leaf = trees.LeafValues.data() + trees.TreeFirstLeafOffsets[t];
            for (size_t l = 0; l < (size_t(1) << trees.TreeSizes[t]); ++l) {
                for (size_t d = 0; d < static_cast<size_t>(m.Dim); ++d) {
                    // [slice][tree][pair of dimensions][leaf][dimension of the pair]; one dimension: [tree][leaf]
                    const size_t slice = d / dims, k = d % dims;
                    const size_t slot = dims == 1 ? l : ((k / 2) * leavesPerTree + l) * 2 + k % 2;
                    values[(slice * tableTrees + t) * leavesPerTree * dims + slot] = leaf[l * m.Dim + d];
                }
            }
        }
        m.TileLeaves.Upload(values);
        m.TileSliceStride = tableTrees * leavesPerTree * dims / 2;
        m.TileRows.Upload(rowsInRegisters(256));
        m.TileRowCount = tileRowsSplit ? tileRowCount : m.LayoutBuckets;  // (a model without splits: its one zero bucket)
        if (tileRowsSplit) {
            m.TileMap.Upload(tileMap);
        }
    }

    // Models of depth 9 to 16 that the register kernels do not take (deeper than 10, one-hot splits, several
    // dimensions, more registers than they have): the same tile, a tree's levels in two halves of eight, leaf values
    // gathered from the model's own table, two dimensions per walk (EvalObliviousDeepTileKernel).
    if (!m.RegKernelUsable && m.Oblivious && m.MaxDepth > 8 && m.MaxDepth <= 16 && TreeCount > 0 &&
        switches.RowTile && tileRowsUsable &&
        DeepTileLdsBytes(tileRowsSplit ? tileRowCount : m.LayoutBuckets, DeepTileDims(m.Dim)) <= kMaxTileLdsBytes) {
        const size_t tableTrees = TreeCount + dev::kPairTreePadding;
        std::vector<uint32_t> rows(tableTrees * 32, 0), first(tableTrees, 0);
        for (size_t t = 0; t < TreeCount; ++t) {
            uint32_t* row = rows.data() + t * 32;
            bool anyXor = false;
            for (int d = 0; d < trees.TreeSizes[t]; ++d) {
                const TTileLevel level = tileLevelOf(trees.RepackedBins[trees.TreeStartOffsets[t] + d]);
                uint32_t* half = row + (d < 8 ? 0 : 16);
                const int slot = d % 8;
                half[slot] = level.Row * 256u | level.Xor << 24;
                half[8 + slot] = level.Add;
                anyXor = anyXor || level.IsXor;
            }
            if (anyXor) {
                row[0] |= dev::kPairRowXorFlag;
            }
            first[t] = firstLeaf[t];
        }
        if (m.Dim > 1) {
            // two dimensions of a leaf side by side, slice after slice
            const size_t dim = static_cast<size_t>(m.Dim), slices = (dim + 1) / 2;
            size_t leafCount = 0;
            for (size_t t = 0; t < TreeCount; ++t) {
                first[t] = static_cast<uint32_t>(leafCount);
                leafCount += size_t(1) << trees.TreeSizes[t];
            }
            CBAMD_ENSURE(leafCount < (size_t(1) << 31), "too many leaves for the deep-tile kernel");
            std::vector<double> pairs(slices * leafCount * 2, 0.0);
            for (size_t t = 0; t < TreeCount; ++t) {
                const double* values = trees.LeafValues.data() + trees.TreeFirstLeafOffsets[t];
                for (size_t leaf = 0; leaf < (size_t(1) << trees.TreeSizes[t]); ++leaf) {
                    for (size_t k = 0; k < dim; ++k) {
                        pairs[((k / 2) * leafCount + first[t] + leaf) * 2 + k % 2] = values[leaf * dim + k];
                    }
                }
            }
            m.DeepLeaves.Upload(pairs);
            m.DeepSliceLeaves = static_cast<uint32_t>(leafCount);
        }
        m.DeepRows.Upload(rows);
        m.DeepFirstLeaf.Upload(first);
        m.TileRowCount = tileRowsSplit ? tileRowCount : m.LayoutBuckets;
        if (tileRowsSplit) {
            m.TileMap.Upload(tileMap);
        }
    }
}

THipEvaluator::~THipEvaluator() = default;

size_t THipEvaluator::QuantizedBytes(size_t docCount) const {
    const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
    return std::max<size_t>(blocks, 1) * Impl->LayoutBuckets * dev::kDocsPerBlock;
}

void THipEvaluator::Synchronize(void* stream) {
    HIP_CHECK(hipStreamSynchronize(Impl->Pick(stream)));
}

namespace {

constexpr uint32_t kBinarizeBlocksPerGroup = 8;

template <int LOG2P, bool CATS_MATRIX>
void LaunchBinarizeRowsPC(size_t blocks, const float* floats, size_t stride, const int32_t* cats, size_t catStride,
                          size_t docCount, const dev::TBinarizeTables& tab, uint32_t* bins, hipStream_t s) {
    const size_t tiles = (tab.BucketCount + dev::kBucketTile - 1) / dev::kBucketTile;
    // a workgroup keeps its tile's borders in LDS over up to kBinarizeBlocksPerGroup document blocks; a small
    // batch gives each fewer blocks, so that there are still about a thousand workgroups
    const uint32_t blocksPerGroup = static_cast<uint32_t>(
        std::max<size_t>(1, std::min<size_t>(kBinarizeBlocksPerGroup, blocks * tiles / 1024)));
    const size_t groups = (blocks + blocksPerGroup - 1) / blocksPerGroup;
    CBAMD_ENSURE(groups * tiles < (size_t(1) << 31), "batch is too large for one binarize launch");
    const dim3 grid(static_cast<uint32_t>(groups * tiles));
    const size_t lds = (static_cast<size_t>(dev::kBucketTile) << LOG2P) * 4 +
                       static_cast<size_t>(dev::kBucketTile) * dev::kLutCells +
                       static_cast<size_t>(dev::kBucketTile) * dev::kTilePitch * 4;
    auto kernel = dev::BinarizeRowsKernel<LOG2P, CATS_MATRIX>;
    EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds, s, floats, static_cast<uint32_t>(stride), cats,
                       static_cast<uint32_t>(catStride), static_cast<uint32_t>(docCount), tab, blocksPerGroup, bins);
}

template <int LOG2P>
void LaunchBinarizeRowsP(size_t blocks, const float* floats, size_t stride, const int32_t* cats, size_t catStride,
                         size_t docCount, const dev::TBinarizeTables& tab, uint32_t* bins, hipStream_t s) {
    if (cats != nullptr) {
        LaunchBinarizeRowsPC<LOG2P, true>(blocks, floats, stride, cats, catStride, docCount, tab, bins, s);
    } else {
        LaunchBinarizeRowsPC<LOG2P, false>(blocks, floats, stride, cats, catStride, docCount, tab, bins, s);
    }
}

// picks the smallest LDS slot count that still exceeds the largest bucket of the model
void LaunchBinarizeRows(uint32_t maxBucketValues, size_t blocks, const float* floats, size_t stride,
                        const int32_t* cats, size_t catStride, size_t docCount, const dev::TBinarizeTables& tab,
                        uint32_t* bins, hipStream_t s) {
    CBAMD_ENSURE(docCount < (size_t(1) << 31) && stride < (size_t(1) << 31) && catStride < (size_t(1) << 31),
                 "batch is too large for one binarize launch");
    if (tab.BucketCount == 0) {
        return;  // a model of CTR features only
    }
    const int log2Slots = BinarizeLog2Slots(maxBucketValues);
    if (log2Slots == 5) {
        LaunchBinarizeRowsP<5>(blocks, floats, stride, cats, catStride, docCount, tab, bins, s);
    } else if (log2Slots == 6) {
        LaunchBinarizeRowsP<6>(blocks, floats, stride, cats, catStride, docCount, tab, bins, s);
    } else if (log2Slots == 7) {
        LaunchBinarizeRowsP<7>(blocks, floats, stride, cats, catStride, docCount, tab, bins, s);
    } else {
        LaunchBinarizeRowsP<8>(blocks, floats, stride, cats, catStride, docCount, tab, bins, s);
    }
}

template <int LOG2P>
void LaunchBinarizeColumnsP(size_t blocks, const float* floats, size_t stride, size_t docCount,
                            const dev::TBinarizeTables& tab, uint32_t* bins, hipStream_t s) {
    const size_t tiles = (tab.BucketCount + dev::kBucketTile - 1) / dev::kBucketTile;
    const uint32_t blocksPerGroup = static_cast<uint32_t>(
        std::max<size_t>(1, std::min<size_t>(kBinarizeBlocksPerGroup, blocks * tiles / 1024)));
    const size_t groups = (blocks + blocksPerGroup - 1) / blocksPerGroup;
    CBAMD_ENSURE(groups * tiles < (size_t(1) << 31), "batch is too large for one binarize launch");
    const size_t lds = (static_cast<size_t>(dev::kBucketTile) << LOG2P) * 4 +
                       static_cast<size_t>(dev::kBucketTile) * dev::kLutCells;
    auto kernel = dev::BinarizeColumnsKernel<LOG2P>;
    EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
    hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(groups * tiles)), dim3(256), lds, s, floats, stride,
                       static_cast<uint32_t>(docCount), tab, blocksPerGroup, bins);
}

// column-major documents: the same choice of LDS slots as for rows
void LaunchBinarizeColumns(uint32_t maxBucketValues, size_t blocks, const float* floats, size_t stride,
                           size_t docCount, const dev::TBinarizeTables& tab, uint32_t* bins, hipStream_t s) {
    CBAMD_ENSURE(docCount < (size_t(1) << 31), "batch is too large for one binarize launch");
    const int log2Slots = BinarizeLog2Slots(maxBucketValues);
    if (log2Slots == 5) {
        LaunchBinarizeColumnsP<5>(blocks, floats, stride, docCount, tab, bins, s);
    } else if (log2Slots == 6) {
        LaunchBinarizeColumnsP<6>(blocks, floats, stride, docCount, tab, bins, s);
    } else if (log2Slots == 7) {
        LaunchBinarizeColumnsP<7>(blocks, floats, stride, docCount, tab, bins, s);
    } else {
        LaunchBinarizeColumnsP<8>(blocks, floats, stride, docCount, tab, bins, s);
    }
}

}  // namespace

void THipEvaluator::QuantizeDevice(const TFeatureBatch& batch, size_t docCount, uint8_t* bins, void* stream) {
    TImpl& m = *Impl;
    if (docCount == 0) {
        return;
    }
    hipStream_t s = m.Pick(stream);
    const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
    CBAMD_ENSURE(blocks <= 0x7fffffffu, "too many documents in one batch");
    if (m.RealBucketCount == 0) {
        // a model without splits: one all-zero bucket per block keeps the layout non-empty
        CBAMD_ENSURE(bins != nullptr, "quantized buffer is null");
        const size_t dwords = QuantizedBytes(docCount) / 4;
        hipLaunchKernelGGL(dev::FillZeroKernel, dim3(static_cast<uint32_t>(std::min<size_t>((dwords + 255) / 256, 4096))),
                           dim3(256), 0, s, reinterpret_cast<uint32_t*>(bins), dwords);
        HIP_CHECK(hipGetLastError());
        return;
    }
    CBAMD_ENSURE(bins != nullptr, "quantized buffer is null");
    CBAMD_ENSURE(batch.Floats != nullptr || (batch.Layout == TFeatureBatch::SplitRows && m.MinFloatSize == 0),
                 "float features pointer is null");
    switch (batch.Layout) {
        case TFeatureBatch::FlatRows: {
            CBAMD_ENSURE(batch.Stride >= m.FlatVectorSize, "insufficient flat features vector size: " +
                                                                std::to_string(batch.Stride) + " expected: " +
                                                                std::to_string(m.FlatVectorSize));
            LaunchBinarizeRows(m.MaxBucketValues, blocks, batch.Floats, batch.Stride, nullptr, 0, docCount,
                               m.BinarizeTables(true), reinterpret_cast<uint32_t*>(bins), s);
            break;
        }
        case TFeatureBatch::SplitRows: {
            CBAMD_ENSURE(batch.Stride >= m.MinFloatSize, "insufficient float features vector size: " +
                                                             std::to_string(batch.Stride) + " expected: " +
                                                             std::to_string(m.MinFloatSize));
            if (m.HasCats) {
                CBAMD_ENSURE(batch.Cats != nullptr, "Model has categorical features but no categorical features provided");
                CBAMD_ENSURE(batch.CatStride >= m.MinCatSize, "insufficient cat features vector size: " +
                                                                  std::to_string(batch.CatStride) + " expected: " +
                                                                  std::to_string(m.MinCatSize));
            }
            // a model with one-hot buckets always reads them from the categorical matrix here
            LaunchBinarizeRows(m.MaxBucketValues, blocks, batch.Floats, batch.Stride, m.HasCats ? batch.Cats : nullptr,
                               batch.CatStride, docCount, m.BinarizeTables(false), reinterpret_cast<uint32_t*>(bins), s);
            break;
        }
        case TFeatureBatch::FlatColumns: {
            CBAMD_ENSURE(batch.Stride >= docCount, "column stride is shorter than the document count");
            if (m.BinarizeBuckets > 0) {
                LaunchBinarizeColumns(m.MaxBucketValues, blocks, batch.Floats, batch.Stride, docCount,
                                      m.BinarizeTables(true), reinterpret_cast<uint32_t*>(bins), s);
            }
            break;
        }
        default:
            CBAMD_ENSURE(false, "unknown feature layout");
    }
    HIP_CHECK(hipGetLastError());
    if (m.CtrCount > 0) {
        // the CTR features read the bins written above and the hashed categorical values
        dev::TCatSource cats;
        cats.SplitColumns = batch.Layout == TFeatureBatch::SplitRows ? 1u : 0u;
        if (batch.Layout == TFeatureBatch::SplitRows) {
            cats.Base = reinterpret_cast<const uint32_t*>(batch.Cats);
            cats.DocStride = batch.CatStride;
            cats.ColumnStride = 1;
        } else if (batch.Layout == TFeatureBatch::FlatRows) {
            cats.Base = reinterpret_cast<const uint32_t*>(batch.Floats);
            cats.DocStride = batch.Stride;
            cats.ColumnStride = 1;
        } else {
            cats.Base = reinterpret_cast<const uint32_t*>(batch.Floats);
            cats.DocStride = 1;
            cats.ColumnStride = batch.Stride;
        }
        CBAMD_ENSURE(m.CtrCount <= 65535, "too many CTR features for one launch");
        const dev::TBinarizeTables tab = m.BinarizeTables(batch.Layout != TFeatureBatch::SplitRows);
        if (m.CtrTileUsable) {
            const dim3 grid(static_cast<uint32_t>(blocks), (m.CtrCount + dev::kCtrGroup - 1) / dev::kCtrGroup);
            const size_t lds = static_cast<size_t>(std::max<uint32_t>(m.CtrCatColumnCount, 1)) * dev::kCtrTilePitch * 4;
            hipLaunchKernelGGL(dev::CtrBinarizeTileKernel, grid, dim3(256), lds, s, cats, static_cast<uint32_t>(docCount),
                               m.CtrTables(), tab, reinterpret_cast<uint32_t*>(bins));
        } else {
            const dim3 grid(static_cast<uint32_t>(blocks), m.CtrCount);
            hipLaunchKernelGGL(dev::CtrBinarizeKernel, grid, dim3(64), 0, s, cats, static_cast<uint32_t>(docCount),
                               m.CtrTables(), tab, reinterpret_cast<uint32_t*>(bins));
        }
        HIP_CHECK(hipGetLastError());
    }
}

namespace {


// LDS of the half-tile kernel: 128 documents' bins, the accumulator, the per-wave leaf regions
size_t HalfTileLdsBytes(uint32_t buckets, int maxd) {
    return ((static_cast<size_t>(buckets) * 128 + 7) & ~size_t(7)) + 128 * sizeof(double) +
           static_cast<size_t>(dev::kTileWaves) * (size_t(1) << maxd) * sizeof(double);
}

// LDS of the per-wave leaf regions of the tile kernel
size_t TileLeafLdsBytes(int maxd, int dchunk, int waves = dev::kTileWaves) {
    return static_cast<size_t>(waves) * (size_t(1) << maxd) * dchunk * sizeof(double);
}

struct TTileArgs {
    const uint8_t* Bins;
    size_t DocCount;
    uint32_t Buckets;
    const uint32_t* PackedTrees;
    const double* Leaves;
    const double* Bias;
    double Scale;
    int Dim;
    uint32_t TreeBegin, TreeEnd;
    double* Out;
    hipStream_t Stream;
    bool LeavesPairAligned;
};

template <bool SEVEN_BIT, int MAXD, int DCHUNK, bool LEAF_LDS, int WAVES>
void LaunchEvalTileW(const TTileArgs& a) {
    const size_t blocks = (a.DocCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
    const size_t lds = TileLdsBytes(a.Buckets, DCHUNK) + (LEAF_LDS ? TileLeafLdsBytes(MAXD, DCHUNK, WAVES) : 0);
    auto kernel = dev::EvalObliviousTileKernel<SEVEN_BIT, MAXD, DCHUNK, LEAF_LDS, WAVES>;
    EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
    hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(blocks)), dim3(64 * WAVES), lds, a.Stream,
                       reinterpret_cast<const uint32_t*>(a.Bins), a.DocCount, a.Buckets, a.PackedTrees, a.Leaves, a.Bias,
                       a.Scale, a.Dim, a.TreeBegin, a.TreeEnd, a.Out);
}

template <bool SEVEN_BIT, int MAXD, int DCHUNK, bool LEAF_LDS>
void LaunchEvalTileL(const TTileArgs& a) {
    // a tile of which only one workgroup fits a CU gets sixteen waves instead of eight, LDS permitting
    const size_t narrow = TileLdsBytes(a.Buckets, DCHUNK) + (LEAF_LDS ? TileLeafLdsBytes(MAXD, DCHUNK) : 0);
    const size_t wide = TileLdsBytes(a.Buckets, DCHUNK) + (LEAF_LDS ? TileLeafLdsBytes(MAXD, DCHUNK, dev::kWideTileWaves) : 0);
    if (2 * narrow > kMaxTileLdsBytes && wide <= kMaxTileLdsBytes) {
        LaunchEvalTileW<SEVEN_BIT, MAXD, DCHUNK, LEAF_LDS, dev::kWideTileWaves>(a);
    } else {
        LaunchEvalTileW<SEVEN_BIT, MAXD, DCHUNK, LEAF_LDS, dev::kTileWaves>(a);
    }
}

template <bool SEVEN_BIT, int MAXD, int DCHUNK>
void LaunchEvalTile(const TTileArgs& a) {
    // leaf values go through LDS whenever the tile, the accumulator and the per-wave leaf regions
    // fit the 160 KB of a CU (gathers from global memory cost ~50 L1 accesses per wave instruction)
    const size_t withLeaves = TileLdsBytes(a.Buckets, DCHUNK) + TileLeafLdsBytes(MAXD, DCHUNK);
    if (a.LeavesPairAligned && withLeaves <= kMaxTileLdsBytes) {
        LaunchEvalTileL<SEVEN_BIT, MAXD, DCHUNK, true>(a);
    } else {
        LaunchEvalTileL<SEVEN_BIT, MAXD, DCHUNK, false>(a);
    }
}

template <bool SEVEN_BIT, int MAXD>
void LaunchEvalTileD(int dchunk, const TTileArgs& a) {
    switch (dchunk) {
        case 1: LaunchEvalTile<SEVEN_BIT, MAXD, 1>(a); break;
        case 2: LaunchEvalTile<SEVEN_BIT, MAXD, 2>(a); break;
        case 4: LaunchEvalTile<SEVEN_BIT, MAXD, 4>(a); break;
        case 8: LaunchEvalTile<SEVEN_BIT, MAXD, 8>(a); break;
        case 12: LaunchEvalTile<SEVEN_BIT, MAXD, 12>(a); break;
        default: LaunchEvalTile<SEVEN_BIT, MAXD, 16>(a); break;
    }
}

template <bool SEVEN_BIT>
void LaunchEvalTileM(uint32_t maxDepth, int dchunk, const TTileArgs& a) {
    if (maxDepth <= 4) {
        LaunchEvalTileD<SEVEN_BIT, 4>(dchunk, a);
    } else if (maxDepth <= 6) {
        LaunchEvalTileD<SEVEN_BIT, 6>(dchunk, a);
    } else {
        LaunchEvalTileD<SEVEN_BIT, 8>(dchunk, a);
    }
}

template <bool NO_XOR, int DCHUNK>
void LaunchEvalNonSymmetricTileX(const uint8_t* bins, size_t docCount, uint32_t buckets, const uint2* entries,
                                 const uint4* rows, const double* leaves, const double* bias, double scale, int dim,
                                 uint32_t treeBegin, uint32_t treeEnd, double* out, hipStream_t s) {
    const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
    const size_t lds = TileLdsBytes(buckets, DCHUNK);
    auto kernel = dev::EvalNonSymmetricTileKernel<NO_XOR, DCHUNK>;
    EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
    hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(blocks)), dim3(64 * dev::kTileWaves), lds, s,
                       reinterpret_cast<const uint32_t*>(bins), docCount, buckets, entries, rows, leaves, bias, scale, dim,
                       treeBegin, treeEnd, out);
}

template <typename... TArgs>
void LaunchEvalNonSymmetricTile(bool noXor, int dchunk, TArgs... args) {
    if (noXor) {
        switch (dchunk) {
            case 1: LaunchEvalNonSymmetricTileX<true, 1>(args...); break;
            case 4: LaunchEvalNonSymmetricTileX<true, 4>(args...); break;
            default: LaunchEvalNonSymmetricTileX<true, 16>(args...); break;
        }
    } else {
        switch (dchunk) {
            case 1: LaunchEvalNonSymmetricTileX<false, 1>(args...); break;
            case 4: LaunchEvalNonSymmetricTileX<false, 4>(args...); break;
            default: LaunchEvalNonSymmetricTileX<false, 16>(args...); break;
        }
    }
}

template <int DCHUNK>
void LaunchEval(bool oblivious, const uint8_t* bins, size_t docCount, uint32_t buckets, const dev::TTreeTables& tt,
                uint32_t treeBegin, uint32_t treeEnd, double* out, hipStream_t s) {
    const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
    if (oblivious) {
        const uint32_t grid = static_cast<uint32_t>((blocks + 3) / 4);
        hipLaunchKernelGGL(dev::EvalObliviousKernel<DCHUNK>, dim3(grid), dim3(256), 0, s,
                           reinterpret_cast<const uint32_t*>(bins), docCount, buckets, tt, treeBegin, treeEnd, out, 0u, 2u);
    } else {
        hipLaunchKernelGGL(dev::EvalNonSymmetricKernel<DCHUNK>, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s,
                           bins, docCount, buckets, tt, treeBegin, treeEnd, out);
    }
}

}  // namespace

void THipEvaluator::EvalQuantizedDevice(const uint8_t* bins, size_t docCount, size_t treeStart, size_t treeEnd,
                                        double* results, void* stream) {
    TImpl& m = *Impl;
    if (docCount == 0) {
        return;
    }
    hipStream_t s = m.Pick(stream);
    CBAMD_ENSURE(results != nullptr, "results pointer is null");
    if (TreeCount == 0) {
        // a model without trees answers with its bias (cpu/formula_evaluator.cpp:29-41)
        const size_t count = docCount * m.Dim;
        hipLaunchKernelGGL(dev::FillBiasKernel, dim3(static_cast<uint32_t>((count + 255) / 256)), dim3(256), 0, s, results,
                           count, m.Bias.Get(), m.Dim);
        HIP_CHECK(hipGetLastError());
        return;
    }
    CBAMD_ENSURE(treeStart <= treeEnd && treeEnd <= TreeCount, "tree range is out of bounds");
    CBAMD_ENSURE(bins != nullptr, "quantized buffer is null");
    const dev::TTreeTables tt = m.TreeTables();
    const uint32_t tb = static_cast<uint32_t>(treeStart), te = static_cast<uint32_t>(treeEnd);
    if (m.RegKernelUsable) {
        // Bins kept in registers, a launch per group of dimensions (RegLaunches). A launch addresses its results with 32
        // bits, so a very large batch goes in slices of whole document blocks.
        const size_t sliceDocs = ((size_t(1) << 29) - 1) / m.Dim / dev::kDocsPerBlock * dev::kDocsPerBlock;
        if (docCount > sliceDocs) {
            for (size_t first = 0; first < docCount; first += sliceDocs) {
                const size_t n = std::min(sliceDocs, docCount - first);
                EvalQuantizedDevice(bins + first * m.LayoutBuckets, n, treeStart, treeEnd, results + first * m.Dim, stream);
            }
            return;
        }
        // The kernels walk whole blocks of RegTreeBlock trees. A range that starts or ends inside a block has
        // those few trees evaluated by the kernel that follows the model's own tables, before and after the
        // whole blocks: the launches hand on raw sums, each adds its trees in tree order, so the result is the
        // same sequence of additions as one pass over the range.
        const uint32_t block = m.RegTreeBlockSize;
        const uint32_t wholeBegin = (tb + block - 1) / block * block;
        const uint32_t wholeEnd = te == TreeCount ? te : te / block * block;  // null trees pad the model's last block
        const bool biased = treeStart == 0;
        const auto generic = [&](uint32_t begin, uint32_t end, uint32_t mode) {
            const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
            const dim3 grid(static_cast<uint32_t>((blocks + 3) / 4));
            const auto launch = [&](auto kernel) {
                hipLaunchKernelGGL(kernel, grid, dim3(256), 0, s, reinterpret_cast<const uint32_t*>(bins), docCount,
                                   m.LayoutBuckets, tt, begin, end, results, mode, biased ? 1u : 0u);
            };
            if (m.Dim == 1) {
                launch(dev::EvalObliviousKernel<1>);
            } else if (m.Dim == 2) {
                launch(dev::EvalObliviousKernel<2>);
            } else if (m.Dim <= 4) {
                launch(dev::EvalObliviousKernel<4>);
            } else if (m.Dim <= 8) {
                launch(dev::EvalObliviousKernel<8>);
            } else {
                launch(dev::EvalObliviousKernel<16>);
            }
            HIP_CHECK(hipGetLastError());
        };
        if (wholeBegin >= wholeEnd) {
            generic(tb, te, 0);  // fewer trees than a block holds (or none: the bias alone)
            return;
        }
        const bool head = tb < wholeBegin, tail = wholeEnd < te;
        if (head) {
            generic(tb, wholeBegin, dev::kEvalRaw);
        }
        TEvalRegLaunchArgs launchArgs = {};
        TEvalRegArgs& args = launchArgs.Reg;
        args.Bins = bins;
        args.Rows = m.RegRows.Get() + static_cast<size_t>(wholeBegin) * m.RegRowDwords;
        args.Out = results;
        args.DocCount = static_cast<uint32_t>(docCount);
        args.BlockCount = static_cast<uint32_t>((docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock);
        args.Flags = (biased && !tail ? 1u : 0u) | (head ? 2u : 0u) | (tail ? 4u : 0u) | (m.RegMap.Get() != nullptr ? kRegFlagMapped : 0u);
        launchArgs.RegMap = m.RegMap.Get();
        args.Scale = m.Scale;
        args.BucketCount = m.LayoutBuckets;
        args.Dim = static_cast<uint32_t>(m.Dim);
        for (const TImpl::TRegLaunch& l : m.RegLaunches) {
            args.TreeBlocks = (wholeEnd - wholeBegin + l.TreeBlock - 1) / l.TreeBlock;
            launchArgs.TreeBlocksPerSlice = args.TreeBlocks;
            args.Leaves = l.Leaves + static_cast<size_t>(wholeBegin) * l.TreeLeafDoubles;
            args.Bias = m.RegBias.Get() + l.FirstDim;
            args.FirstDim = l.FirstDim;
            args.StoreDims = l.StoreDims;
            const uint32_t grid = (args.BlockCount + l.Waves - 1) / l.Waves;
            size_t argSize = sizeof(launchArgs);
            void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &launchArgs, HIP_LAUNCH_PARAM_BUFFER_SIZE, &argSize,
                              HIP_LAUNCH_PARAM_END};
            HIP_CHECK(hipModuleLaunchKernel(l.Function, grid, 1, 1, 64 * l.Waves, 1, 1, 0, s, nullptr, config));
        }
        if (tail) {
            generic(wholeEnd, te, dev::kEvalContinue);
        }
        return;
    }
    const int dchunk = TileChunk(m.Dim);
    if (m.TileRows.Get() != nullptr) {
        // 7-bit bins, the tile fits: a tree's row in registers
        const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
        const uint32_t waves = RowTileWaves(m.TileRowCount, m.MaxDepth, m.Dim);
        const uint32_t dims = RowTileDims(m.MaxDepth, m.Dim);
        const size_t lds = RowTileLdsBytes(m.TileRowCount, m.MaxDepth, dims, waves);
        const auto launch = [&](auto kernel) {
            EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(blocks)), dim3(64 * waves), lds, s,
                               reinterpret_cast<const uint32_t*>(bins), docCount, m.LayoutBuckets, m.TileMap.Get(),
                               m.TileRowCount, reinterpret_cast<const uint4*>(m.TileRows.Get()),
                               reinterpret_cast<const double2*>(m.TileLeaves.Get()), m.Bias.Get(), m.Scale,
                               static_cast<uint32_t>(m.Dim), m.TileSliceStride, tb, te, results);
        };
        const bool wide = waves == dev::kWideTileWaves;
        if (m.MaxDepth <= 6) {
            if (dims == 1) {
                wide ? launch(dev::EvalObliviousRowTileKernel<6, dev::kWideTileWaves, 1>)
                     : launch(dev::EvalObliviousRowTileKernel<6, dev::kTileWaves, 1>);
            } else if (dims == 2) {
                wide ? launch(dev::EvalObliviousRowTileKernel<6, dev::kWideTileWaves, 2>)
                     : launch(dev::EvalObliviousRowTileKernel<6, dev::kTileWaves, 2>);
            } else {
                wide ? launch(dev::EvalObliviousRowTileKernel<6, dev::kWideTileWaves, 4>)
                     : launch(dev::EvalObliviousRowTileKernel<6, dev::kTileWaves, 4>);
            }
        } else if (dims == 1) {
            wide ? launch(dev::EvalObliviousRowTileKernel<8, dev::kWideTileWaves, 1>)
                 : launch(dev::EvalObliviousRowTileKernel<8, dev::kTileWaves, 1>);
        } else {
            wide ? launch(dev::EvalObliviousRowTileKernel<8, dev::kWideTileWaves, 2>)
                 : launch(dev::EvalObliviousRowTileKernel<8, dev::kTileWaves, 2>);
        }
        HIP_CHECK(hipGetLastError());
        return;
    }
    if (m.Oblivious && m.MaxDepth <= 8 && TileLdsBytes(m.LayoutBuckets, dchunk) <= kMaxTileLdsBytes) {
        // byte-parallel kernel over an LDS tile of bins
        const TTileArgs args{bins, docCount, m.LayoutBuckets, m.PackedTrees.Get(),
                             m.Dim == 1 ? m.Leaves.Get() : m.LeavesPadded.Get(), m.Bias.Get(), m.Scale, m.Dim, tb, te,
                             results, s, m.Dim == 1 ? m.LeavesPairAligned : true};
        if (m.PackedSevenBit) {
            LaunchEvalTileM<true>(m.MaxDepth, dchunk, args);
        } else {
            LaunchEvalTileM<false>(m.MaxDepth, dchunk, args);
        }
        HIP_CHECK(hipGetLastError());
        return;
    }
    if (m.QuadRows.Get() != nullptr) {
        // the rows do not fit the half tile: quarter blocks, four trees per wave
        const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
        const int maxd = m.MaxDepth <= 6 ? 6 : 8;
        const uint32_t waves = QuadTileWaves(m.TileRowCount, maxd);
        const size_t lds = QuadTileLdsBytes(m.TileRowCount, maxd, waves);
        CBAMD_ENSURE(4 * blocks < (size_t(1) << 31), "batch is too large for one evaluate launch");
        const auto launch = [&](auto kernel) {
            EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(4 * blocks)), dim3(64 * waves), lds, s, bins,
                               docCount, m.LayoutBuckets, m.TileMap.Get(), m.TileRowCount,
                               reinterpret_cast<const uint4*>(m.QuadRows.Get()),
                               reinterpret_cast<const double2*>(m.HalfTileLeaves.Get()), m.Bias.Get(), m.Scale, tb, te,
                               results);
        };
        if (maxd == 6) {
            waves == 8 ? launch(dev::EvalObliviousQuadTileKernel<6, 8>) : launch(dev::EvalObliviousQuadTileKernel<6, 4>);
        } else {
            waves == 8 ? launch(dev::EvalObliviousQuadTileKernel<8, 8>) : launch(dev::EvalObliviousQuadTileKernel<8, 4>);
        }
        HIP_CHECK(hipGetLastError());
        return;
    }
    if (m.Oblivious && m.MaxDepth <= 8 && m.Dim == 1 && m.HalfTileLeaves.Get() != nullptr &&
        HalfTileLdsBytes(m.LayoutBuckets, 8) <= kMaxTileLdsBytes) {
        // the bins of a block exceed the 256-document tile: half blocks
        const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
        const int maxd = m.MaxDepth <= 6 ? 6 : 8;
        if (m.PairRows.Get() != nullptr) {
            const size_t lds = PairTileLdsBytes(m.TileRowCount, maxd);
            const auto launch = [&](auto kernel) {
                EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
                hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(2 * blocks)), dim3(64 * dev::kTileWaves), lds, s,
                                   reinterpret_cast<const uint16_t*>(bins), docCount, m.LayoutBuckets, m.TileMap.Get(),
                                   m.TileRowCount, reinterpret_cast<const uint4*>(m.PairRows.Get()),
                                   reinterpret_cast<const double2*>(m.HalfTileLeaves.Get()), m.Bias.Get(), m.Scale, tb, te,
                                   results);
            };
            if (maxd == 6) {
                m.PairSix ? launch(dev::EvalObliviousPairTileKernel<6, true>) : launch(dev::EvalObliviousPairTileKernel<6, false>);
            } else {
                m.PairSix ? launch(dev::EvalObliviousPairTileKernel<8, true>) : launch(dev::EvalObliviousPairTileKernel<8, false>);
            }
            HIP_CHECK(hipGetLastError());
            return;
        }
        const size_t lds = HalfTileLdsBytes(m.LayoutBuckets, maxd);
        const auto launch = [&](auto kernel) {
            EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(2 * blocks)), dim3(64 * dev::kTileWaves), lds, s,
                               reinterpret_cast<const uint16_t*>(bins), docCount, m.LayoutBuckets, m.PackedMixed.Get(),
                               m.HalfTileLeaves.Get(), m.Bias.Get(), m.Scale, tb, te, results);
        };
        if (maxd == 6) {
            launch(dev::EvalObliviousHalfTileKernel<6>);
        } else {
            launch(dev::EvalObliviousHalfTileKernel<8>);
        }
        HIP_CHECK(hipGetLastError());
        return;
    }
    // A unit holds trees of like height from anywhere in the model, so a range of the trees still walks most
    // units: below about a third of the trees the kernel that walks the range's trees alone is the faster
    // (C4, 1M documents: all trees 1.4 against 3.5 ms, half of them 1.3 against 1.8, a fifth 0.9 against 0.7).
    if (!m.Oblivious && m.NsLdsUsable && (treeEnd - treeStart) * 10 >= TreeCount * 3) {
        const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
        const uint32_t dims = NsLdsDims(m.Dim);
        const size_t lds = NsLdsKernelBytes(m.LayoutBuckets, m.NsLdsShape.Waves, m.NsLdsShape.Entries, dims);
        const auto launch = [&](auto kernel) {
            EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
            const dim3 grid(static_cast<uint32_t>(blocks), (static_cast<uint32_t>(m.Dim) + dims - 1) / dims);
            hipLaunchKernelGGL(kernel, grid, dim3(64 * m.NsLdsShape.Waves), lds, s,
                               reinterpret_cast<const uint32_t*>(bins), docCount, m.LayoutBuckets,
                               m.NsCompactEntries.Get(), reinterpret_cast<const uint4*>(m.NsCompactRows.Get()),
                               m.NsUnitCount, m.NsValuesByEntry.Get(), m.Bias.Get(), m.Scale,
                               static_cast<uint32_t>(m.Dim), m.NsEntryCount, tb, te, results);
        };
        const auto launchDims = [&](auto one, auto two, auto four) {
            if (dims == 1) {
                launch(one);
            } else if (dims == 2) {
                launch(two);
            } else {
                launch(four);
            }
        };
        if (m.NsLdsShape.Waves == 16) {
            launchDims(dev::EvalNonSymmetricLdsKernel<16, 1024, 1>, dev::EvalNonSymmetricLdsKernel<16, 1024, 2>,
                       dev::EvalNonSymmetricLdsKernel<16, 1024, 4>);
        } else if (m.NsLdsShape.Waves == 12) {
            launchDims(dev::EvalNonSymmetricLdsKernel<12, 1536, 1>, dev::EvalNonSymmetricLdsKernel<12, 1536, 2>,
                       dev::EvalNonSymmetricLdsKernel<12, 1536, 4>);
        } else if (m.NsLdsShape.Waves == 6) {
            launchDims(dev::EvalNonSymmetricLdsKernel<6, 2048, 1>, dev::EvalNonSymmetricLdsKernel<6, 2048, 2>,
                       dev::EvalNonSymmetricLdsKernel<6, 2048, 4>);
        } else if (m.NsLdsShape.Waves == 4) {
            launchDims(dev::EvalNonSymmetricLdsKernel<4, 2048, 1>, dev::EvalNonSymmetricLdsKernel<4, 2048, 2>,
                       dev::EvalNonSymmetricLdsKernel<4, 2048, 4>);
        } else {
            launchDims(dev::EvalNonSymmetricLdsKernel<8, 2048, 1>, dev::EvalNonSymmetricLdsKernel<8, 2048, 2>,
                       dev::EvalNonSymmetricLdsKernel<8, 2048, 4>);
        }
        HIP_CHECK(hipGetLastError());
        return;
    }
    if (!m.Oblivious && m.NsTileUsable) {
        const int nsChunk = m.Dim == 1 ? 1 : m.Dim <= 4 ? 4 : 16;
        if (TileLdsBytes(m.LayoutBuckets, nsChunk) <= kMaxTileLdsBytes) {
            LaunchEvalNonSymmetricTile(m.NsNoXor, nsChunk, bins, docCount, m.LayoutBuckets,
                                       reinterpret_cast<const uint2*>(m.NsEntries.Get()),
                                       reinterpret_cast<const uint4*>(m.NsRows.Get()), m.Leaves.Get(), m.Bias.Get(),
                                       m.Scale, m.Dim, tb, te, results, s);
            HIP_CHECK(hipGetLastError());
            return;
        }
    }
    if (m.DeepRows.Get() != nullptr) {
        const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
        const int dims = DeepTileDims(m.Dim);
        const uint32_t slices = (static_cast<uint32_t>(m.Dim) + dims - 1) / dims;
        const size_t lds = DeepTileLdsBytes(m.TileRowCount, dims);
        const bool wide = 2 * lds > kMaxTileLdsBytes;  // one workgroup per CU: sixteen waves
        const dim3 grid(static_cast<uint32_t>(blocks), slices), threads(64 * (wide ? dev::kWideTileWaves : dev::kTileWaves));
        const auto launch = [&](auto kernel) {
            EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
            hipLaunchKernelGGL(kernel, grid, threads, lds, s, reinterpret_cast<const uint32_t*>(bins), docCount, m.LayoutBuckets,
                               m.TileMap.Get(), m.TileRowCount, reinterpret_cast<const uint4*>(m.DeepRows.Get()),
                               m.DeepFirstLeaf.Get(), m.Leaves.Get(), m.Bias.Get(), m.Scale, tb, te, results);
        };
        const auto launchPairs = [&](auto kernel) {
            EnsureDynamicLds(reinterpret_cast<const void*>(kernel), lds);
            hipLaunchKernelGGL(kernel, grid, threads, lds, s, reinterpret_cast<const uint32_t*>(bins), docCount, m.LayoutBuckets,
                               m.TileMap.Get(), m.TileRowCount, reinterpret_cast<const uint4*>(m.DeepRows.Get()),
                               m.DeepFirstLeaf.Get(), m.DeepLeaves.Get(), m.Bias.Get(), m.Scale, static_cast<uint32_t>(m.Dim),
                               m.DeepSliceLeaves, tb, te, results);
        };
        if (dims == 1) {
            if (m.MaxDepth <= 12) {
                wide ? launch(dev::EvalObliviousDeepTileKernel<4, dev::kWideTileWaves>)
                     : launch(dev::EvalObliviousDeepTileKernel<4, dev::kTileWaves>);
            } else {
                wide ? launch(dev::EvalObliviousDeepTileKernel<8, dev::kWideTileWaves>)
                     : launch(dev::EvalObliviousDeepTileKernel<8, dev::kTileWaves>);
            }
        } else if (m.MaxDepth <= 12) {
            wide ? launchPairs(dev::EvalObliviousDeepTilePairsKernel<4, dev::kWideTileWaves>)
                 : launchPairs(dev::EvalObliviousDeepTilePairsKernel<4, dev::kTileWaves>);
        } else {
            wide ? launchPairs(dev::EvalObliviousDeepTilePairsKernel<8, dev::kWideTileWaves>)
                 : launchPairs(dev::EvalObliviousDeepTilePairsKernel<8, dev::kTileWaves>);
        }
        HIP_CHECK(hipGetLastError());
        return;
    }
    if (m.Dim == 1) {
        LaunchEval<1>(m.Oblivious, bins, docCount, m.LayoutBuckets, tt, tb, te, results, s);
    } else if (m.Dim == 2) {
        LaunchEval<2>(m.Oblivious, bins, docCount, m.LayoutBuckets, tt, tb, te, results, s);
    } else if (m.Dim <= 4) {
        LaunchEval<4>(m.Oblivious, bins, docCount, m.LayoutBuckets, tt, tb, te, results, s);
    } else if (m.Dim <= 8) {
        LaunchEval<8>(m.Oblivious, bins, docCount, m.LayoutBuckets, tt, tb, te, results, s);
    } else {
        LaunchEval<16>(m.Oblivious, bins, docCount, m.LayoutBuckets, tt, tb, te, results, s);
    }
    HIP_CHECK(hipGetLastError());
}

uint32_t THipEvaluator::TreeSlicesFor(size_t docCount) const {
    const TImpl& m = *Impl;
    if (!m.RegKernelUsable || !m.SmallBatchSlices || docCount == 0) {
        return 1;
    }
    // Workgroups of a plain launch; below one per CU the launch lasts as long as one wave's walk through the
    // whole model, so the trees are cut into slices with workgroups of their own. A slice is two tree blocks
    // whatever the batch, so that a document's value does not depend on how many documents came with it
    // (as long as the batch is small enough to be sliced at all).
    const size_t blocks = (docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock;
    const size_t groups = (blocks + m.RegWaves - 1) / m.RegWaves;
    const size_t sliceTrees = RegSliceTrees(m.RegTreeBlockSize);
    if (groups >= 256 || TreeCount < 2 * sliceTrees) {
        return 1;
    }
    return static_cast<uint32_t>((TreeCount + sliceTrees - 1) / sliceTrees);
}

size_t THipEvaluator::TreeSliceScratchDoubles(size_t docCount) const {
    const uint32_t slices = TreeSlicesFor(docCount);
    return slices > 1 ? static_cast<size_t>(slices) * docCount * Impl->Dim : 0;
}

void THipEvaluator::EvalQuantizedSlicedDevice(const uint8_t* bins, size_t docCount, double* results, double* partials,
                                              void* stream) {
    TImpl& m = *Impl;
    const uint32_t slices = TreeSlicesFor(docCount);
    if (slices <= 1) {
        EvalQuantizedDevice(bins, docCount, 0, TreeCount, results, stream);
        return;
    }
    CBAMD_ENSURE(bins != nullptr && results != nullptr && partials != nullptr, "null pointer passed to the sliced evaluation");
    hipStream_t s = m.Pick(stream);
    TEvalRegLaunchArgs launchArgs = {};
    TEvalRegArgs& args = launchArgs.Reg;
    args.Bins = bins;
    args.Rows = m.RegRows.Get();
    args.Out = partials;
    args.DocCount = static_cast<uint32_t>(docCount);
    args.BlockCount = static_cast<uint32_t>((docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock);
    args.Flags = 4 | (m.RegMap.Get() != nullptr ? kRegFlagMapped : 0u);  // raw sums per slice
    launchArgs.RegMap = m.RegMap.Get();
    args.Scale = m.Scale;
    args.BucketCount = m.LayoutBuckets;
    args.Dim = static_cast<uint32_t>(m.Dim);
    // a slice is the same number of trees in every launch
    const uint32_t sliceTrees = RegSliceTrees(m.RegTreeBlockSize);
    for (const TImpl::TRegLaunch& l : m.RegLaunches) {
        args.TreeBlocks = static_cast<uint32_t>((TreeCount + l.TreeBlock - 1) / l.TreeBlock);
        launchArgs.TreeBlocksPerSlice = sliceTrees / l.TreeBlock;
        args.Leaves = l.Leaves;
        args.Bias = m.RegBias.Get() + l.FirstDim;
        args.FirstDim = l.FirstDim;
        args.StoreDims = l.StoreDims;
        const uint32_t grid = (args.BlockCount + l.Waves - 1) / l.Waves;
        size_t argSize = sizeof(launchArgs);
        void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &launchArgs, HIP_LAUNCH_PARAM_BUFFER_SIZE, &argSize,
                          HIP_LAUNCH_PARAM_END};
        HIP_CHECK(hipModuleLaunchKernel(l.Function, grid, slices, 1, 64 * l.Waves, 1, 1, 0, s, nullptr, config));
    }
    const size_t count = docCount * m.Dim;
    hipLaunchKernelGGL(dev::CombineSlicesKernel, dim3(static_cast<uint32_t>((count + 255) / 256)), dim3(256), 0, s, partials,
                       slices, count, m.Scale, m.Bias.Get(), m.Dim, results);
    HIP_CHECK(hipGetLastError());
}

int THipEvaluator::FusedLayoutFor(int layout, size_t stride, size_t docCount, size_t treeStart, size_t treeEnd, bool anyBatchSize) const {
    const TImpl& m = *Impl;
    const int layoutIndex = layout == TFeatureBatch::FlatRows ? 0 : layout == TFeatureBatch::SplitRows ? 1 : -1;
    if (layoutIndex < 0 || !m.Fused[layoutIndex].Usable || docCount == 0 || treeStart != 0 || treeEnd != TreeCount ||
        docCount >= (size_t(1) << 29) || stride >= (size_t(1) << 20)) {
        return -1;
    }
    if (!anyBatchSize && docCount < m.FusedMinDocs()) {
        return -1;
    }
    return layoutIndex;
}

bool THipEvaluator::EvalRowsFusedDevice(const TFeatureBatch& batch, size_t docCount, size_t treeStart, size_t treeEnd,
                                        double* results, void* stream, bool anyBatchSize) {
    TImpl& m = *Impl;
    const int layoutIndex = FusedLayoutFor(batch.Layout, batch.Stride, docCount, treeStart, treeEnd, anyBatchSize);
    if (layoutIndex < 0) {
        return false;
    }
    const TImpl::TFused& f = m.Fused[layoutIndex];
    CBAMD_ENSURE(results != nullptr, "results pointer is null");
    CBAMD_ENSURE(batch.Floats != nullptr, "float features pointer is null");
    const size_t need = layoutIndex == 0 ? m.FlatVectorSize : m.MinFloatSize;
    CBAMD_ENSURE(batch.Stride >= need, (layoutIndex == 0 ? "insufficient flat features vector size: " : "insufficient float features vector size: ") +
                                           std::to_string(batch.Stride) + " expected: " + std::to_string(need));
    TEvalFusedArgs args = {};
    args.Reg.Rows = f.Rows.Get();
    args.Reg.Leaves = f.Table.Get();
    args.Reg.Out = results;
    args.Reg.DocCount = static_cast<uint32_t>(docCount);
    args.Reg.BlockCount = static_cast<uint32_t>((docCount + dev::kDocsPerBlock - 1) / dev::kDocsPerBlock);
    args.Reg.TreeBlocks = m.RegTreeBlocks;
    args.Reg.Flags = 1;
    args.Reg.Scale = m.Scale;
    args.Reg.Bias = m.RegBias.Get();
    args.Reg.BucketCount = m.LayoutBuckets;
    args.Reg.Dim = 1;
    args.Reg.FirstDim = 0;
    args.Reg.StoreDims = 1;
    args.Floats = batch.Floats;
    args.Units = f.Units.Get();
    args.StrideBytes = static_cast<uint32_t>(batch.Stride * sizeof(float));
    args.UnitCount = f.UnitCount;
    const uint32_t grid = (args.Reg.BlockCount + m.FusedWaves - 1) / m.FusedWaves;
    size_t argSize = sizeof(args);
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &argSize, HIP_LAUNCH_PARAM_END};
    HIP_CHECK(hipModuleLaunchKernel(m.FusedFunction, grid, 1, 1, 64 * m.FusedWaves, 1, 1, 0, m.Pick(stream), nullptr, config));
    return true;
}

std::string THipEvaluator::DescribeKernels(int layout, size_t docCount, size_t stride) const {
    const TImpl& m = *Impl;
    // whole-model calls only: a call for a range of the trees may take other kernels
    if (FusedLayoutFor(layout, stride, docCount, 0, TreeCount, false) >= 0) {
        return std::string("fused=") + m.FusedKernelName;
    }
    std::string binarize = m.BinarizeBuckets == 0 ? "none"
                           : layout == TFeatureBatch::FlatColumns
                               ? "BinarizeColumnsKernel"
                               : "BinarizeRowsKernel<" + std::to_string(BinarizeLog2Slots(m.MaxBucketValues)) + ">";
    if (m.CtrCount > 0) {
        binarize += m.CtrTileUsable ? "+CtrBinarizeTileKernel" : "+CtrBinarizeKernel";
    }
    const int dchunk = TileChunk(m.Dim);
    std::string evaluate;
    if (TreeCount == 0) {
        evaluate = "FillBiasKernel";
    } else if (m.RegKernelUsable) {
        evaluate = m.RegKernelName;
        if (m.RegLaunches.size() > 1) {
            const size_t main = m.RegLaunches.size() - (m.RegTailLeaves.Get() != nullptr ? 1 : 0);
            if (main > 1) {
                evaluate += " x " + std::to_string(main) + " launches";
            }
            if (main < m.RegLaunches.size()) {
                evaluate += std::string(" + ") + m.RegLaunches.back().Name;
            }
        }
        const uint32_t slices = TreeSlicesFor(docCount);
        if (slices > 1) {
            evaluate += " x " + std::to_string(slices) + " slices of the trees + CombineSlicesKernel";
        }
    } else if (m.TileRows.Get() != nullptr) {
        evaluate = "EvalObliviousRowTileKernel";
    } else if (m.Oblivious && m.MaxDepth <= 8 && TileLdsBytes(m.LayoutBuckets, dchunk) <= kMaxTileLdsBytes) {
        evaluate = "EvalObliviousTileKernel";
    } else if (m.QuadRows.Get() != nullptr) {
        evaluate = "EvalObliviousQuadTileKernel";
    } else if (m.Oblivious && m.MaxDepth <= 8 && m.Dim == 1 && m.HalfTileLeaves.Get() != nullptr &&
               TileLdsBytes(m.LayoutBuckets, 1) > kMaxTileLdsBytes && HalfTileLdsBytes(m.LayoutBuckets, 8) <= kMaxTileLdsBytes) {
        evaluate = m.PairRows.Get() != nullptr ? "EvalObliviousPairTileKernel" : "EvalObliviousHalfTileKernel";
    } else if (m.DeepRows.Get() != nullptr) {
        evaluate = "EvalObliviousDeepTileKernel";
    } else if (m.Oblivious) {
        evaluate = "EvalObliviousKernel";
    } else if (m.NsLdsUsable) {
        evaluate = "EvalNonSymmetricLdsKernel<" + std::to_string(m.NsLdsShape.Waves) + ", " +
                   std::to_string(m.NsLdsShape.Entries) + (m.Dim > 1 ? ", " + std::to_string(NsLdsDims(m.Dim)) : "") + ">";
    } else if (m.NsTileUsable && TileLdsBytes(m.LayoutBuckets, m.Dim == 1 ? 1 : m.Dim <= 4 ? 4 : 16) <= kMaxTileLdsBytes) {
        evaluate = "EvalNonSymmetricTileKernel";
    } else {
        evaluate = "EvalNonSymmetricKernel";
    }
    return "binarize=" + binarize + ";evaluate=" + evaluate;
}

void THipEvaluator::LeafIndexesQuantizedDevice(const uint8_t* bins, size_t docCount, size_t treeStart, size_t treeEnd,
                                               uint32_t* indexes, void* stream) {
    TImpl& m = *Impl;
    CBAMD_ENSURE(treeStart <= treeEnd && treeEnd <= TreeCount, "tree range is out of bounds");
    if (docCount == 0 || treeStart == treeEnd) {
        return;
    }
    CBAMD_ENSURE(bins != nullptr && indexes != nullptr, "null pointer passed to leaf index calculation");
    hipStream_t s = m.Pick(stream);
    const size_t blocks = (docCount + 255) / 256;
    const size_t tileLds = static_cast<size_t>(m.LayoutBuckets) * dev::kDocsPerBlock + dev::kWave * dev::kLeafIndexPitch * 4;
    if (m.Oblivious && m.MaxDepth <= 8 && m.PackedTrees.Get() != nullptr && tileLds <= kMaxTileLdsBytes) {
        const auto launch = [&](auto kernel) {
            EnsureDynamicLds(reinterpret_cast<const void*>(kernel), tileLds);
            hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), tileLds, s,
                               reinterpret_cast<const uint32_t*>(bins), docCount, m.LayoutBuckets, m.PackedTrees.Get(),
                               static_cast<uint32_t>(treeStart), static_cast<uint32_t>(treeEnd), indexes);
        };
        if (m.PackedSevenBit) {
            launch(dev::LeafIndexesTileKernel<true>);
        } else {
            launch(dev::LeafIndexesTileKernel<false>);
        }
        HIP_CHECK(hipGetLastError());
        return;
    }
    hipLaunchKernelGGL(dev::LeafIndexesKernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s, bins, docCount,
                       m.LayoutBuckets, m.TreeTables(), m.Oblivious ? 1 : 0, static_cast<uint32_t>(treeStart),
                       static_cast<uint32_t>(treeEnd), indexes);
    HIP_CHECK(hipGetLastError());
}

void THipEvaluator::ExportQuantizedDevice(const uint8_t* bins, size_t docCount, uint8_t* referenceLayout, void* stream) {
    TImpl& m = *Impl;
    if (docCount == 0 || m.RealBucketCount == 0) {
        return;
    }
    hipStream_t s = m.Pick(stream);
    hipLaunchKernelGGL(dev::ExportBinsKernel, dim3(static_cast<uint32_t>((docCount + 255) / 256)), dim3(256), 0, s, bins,
                       docCount, m.LayoutBuckets, referenceLayout);
    HIP_CHECK(hipGetLastError());
}

void THipEvaluator::ApplyPredictionTypeDevice(int predictionType, size_t firstDoc, size_t totalDocs, size_t docCount,
                                              const double* raw, double* result, void* stream) {
    TImpl& m = *Impl;
    const uint32_t dim = static_cast<uint32_t>(m.Dim);
    CBAMD_ENSURE(predictionType >= dev::kPredRaw && predictionType <= dev::kPredMultiProbability, "unknown prediction type");
    // one dimension: the types TEvalResultProcessor accepts (eval_processing.h:182-204)
    CBAMD_ENSURE(dim > 1 || predictionType == dev::kPredRaw || predictionType == dev::kPredExponent ||
                     predictionType == dev::kPredProbability || predictionType == dev::kPredClass,
                 "unsupported prediction type");
    CBAMD_ENSURE(firstDoc <= totalDocs && docCount <= totalDocs - firstDoc, "document range exceeds the batch");
    CBAMD_ENSURE(firstDoc % 128 == 0, "a chunk must start at a multiple of 128 documents");
    if (docCount == 0) {
        return;
    }
    CBAMD_ENSURE(raw != nullptr && result != nullptr, "prediction buffers are null");
    CBAMD_ENSURE(!(predictionType == dev::kPredClass && dim > 1 && raw == result),
                 "Class of a multi-dimensional model cannot be computed in place");
    HIP_CHECK(hipSetDevice(m.DeviceId));
    hipStream_t s = m.Pick(stream);
    const TFastExpConstants constants = FastExpConstants();
    dev::TFastExpDev c;
    c.Mantissa = m.ExpMantissa.Get();
    c.Scale = constants.Scale;
    c.InvScale = constants.InvScale;
    CBAMD_ENSURE((docCount + 255) / 256 <= 0x7fffffffu, "too many documents in one batch");
    hipLaunchKernelGGL(dev::ApplyPredictionTypeKernel, dim3(static_cast<uint32_t>((docCount + 255) / 256)), dim3(256), 0, s,
                       predictionType, dim, firstDoc, totalDocs, docCount, c, raw, result);
    HIP_CHECK(hipGetLastError());
}

void THipEvaluator::CalcDevice(const TFeatureBatch& batch, size_t docCount, size_t treeStart, size_t treeEnd,
                               double* results, void* stream) {
    TImpl& m = *Impl;
    HIP_CHECK(hipSetDevice(m.DeviceId));
    TImpl::TContextLease ctx(m);
    hipStream_t s = stream ? static_cast<hipStream_t>(stream) : m.Stream;
    TKernelTimes times;
    HIP_CHECK(hipEventRecord(ctx->Ev[0], s));
    if (EvalRowsFusedDevice(batch, docCount, treeStart, treeEnd, results, s)) {
        // one launch does both: its whole duration is reported as the evaluate time
        HIP_CHECK(hipEventRecord(ctx->Ev[2], s));
        HIP_CHECK(hipStreamSynchronize(s));
        HIP_CHECK(hipEventElapsedTime(&times.EvalMs, ctx->Ev[0], ctx->Ev[2]));
    } else {
        ctx->ScratchBins.Reserve(QuantizedBytes(docCount));
        const bool sliced = treeStart == 0 && treeEnd == TreeCount && TreeSlicesFor(docCount) > 1;
        if (sliced) {
            ctx->SlicePartials.Reserve(TreeSliceScratchDoubles(docCount));
        }
        QuantizeDevice(batch, docCount, ctx->ScratchBins.Get(), s);
        HIP_CHECK(hipEventRecord(ctx->Ev[1], s));
        if (sliced) {
            EvalQuantizedSlicedDevice(ctx->ScratchBins.Get(), docCount, results, ctx->SlicePartials.Get(), s);
        } else {
            EvalQuantizedDevice(ctx->ScratchBins.Get(), docCount, treeStart, treeEnd, results, s);
        }
        HIP_CHECK(hipEventRecord(ctx->Ev[2], s));
        HIP_CHECK(hipStreamSynchronize(s));
        HIP_CHECK(hipEventElapsedTime(&times.BinarizeMs, ctx->Ev[0], ctx->Ev[1]));
        HIP_CHECK(hipEventElapsedTime(&times.EvalMs, ctx->Ev[1], ctx->Ev[2]));
    }
    SetLastTimes(times);
}

void THipEvaluator::SetSmallBatchSlicing(bool on) {
    Impl->SmallBatchSlices = on;
}

bool THipEvaluator::SmallBatchSlicing() const {
    return Impl->SmallBatchSlices;
}

void THipEvaluator::CalcDeviceNoAlloc(const TFeatureBatch& batch, size_t docCount, size_t treeStart, size_t treeEnd,
                                      double* results, void* stream) {
    TImpl& m = *Impl;
    const size_t maxDocs = kNoAllocScratchBytes / (static_cast<size_t>(m.LayoutBuckets) * dev::kDocsPerBlock) * dev::kDocsPerBlock;
    // the fused kernel keeps the bins in registers: no buffer at all. A batch whose bins do not fit the fixed
    // buffer takes it whatever its size (below the size from which it is the faster as well)
    if (EvalRowsFusedDevice(batch, docCount, treeStart, treeEnd, results, stream, docCount > maxDocs)) {
        return;
    }
    CBAMD_ENSURE(docCount <= maxDocs, "batch of " + std::to_string(docCount) + " documents exceeds the fixed bin buffer: at most " +
                                          std::to_string(maxDocs) + " documents per call for this model");
    // every (block, bucket) cell that the evaluate kernels read is written by the binarize kernels of
    // the same call, so nothing of the previous call's contents has to be cleared
    QuantizeDevice(batch, docCount, m.NoAllocScratch, stream);
    EvalQuantizedDevice(m.NoAllocScratch, docCount, treeStart, treeEnd, results, stream);
}

// ---------------------------------------------------------------------------- host staging ----

namespace {

// documents per slot of the staging pipeline: small enough that gathering the next slot on the host
// overlaps the transfer and the kernels of the current one
size_t PipelineDocs(size_t bytesPerDoc) {
    size_t docs = (size_t(64) << 20) / std::max<size_t>(1, bytesPerDoc);
    docs = std::max<size_t>(docs, 4096);
    docs = std::min<size_t>(docs, size_t(1) << 20);
    return docs / dev::kDocsPerBlock * dev::kDocsPerBlock;
}

// Runs `work(begin, end)` over [0, count) on a few threads when the bytes to move make it worthwhile.
template <typename TWork>
void ParallelCopy(size_t count, size_t bytes, const TWork& work) {
    size_t threads = std::min<size_t>(std::max(1u, std::thread::hardware_concurrency()), 16);
    threads = std::min(threads, bytes / (size_t(4) << 20) + 1);
    threads = std::min(threads, std::max<size_t>(count, 1));
    if (threads <= 1) {
        work(size_t(0), count);
        return;
    }
    std::vector<std::thread> pool;
    const size_t per = (count + threads - 1) / threads;
    for (size_t t = 1; t < threads; ++t) {
        pool.emplace_back(work, std::min(count, t * per), std::min(count, (t + 1) * per));
    }
    work(size_t(0), std::min(count, per));
    for (auto& th : pool) {
        th.join();
    }
}

// Copies `count` rows of `rowLen` elements each, given by pointer, into a dense matrix (the copy is
// what bounds the pointer-per-row entry points).
template <typename T>
void GatherRows(const T* const* rows, size_t count, size_t rowLen, T* dst) {
    ParallelCopy(count, count * rowLen * sizeof(T), [=](size_t begin, size_t end) {
        for (size_t d = begin; d < end; ++d) {
            std::memcpy(dst + d * rowLen, rows[d], rowLen * sizeof(T));
        }
    });
}

// A model without trees answers with its bias whatever the prediction type: the reference fills the result
// array with the bias values in turn and returns before any post-processing (cpu/formula_evaluator.cpp:29-41).
void FillBiasOnly(const std::vector<double>& bias, size_t count, double* results) {
    for (size_t i = 0; i < count; ++i) {
        results[i] = bias.empty() ? 0.0 : bias[i % bias.size()];
    }
}

// The two-slot pipeline of the host entry points: documents go in chunks; while the GPU copies in, runs and
// copies out the chunk of one slot, the host fills the other slot. stage(slot, begin, n) fills the slot's
// pinned memory and enqueues everything up to the event Ev[3] of the slot; collect(slot, begin, n) runs once
// that event has passed.
template <typename TStage, typename TCollect>
void RunPipeline(size_t docCount, size_t chunk, hipEvent_t (&done)[2], const TStage& stage, const TCollect& collect) {
    size_t pendingBegin[2] = {0, 0}, pendingDocs[2] = {0, 0};
    size_t index = 0;
    const auto finish = [&](int slot) {
        if (pendingDocs[slot]) {
            HIP_CHECK(hipEventSynchronize(done[slot]));
            collect(slot, pendingBegin[slot], pendingDocs[slot]);
            pendingDocs[slot] = 0;
        }
    };
    for (size_t begin = 0; begin < docCount; begin += chunk, ++index) {
        const int slot = static_cast<int>(index & 1);
        const size_t n = std::min(chunk, docCount - begin);
        finish(slot);  // the slot's previous chunk must be out before its buffers are reused
        stage(slot, begin, n);
        pendingBegin[slot] = begin;
        pendingDocs[slot] = n;
    }
    // the (up to) two chunks still in flight, older first
    finish(static_cast<int>(index & 1));
    finish(static_cast<int>((index + 1) & 1));
}

}  // namespace

void THipEvaluator::SetLastTimes(const TKernelTimes& times) {
    std::lock_guard<std::mutex> guard(TimesLock);
    LastTimes = times;
}

TKernelTimes THipEvaluator::LastKernelTimes() const {
    std::lock_guard<std::mutex> guard(TimesLock);
    return LastTimes;
}

// Stages one chunk of rows given by pointer (the reference API's float** / hashed int**) and returns the
// batch that describes it on the device.
static TFeatureBatch StageRowChunk(THipEvaluator::TImpl::THostSlot& slot, hipStream_t s, const float* const* rows,
                                   const int32_t* const* catRows, size_t begin, size_t n, size_t needFloats,
                                   size_t needCats, bool flat) {
    if (needFloats) {
        GatherRows(rows + begin, n, needFloats, slot.PinnedFloats.Get());
        HIP_CHECK(hipMemcpyAsync(slot.StageFloats.Get(), slot.PinnedFloats.Get(), n * needFloats * sizeof(float),
                                 hipMemcpyHostToDevice, s));
    }
    if (needCats) {
        GatherRows(catRows + begin, n, needCats, slot.PinnedCats.Get());
        HIP_CHECK(hipMemcpyAsync(slot.StageCats.Get(), slot.PinnedCats.Get(), n * needCats * sizeof(int32_t),
                                 hipMemcpyHostToDevice, s));
    }
    TFeatureBatch batch;
    batch.Layout = flat ? TFeatureBatch::FlatRows : TFeatureBatch::SplitRows;
    batch.Floats = slot.StageFloats.Get();
    batch.Stride = needFloats;
    batch.Cats = needCats ? slot.StageCats.Get() : nullptr;
    batch.CatStride = needCats;
    return batch;
}

// What the prediction entry points share once a chunk's features are on the device: binarize, evaluate,
// prediction type, copy back; the slot's events bracket the kernels.
static void RunPredictionChunk(THipEvaluator& ev, THipEvaluator::TImpl::THostContext& ctx, int slotIndex,
                               const TFeatureBatch& batch, size_t begin, size_t n, size_t docCount, size_t stageDocs,
                               size_t treeStart, size_t treeEnd, int predictionType) {
    THipEvaluator::TImpl::THostSlot& slot = ctx.Slots[slotIndex];
    hipStream_t s = ctx.Stream;
    const size_t dim = static_cast<size_t>(ev.GetApproxDimension());
    const size_t outDim = predictionType == dev::kPredClass ? 1 : dim;
    HIP_CHECK(hipEventRecord(slot.Ev[0], s));
    if (ev.FusedLayoutFor(batch.Layout, batch.Stride, n, treeStart, treeEnd, false) >= 0) {
        // one launch does both: its whole duration is reported as the evaluate time, as CalcDevice does
        HIP_CHECK(hipEventRecord(slot.Ev[1], s));
        ev.EvalRowsFusedDevice(batch, n, treeStart, treeEnd, slot.StageResults.Get(), s);
    } else {
        ev.QuantizeDevice(batch, n, ctx.ScratchBins.Get(), s);
        HIP_CHECK(hipEventRecord(slot.Ev[1], s));
        if (treeStart == 0 && treeEnd == ev.GetTreeCount() && ev.TreeSlicesFor(n) > 1) {
            ctx.SlicePartials.Reserve(ev.TreeSliceScratchDoubles(n));
            ev.EvalQuantizedSlicedDevice(ctx.ScratchBins.Get(), n, slot.StageResults.Get(), ctx.SlicePartials.Get(), s);
        } else {
            ev.EvalQuantizedDevice(ctx.ScratchBins.Get(), n, treeStart, treeEnd, slot.StageResults.Get(), s);
        }
    }
    HIP_CHECK(hipEventRecord(slot.Ev[2], s));
    const double* final = slot.StageResults.Get();
    if (predictionType != dev::kPredRaw) {
        // raw values, and behind them room for a prediction type that cannot be computed in place
        double* processed = slot.StageResults.Get() + (outDim == dim ? 0 : stageDocs * dim);
        ev.ApplyPredictionTypeDevice(predictionType, begin, docCount, n, slot.StageResults.Get(), processed, s);
        final = processed;
    }
    HIP_CHECK(hipMemcpyAsync(slot.PinnedResults.Get(), final, n * outDim * sizeof(double), hipMemcpyDeviceToHost, s));
    HIP_CHECK(hipEventRecord(slot.Ev[3], s));
}

void THipEvaluator::CalcHostRows(const float* const* rows, size_t rowLen, bool flat, const int32_t* const* catRows,
                                 size_t catRowLen, size_t docCount, size_t treeStart, size_t treeEnd, double* results,
                                 int predictionType) {
    TImpl& m = *Impl;
    const size_t outDim = predictionType == dev::kPredClass ? 1 : static_cast<size_t>(m.Dim);
    // only the columns the model can address are staged
    const size_t needFloats = flat ? m.FlatVectorSize : m.MinFloatSize;
    const size_t needCats = (!flat && m.HasCats) ? m.MinCatSize : 0;
    CBAMD_ENSURE(needFloats == 0 || rows != nullptr, "Model has float features but no float features provided");
    CBAMD_ENSURE(rowLen >= needFloats, (flat ? "insufficient flat features vector size: " : "insufficient float features vector size: ") +
                                           std::to_string(rowLen) + " expected: " + std::to_string(needFloats));
    CBAMD_ENSURE(needCats == 0 || catRows != nullptr, "Model has categorical features but no categorical features provided");
    CBAMD_ENSURE(catRowLen >= needCats, "insufficient cat features vector size: " + std::to_string(catRowLen) +
                                            " expected: " + std::to_string(needCats));
    if (TreeCount == 0) {
        FillBiasOnly(m.HostBias, docCount * outDim, results);
        return;
    }
    HIP_CHECK(hipSetDevice(m.DeviceId));
    TImpl::TContextLease ctx(m);
    const size_t chunk = PipelineDocs((needFloats + needCats) * 4);
    const size_t stageDocs = std::min(chunk, docCount);
    for (int i = 0; i < (docCount > chunk ? 2 : 1); ++i) {
        TImpl::THostSlot& slot = ctx->Slots[i];
        slot.PinnedFloats.Reserve(std::max<size_t>(1, stageDocs * needFloats));
        slot.StageFloats.Reserve(std::max<size_t>(1, stageDocs * needFloats));
        if (needCats) {
            slot.PinnedCats.Reserve(stageDocs * needCats);
            slot.StageCats.Reserve(stageDocs * needCats);
        }
        slot.PinnedResults.Reserve(std::max<size_t>(1, stageDocs * m.Dim));
        slot.StageResults.Reserve(std::max<size_t>(1, stageDocs * (m.Dim + 1)));
    }
    ctx->ScratchBins.Reserve(QuantizedBytes(stageDocs));
    TKernelTimes times;
    hipEvent_t done[2] = {ctx->Slots[0].Ev[3], ctx->Slots[1].Ev[3]};
    RunPipeline(
        docCount, chunk, done,
        [&](int i, size_t begin, size_t n) {
            const TFeatureBatch batch = StageRowChunk(ctx->Slots[i], ctx->Stream, rows, catRows, begin, n, needFloats, needCats, flat);
            RunPredictionChunk(*this, *ctx, i, batch, begin, n, docCount, stageDocs, treeStart, treeEnd, predictionType);
        },
        [&](int i, size_t begin, size_t n) {
            TImpl::THostSlot& slot = ctx->Slots[i];
            std::memcpy(results + begin * outDim, slot.PinnedResults.Get(), n * outDim * sizeof(double));
            float a = 0.f, b = 0.f;
            HIP_CHECK(hipEventElapsedTime(&a, slot.Ev[0], slot.Ev[1]));
            HIP_CHECK(hipEventElapsedTime(&b, slot.Ev[1], slot.Ev[2]));
            times.BinarizeMs += a;
            times.EvalMs += b;
        });
    SetLastTimes(times);
}

// Columns by pointer (CalcModelPredictionFlatTransposed): a chunk is staged as a dense [feature][document]
// matrix, the columns copied by a few threads, and goes through the same two-slot pipeline.
void THipEvaluator::CalcHostColumns(const float* const* columns, size_t columnCount, size_t docCount, size_t treeStart,
                                    size_t treeEnd, double* results, int predictionType) {
    TImpl& m = *Impl;
    const size_t outDim = predictionType == dev::kPredClass ? 1 : static_cast<size_t>(m.Dim);
    const size_t need = m.FlatVectorSize;
    CBAMD_ENSURE(columnCount >= need, "Not enough features provided");
    CBAMD_ENSURE(need == 0 || columns != nullptr, "Not enough features provided");
    if (TreeCount == 0) {
        FillBiasOnly(m.HostBias, docCount * outDim, results);
        return;
    }
    HIP_CHECK(hipSetDevice(m.DeviceId));
    TImpl::TContextLease ctx(m);
    const size_t chunk = PipelineDocs(need * 4);
    const size_t stageDocs = std::min(chunk, docCount);
    for (int i = 0; i < (docCount > chunk ? 2 : 1); ++i) {
        TImpl::THostSlot& slot = ctx->Slots[i];
        slot.PinnedFloats.Reserve(std::max<size_t>(1, stageDocs * need));
        slot.StageFloats.Reserve(std::max<size_t>(1, stageDocs * need));
        slot.PinnedResults.Reserve(std::max<size_t>(1, stageDocs * m.Dim));
        slot.StageResults.Reserve(std::max<size_t>(1, stageDocs * (m.Dim + 1)));
    }
    ctx->ScratchBins.Reserve(QuantizedBytes(stageDocs));
    TKernelTimes times;
    hipEvent_t done[2] = {ctx->Slots[0].Ev[3], ctx->Slots[1].Ev[3]};
    RunPipeline(
        docCount, chunk, done,
        [&](int i, size_t begin, size_t n) {
            TImpl::THostSlot& slot = ctx->Slots[i];
            float* dst = slot.PinnedFloats.Get();
            ParallelCopy(need, need * n * sizeof(float), [=](size_t first, size_t last) {
                for (size_t f = first; f < last; ++f) {
                    if (columns[f] != nullptr) {
                        std::memcpy(dst + f * n, columns[f] + begin, n * sizeof(float));
                    } else {
                        std::memset(dst + f * n, 0, n * sizeof(float));
                    }
                }
            });
            if (need) {
                HIP_CHECK(hipMemcpyAsync(slot.StageFloats.Get(), dst, n * need * sizeof(float), hipMemcpyHostToDevice, ctx->Stream));
            }
            TFeatureBatch batch;
            batch.Layout = TFeatureBatch::FlatColumns;
            batch.Floats = slot.StageFloats.Get();
            batch.Stride = n;
            RunPredictionChunk(*this, *ctx, i, batch, begin, n, docCount, stageDocs, treeStart, treeEnd, predictionType);
        },
        [&](int i, size_t begin, size_t n) {
            TImpl::THostSlot& slot = ctx->Slots[i];
            std::memcpy(results + begin * outDim, slot.PinnedResults.Get(), n * outDim * sizeof(double));
            float a = 0.f, b = 0.f;
            HIP_CHECK(hipEventElapsedTime(&a, slot.Ev[0], slot.Ev[1]));
            HIP_CHECK(hipEventElapsedTime(&b, slot.Ev[1], slot.Ev[2]));
            times.BinarizeMs += a;
            times.EvalMs += b;
        });
    SetLastTimes(times);
}

void THipEvaluator::LeafIndexesHostRows(const float* const* rows, size_t rowLen, bool flat,
                                        const int32_t* const* catRows, size_t catRowLen, size_t docCount,
                                        size_t treeStart, size_t treeEnd, uint32_t* indexes) {
    TImpl& m = *Impl;
    CBAMD_ENSURE(treeStart <= treeEnd && treeEnd <= TreeCount, "tree range is out of bounds");
    const size_t treeCount = treeEnd - treeStart;
    const size_t needFloats = flat ? m.FlatVectorSize : m.MinFloatSize;
    const size_t needCats = (!flat && m.HasCats) ? m.MinCatSize : 0;
    CBAMD_ENSURE(needFloats == 0 || rows != nullptr, "Model has float features but no float features provided");
    CBAMD_ENSURE(rowLen >= needFloats, "insufficient float features vector size: " + std::to_string(rowLen) +
                                           " expected: " + std::to_string(needFloats));
    CBAMD_ENSURE(needCats == 0 || catRows != nullptr, "Model has categorical features but no categorical features provided");
    CBAMD_ENSURE(catRowLen >= needCats, "insufficient cat features vector size");
    if (docCount == 0 || treeCount == 0) {
        return;
    }
    HIP_CHECK(hipSetDevice(m.DeviceId));
    TImpl::TContextLease ctx(m);
    const size_t chunk = PipelineDocs((needFloats + needCats + treeCount) * 4);
    const size_t stageDocs = std::min(chunk, docCount);
    for (int i = 0; i < (docCount > chunk ? 2 : 1); ++i) {
        TImpl::THostSlot& slot = ctx->Slots[i];
        slot.PinnedFloats.Reserve(std::max<size_t>(1, stageDocs * needFloats));
        slot.StageFloats.Reserve(std::max<size_t>(1, stageDocs * needFloats));
        if (needCats) {
            slot.PinnedCats.Reserve(stageDocs * needCats);
            slot.StageCats.Reserve(stageDocs * needCats);
        }
        slot.PinnedIndexes.Reserve(stageDocs * treeCount);
        slot.StageIndexes.Reserve(stageDocs * treeCount);
    }
    ctx->ScratchBins.Reserve(QuantizedBytes(stageDocs));
    hipEvent_t done[2] = {ctx->Slots[0].Ev[3], ctx->Slots[1].Ev[3]};
    RunPipeline(
        docCount, chunk, done,
        [&](int i, size_t begin, size_t n) {
            TImpl::THostSlot& slot = ctx->Slots[i];
            hipStream_t s = ctx->Stream;
            const TFeatureBatch batch = StageRowChunk(slot, s, rows, catRows, begin, n, needFloats, needCats, flat);
            QuantizeDevice(batch, n, ctx->ScratchBins.Get(), s);
            LeafIndexesQuantizedDevice(ctx->ScratchBins.Get(), n, treeStart, treeEnd, slot.StageIndexes.Get(), s);
            HIP_CHECK(hipMemcpyAsync(slot.PinnedIndexes.Get(), slot.StageIndexes.Get(), n * treeCount * sizeof(uint32_t),
                                     hipMemcpyDeviceToHost, s));
            HIP_CHECK(hipEventRecord(slot.Ev[3], s));
        },
        [&](int i, size_t begin, size_t n) {
            // 4 bytes per document and tree: the copy out of the pinned buffer bounds this call, so it is shared out
            uint32_t* dst = indexes + begin * treeCount;
            const uint32_t* src = ctx->Slots[i].PinnedIndexes.Get();
            ParallelCopy(n, n * treeCount * sizeof(uint32_t), [=](size_t first, size_t last) {
                std::memcpy(dst + first * treeCount, src + first * treeCount, (last - first) * treeCount * sizeof(uint32_t));
            });
        });
}

void THipEvaluator::QuantizeHostRows(const float* const* rows, size_t rowLen, bool flat, const int32_t* const* catRows,
                                     size_t catRowLen, size_t docCount, uint8_t* referenceLayout) {
    TImpl& m = *Impl;
    const size_t needFloats = flat ? m.FlatVectorSize : m.MinFloatSize;
    const size_t needCats = (!flat && m.HasCats) ? m.MinCatSize : 0;
    CBAMD_ENSURE(needFloats == 0 || rows != nullptr, "Model has float features but no float features provided");
    CBAMD_ENSURE(rowLen >= needFloats, "insufficient float features vector size: " + std::to_string(rowLen) +
                                           " expected: " + std::to_string(needFloats));
    CBAMD_ENSURE(needCats == 0 || catRows != nullptr, "Model has categorical features but no categorical features provided");
    CBAMD_ENSURE(catRowLen >= needCats, "insufficient cat features vector size");
    if (docCount == 0 || m.RealBucketCount == 0) {
        return;
    }
    HIP_CHECK(hipSetDevice(m.DeviceId));
    TImpl::TContextLease ctx(m);
    // chunks end on a multiple of 256 documents, so that the reference's blocks of 128 do not straddle them
    const size_t chunk = PipelineDocs((needFloats + needCats) * 4 + m.RealBucketCount);
    const size_t stageDocs = std::min(chunk, docCount);
    for (int i = 0; i < (docCount > chunk ? 2 : 1); ++i) {
        TImpl::THostSlot& slot = ctx->Slots[i];
        slot.PinnedFloats.Reserve(std::max<size_t>(1, stageDocs * needFloats));
        slot.StageFloats.Reserve(std::max<size_t>(1, stageDocs * needFloats));
        if (needCats) {
            slot.PinnedCats.Reserve(stageDocs * needCats);
            slot.StageCats.Reserve(stageDocs * needCats);
        }
        slot.PinnedExport.Reserve(stageDocs * m.RealBucketCount);
        slot.StageExport.Reserve(stageDocs * m.RealBucketCount);
    }
    ctx->ScratchBins.Reserve(QuantizedBytes(stageDocs));
    hipEvent_t done[2] = {ctx->Slots[0].Ev[3], ctx->Slots[1].Ev[3]};
    RunPipeline(
        docCount, chunk, done,
        [&](int i, size_t begin, size_t n) {
            TImpl::THostSlot& slot = ctx->Slots[i];
            hipStream_t s = ctx->Stream;
            const TFeatureBatch batch = StageRowChunk(slot, s, rows, catRows, begin, n, needFloats, needCats, flat);
            QuantizeDevice(batch, n, ctx->ScratchBins.Get(), s);
            ExportQuantizedDevice(ctx->ScratchBins.Get(), n, slot.StageExport.Get(), s);
            HIP_CHECK(hipMemcpyAsync(slot.PinnedExport.Get(), slot.StageExport.Get(), n * m.RealBucketCount,
                                     hipMemcpyDeviceToHost, s));
            HIP_CHECK(hipEventRecord(slot.Ev[3], s));
        },
        [&](int i, size_t begin, size_t n) {
            std::memcpy(referenceLayout + begin * m.RealBucketCount, ctx->Slots[i].PinnedExport.Get(), n * m.RealBucketCount);
        });
}

}  // namespace cbamd
