#include "fast_exp.h"

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <mutex>

namespace cbamd {

namespace {

constexpr int kTableBits = 11;  // fmath EXPD_TABLE_SIZE

// ExpdVar<11> of fmath.hpp:150-185: mantissas of 2^(i / 2048), 2048 / ln 2 and its reciprocal,
// produced at start-up by the C library like in the reference
struct TExpTable {
    uint64_t Mantissa[1 << kTableBits];
    double Scale;
    double InvScale;

    TExpTable() {
        const int size = 1 << kTableBits;
        Scale = size / std::log(2.0);
        InvScale = 1 / Scale;
        for (int i = 0; i < size; ++i) {
            const double p = std::pow(2.0, i * (1.0 / size));
            uint64_t bits;
            std::memcpy(&bits, &p, sizeof(bits));
            Mantissa[i] = bits & ((uint64_t(1) << 52) - 1);
        }
    }
};

const TExpTable& Table() {
    static const TExpTable table;
    return table;
}

// Shared arithmetic of both forms; `indexBits` is what the table index (low 11 bits) and the binary
// exponent (bits 11..22, biased by kAdjust) are read from. The library is built with
// -ffp-contract=off: every operation below rounds on its own, as the SSE/AVX intrinsics do.
inline double ExpFromRounded(const TExpTable& c, double x, double rounded, uint64_t indexBits) {
    constexpr double kMagic = static_cast<double>(uint64_t(3) << 51);
    constexpr uint64_t kAdjust = (uint64_t(1) << (kTableBits + 10)) - (uint64_t(1) << kTableBits);
    constexpr double kC1 = 1.0, kC2 = 0.16666666685227835064, kC3 = 3.0000000027955394;
    const uint64_t mantissa = c.Mantissa[indexBits & ((1u << kTableBits) - 1)];
    const uint64_t power = (((indexBits + kAdjust) >> kTableBits) << 52) | mantissa;
    double t = rounded - kMagic;
    t = t * c.InvScale;
    t = t - x;
    double y = kC3 - t;
    y = y * (t * t);
    y = y * kC2;
    y = y - t;
    y = y + kC1;
    double powerOfTwo;
    std::memcpy(&powerOfTwo, &power, sizeof(powerOfTwo));
    return y * powerOfTwo;
}

inline double RoundedArgument(const TExpTable& c, double x) {
    constexpr double kMagic = static_cast<double>(uint64_t(3) << 51);
    double d = x * c.Scale;
    d = d + kMagic;  // the integer part of x * 2048 / ln 2 lands in the low mantissa bits
    return d;
}

}  // namespace

TFastExpConstants FastExpConstants() {
    const TExpTable& c = Table();
    static_assert(sizeof(unsigned long long) == sizeof(uint64_t), "64-bit table entries");
    return {reinterpret_cast<const unsigned long long*>(c.Mantissa), c.Scale, c.InvScale};
}

void FastExpInplace(double* x, size_t count) {
    const TExpTable& c = Table();
    const size_t vectorCount = count & ~size_t(3);
    for (size_t i = 0; i < vectorCount; ++i) {
        // min_pd / max_pd return their second operand whenever the compare fails, NaN included
        double v = x[i];
        v = v < 709.78272569338397 ? v : 709.78272569338397;
        v = v > -708.39641853226408 ? v : -708.39641853226408;
        const double d = RoundedArgument(c, v);
        uint64_t bits;
        std::memcpy(&bits, &d, sizeof(bits));
        x[i] = ExpFromRounded(c, v, d, bits);
    }
    for (size_t i = vectorCount; i < count; ++i) {
        const double v = x[i];
        if (v <= -708.39641853226408) {
            x[i] = 0;
        } else if (v >= 709.78271289338397) {
            x[i] = std::numeric_limits<double>::infinity();
        } else {
            const double d = RoundedArgument(c, v);
            uint64_t bits;
            std::memcpy(&bits, &d, sizeof(bits));
            // the scalar form reads the low 32 bits as a signed int
            const uint64_t low = static_cast<uint64_t>(static_cast<int64_t>(static_cast<int32_t>(static_cast<uint32_t>(bits))));
            x[i] = ExpFromRounded(c, v, d, low);
        }
    }
}

}  // namespace cbamd
