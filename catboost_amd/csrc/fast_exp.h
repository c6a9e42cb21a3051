// The exponent the reference applies to raw formula values (prediction types Probability,
// Exponent, MultiProbability, RMSEWithUncertainty).
#pragma once

#include <cstddef>

namespace cbamd {

// x[i] = exp(x[i]) the way NCB::FastExpWithInfInplace computes it on an x86 host with AVX2
// (catboost/libs/helpers/math_utils.cpp:14-27 -> library/cpp/fast_exp/fast_exp_avx2.cpp ->
// fmath::expd_v, contrib/libs/fmath/fmath.hpp:565-648): a 2048-entry table of 2^(i/2048) and a cubic
// in the remainder. Values at positions below count & ~3 go through the vector form (arguments
// clamped to [-708.396, 709.783], NaN treated as the upper clamp), the last count & 3 through
// fmath::expd (:474-512: 0 below the lower bound, +inf above the upper one).
void FastExpInplace(double* x, size_t count);

// The constants behind it, for the device version of the same arithmetic: 2048 mantissas of
// 2^(i / 2048), then 2048 / ln 2 and its reciprocal.
struct TFastExpConstants {
    const unsigned long long* Mantissa;
    double Scale;
    double InvScale;
};
TFastExpConstants FastExpConstants();

}  // namespace cbamd
