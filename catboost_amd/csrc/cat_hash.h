// Hash of a categorical feature value: CityHash64 (version 1.0, as pinned by the reference in
// util/digest/city.h:8-9) truncated to 32 bits, catboost/libs/cat_feature/cat_feature.cpp:6-8.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>

namespace cbamd {

uint64_t CityHash64(const char* s, size_t len) noexcept;

inline uint32_t CalcCatFeatureHash(const char* s, size_t len) noexcept {
    return static_cast<uint32_t>(CityHash64(s, len) & 0xffffffffULL);
}

inline int CalcCatFeatureHashInt(const char* s, size_t len) noexcept {
    const uint32_t h = CalcCatFeatureHash(s, len);
    int r;
    std::memcpy(&r, &h, sizeof(r));
    return r;
}

}  // namespace cbamd
