// CityHash64 v1.0 (Geoff Pike, Jyrki Alakuijala; published algorithm). The reference vendors the
// same version in util/digest/city.cpp:58-200; categorical values are hashed with it so the
// constants, rotations and the order of operations below are fixed by the model format.
#include "cat_hash.h"

#include <utility>

namespace cbamd {
namespace {

constexpr uint64_t kPrime0 = 0xc3a5c85c97cb3127ULL;
constexpr uint64_t kPrime1 = 0xb492b66fbe98f273ULL;
constexpr uint64_t kPrime2 = 0x9ae16a3b2f90404fULL;
constexpr uint64_t kPrime3 = 0xc949d7c7509e6557ULL;
constexpr uint64_t kMurmurMul = 0x9ddfea08eb382d69ULL;

struct TBytes {
    const char* P;
    uint64_t U64(size_t at) const {
        uint64_t v;
        std::memcpy(&v, P + at, sizeof(v));
        return v;
    }
    uint64_t U32(size_t at) const {
        uint32_t v;
        std::memcpy(&v, P + at, sizeof(v));
        return v;
    }
    uint8_t U8(size_t at) const { return static_cast<uint8_t>(P[at]); }
};

inline uint64_t Ror(uint64_t v, unsigned s) { return s ? (v >> s) | (v << (64 - s)) : v; }
inline uint64_t Mix47(uint64_t v) { return v ^ (v >> 47); }

// 128 -> 64 bit fold (util/digest/city.h:36-45)
inline uint64_t Fold(uint64_t lo, uint64_t hi) {
    uint64_t a = Mix47((lo ^ hi) * kMurmurMul);
    uint64_t b = Mix47((hi ^ a) * kMurmurMul);
    return b * kMurmurMul;
}

uint64_t Short(TBytes s, size_t n) {  // 0..16 bytes
    if (n > 8) {
        const uint64_t head = s.U64(0), tail = s.U64(n - 8);
        return Fold(head, Ror(tail + n, static_cast<unsigned>(n))) ^ tail;
    }
    if (n >= 4) {
        return Fold(n + (s.U32(0) << 3), s.U32(n - 4));
    }
    if (n > 0) {
        const uint32_t y = s.U8(0) + (static_cast<uint32_t>(s.U8(n >> 1)) << 8);
        const uint32_t z = static_cast<uint32_t>(n) + (static_cast<uint32_t>(s.U8(n - 1)) << 2);
        return Mix47(y * kPrime2 ^ z * kPrime3) * kPrime2;
    }
    return kPrime2;
}

uint64_t Medium(TBytes s, size_t n) {  // 17..32 bytes
    const uint64_t a = s.U64(0) * kPrime1, b = s.U64(8);
    const uint64_t c = s.U64(n - 8) * kPrime2, d = s.U64(n - 16) * kPrime0;
    return Fold(Ror(a - b, 43) + Ror(c, 30) + d, a + Ror(b ^ kPrime3, 20) - c + n);
}

using TPair = std::pair<uint64_t, uint64_t>;

TPair Weak32(TBytes s, size_t at, uint64_t a, uint64_t b) {
    const uint64_t w = s.U64(at), x = s.U64(at + 8), y = s.U64(at + 16), z = s.U64(at + 24);
    a += w;
    b = Ror(b + a + z, 21);
    const uint64_t c = a;
    a += x;
    a += y;
    b += Ror(a, 44);
    return {a + z, b + c};
}

uint64_t Long33to64(TBytes s, size_t n) {
    uint64_t z = s.U64(24);
    uint64_t a = s.U64(0) + (n + s.U64(n - 16)) * kPrime0;
    uint64_t b = Ror(a + z, 52);
    uint64_t c = Ror(a, 37);
    a += s.U64(8);
    c += Ror(a, 7);
    a += s.U64(16);
    const uint64_t vf = a + z, vs = b + Ror(a, 31) + c;
    a = s.U64(16) + s.U64(n - 32);
    z = s.U64(n - 8);
    b = Ror(a + z, 52);
    c = Ror(a, 37);
    a += s.U64(n - 24);
    c += Ror(a, 7);
    a += s.U64(n - 16);
    const uint64_t wf = a + z, ws = b + Ror(a, 31) + c;
    const uint64_t r = Mix47((vf + ws) * kPrime2 + (wf + vs) * kPrime0);
    return Mix47(r * kPrime0 + vs) * kPrime2;
}

}  // namespace

uint64_t CityHash64(const char* data, size_t n) noexcept {
    TBytes s{data};
    if (n <= 16) {
        return Short(s, n);
    }
    if (n <= 32) {
        return Medium(s, n);
    }
    if (n <= 64) {
        return Long33to64(s, n);
    }
    uint64_t x = s.U64(0);
    uint64_t y = s.U64(n - 16) ^ kPrime1;
    uint64_t z = s.U64(n - 56) ^ kPrime0;
    TPair v = Weak32(s, n - 64, n, y);
    TPair w = Weak32(s, n - 32, n * kPrime1, kPrime0);
    z += Mix47(v.second) * kPrime1;
    x = Ror(z + x, 39) * kPrime1;
    y = Ror(y, 33) * kPrime1;
    size_t at = 0;
    for (size_t left = (n - 1) & ~static_cast<size_t>(63); left != 0; left -= 64, at += 64) {
        x = Ror(x + y + v.first + s.U64(at + 16), 37) * kPrime1;
        y = Ror(y + v.second + s.U64(at + 48), 42) * kPrime1;
        x ^= w.second;
        y ^= v.first;
        z = Ror(z ^ w.first, 33);
        v = Weak32(s, at, v.second * kPrime1, x + w.first);
        w = Weak32(s, at + 32, z + w.second, y);
        std::swap(z, x);
    }
    return Fold(Fold(v.first, w.first) + Mix47(y) * kPrime1 + z, Fold(v.second, w.second) + x);
}

}  // namespace cbamd
