// Driver around the reference's vendored fmath (contrib/libs/fmath/fmath.hpp), the exponent behind
// NCB::FastExpWithInfInplace on AVX2 hosts (catboost/libs/helpers/math_utils.cpp:14-27,
// library/cpp/fast_exp/fast_exp_avx2.cpp). Built by oracle/build_ref.sh into oracle/_ref/fmath_exp.
//   fmath_exp IN.f64 OUT.f64 CHUNK   applies fmath::expd_v to consecutive runs of CHUNK doubles
//                                    (the last run may be shorter), as the callers apply it to
//                                    blocks and to single documents
#include <contrib/libs/fmath/fmath.hpp>

#include <cstdio>
#include <cstdlib>
#include <vector>

int main(int argc, char** argv) {
    if (argc != 4) {
        std::fprintf(stderr, "usage: fmath_exp IN.f64 OUT.f64 CHUNK\n");
        return 2;
    }
    std::FILE* in = std::fopen(argv[1], "rb");
    if (!in) {
        return 1;
    }
    std::vector<double> data;
    double buf[4096];
    size_t got;
    while ((got = std::fread(buf, sizeof(double), 4096, in)) > 0) {
        data.insert(data.end(), buf, buf + got);
    }
    std::fclose(in);
    const size_t chunk = std::strtoull(argv[3], nullptr, 10);
    for (size_t begin = 0; begin < data.size(); begin += chunk) {
        const size_t n = data.size() - begin < chunk ? data.size() - begin : chunk;
        fmath::expd_v(data.data() + begin, n);
    }
    std::FILE* out = std::fopen(argv[2], "wb");
    if (!out) {
        return 1;
    }
    std::fwrite(data.data(), sizeof(double), data.size(), out);
    std::fclose(out);
    return 0;
}
