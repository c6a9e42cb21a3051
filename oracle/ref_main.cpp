// Driver around the reference's own standalone evaluator
// (catboost/libs/standalone_evaluator/evaluator.{h,cpp}), built by oracle/build_ref.sh from the
// sources under /root/reference. TEST INFRASTRUCTURE ONLY.
//
//   standalone_eval verify MODEL.cbm            runs the reference flatbuffers verifier on the core
//   standalone_eval apply MODEL.cbm DOCS.f32 N   N docs of raw float32 rows; prints one %.17g per doc
#include "evaluator.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

static std::vector<unsigned char> ReadAll(const char* path) {
    std::ifstream f(path, std::ios::binary);
    return std::vector<unsigned char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

int main(int argc, char** argv) {
    if (argc < 3) {
        std::fprintf(stderr, "usage: %s verify|apply model.cbm [docs.f32 doc_count]\n", argv[0]);
        return 2;
    }
    const std::string mode = argv[1];
    std::vector<unsigned char> blob = ReadAll(argv[2]);
    if (blob.size() < 8 || std::memcmp(blob.data(), "CBM1", 4) != 0) {
        std::fprintf(stderr, "not a CBM1 file\n");
        return 1;
    }
    unsigned int coreSize;
    std::memcpy(&coreSize, blob.data() + 4, 4);
    if (mode == "verify") {
        flatbuffers::Verifier verifier(blob.data() + 8, coreSize, 64, 256000000);
        const bool ok = NCatBoostFbs::VerifyTModelCoreBuffer(verifier);
        std::printf("%s\n", ok ? "OK" : "FAILED");
        return ok ? 0 : 1;
    }
    if (argc < 5) {
        return 2;
    }
    NCatboostStandalone::TOwningEvaluator evaluator(blob);
    std::vector<unsigned char> docs = ReadAll(argv[3]);
    const size_t n = std::strtoull(argv[4], nullptr, 10);
    if (n == 0 || docs.size() % (n * sizeof(float)) != 0) {
        std::fprintf(stderr, "document file size does not match the document count\n");
        return 1;
    }
    const size_t width = docs.size() / sizeof(float) / n;
    const float* p = reinterpret_cast<const float*>(docs.data());
    for (size_t i = 0; i < n; ++i) {
        std::vector<float> row(p + i * width, p + (i + 1) * width);
        std::printf("%.17g\n", evaluator.Apply(row, NCatboostStandalone::EPredictionType::RawValue));
    }
    return 0;
}
