// C++ client written against the reference's own header-only wrapper
// (catboost/libs/model_interface/wrapped_calcer.h, which includes the reference's c_api.h) and linked
// against this repository's libcatboostmodel.so: what a user of the reference library compiles unchanged.
//
// Usage: wrapped_calcer_client model.cbm < documents
// One document per input line: float features, then '|', then categorical features as strings.
// Prints one line per way of calling the model, "<name> <prediction>...".
#include <wrapped_calcer.h>

#include <cstdio>
#include <fstream>
#include <iostream>
#include <iterator>
#include <sstream>

namespace {

void PrintLine(const char* name, const std::vector<double>& values) {
    std::printf("%s", name);
    for (double v : values) {
        std::printf(" %.17g", v);
    }
    std::printf("\n");
}

}  // namespace

int main(int argc, char** argv) {
    if (argc != 2) {
        std::fprintf(stderr, "usage: %s model.cbm < documents\n", argv[0]);
        return 2;
    }
    std::vector<std::vector<float>> floats;
    std::vector<std::vector<std::string>> cats;
    for (std::string line; std::getline(std::cin, line);) {
        if (line.empty()) {
            continue;
        }
        std::istringstream in(line);
        floats.emplace_back();
        cats.emplace_back();
        bool inCats = false;
        for (std::string token; in >> token;) {
            if (token == "|") {
                inCats = true;
            } else if (inCats) {
                cats.back().push_back(token);
            } else {
                floats.back().push_back(std::stof(token));
            }
        }
    }
    try {
        ModelCalcerWrapper calcer{std::string(argv[1])};
        calcer.EnableGPUEvaluation(0);
        std::printf("counts %zu %zu %zu %zu %zu\n", calcer.GetTreeCount(), calcer.GetFloatFeaturesCount(),
                    calcer.GetCatFeaturesCount(), calcer.GetTextFeaturesCount(), calcer.GetEmbeddingFeaturesCount());
        std::printf("evaluators %zu\n", calcer.GetSupportedEvaluatorTypes().size());
        std::printf("names");
        for (const auto& name : calcer.GetUsedFeaturesNames()) {
            std::printf(" %s", name.c_str());
        }
        std::printf("\n");
        std::printf("float_indices");
        for (size_t index : calcer.GetFloatFeatureIndices()) {
            std::printf(" %zu", index);
        }
        std::printf("\ncat_indices");
        for (size_t index : calcer.GetCatFeatureIndices()) {
            std::printf(" %zu", index);
        }
        std::printf("\n");
        std::printf("has_params %d\n", calcer.CheckMetadataHasKey("params") ? 1 : 0);
        std::printf("missing_key [%s]\n", calcer.GetMetadataKeyValue("no such key").c_str());

        std::vector<double> single;
        for (size_t i = 0; i < floats.size(); ++i) {
            single.push_back(calcer.Calc(floats[i], cats[i]));
        }
        PrintLine("single", single);
        PrintLine("batch", calcer.Calc(floats, cats));

        std::vector<std::vector<int>> hashes;
        for (const auto& doc : cats) {
            hashes.emplace_back();
            for (const auto& value : doc) {
                hashes.back().push_back(GetStringCatFeatureHash(value.data(), value.size()));
            }
        }
        PrintLine("hashed", calcer.CalcHashed(floats, hashes));

        if (calcer.GetCatFeaturesCount() == 0) {
            std::vector<double> flatSingle;
            for (const auto& doc : floats) {
                flatSingle.push_back(calcer.CalcFlat(doc));
            }
            PrintLine("flat_single", flatSingle);
            PrintLine("flat", calcer.CalcFlat(floats));
            std::vector<std::vector<float>> columns(floats.empty() ? 0 : floats[0].size());
            for (const auto& doc : floats) {
                for (size_t f = 0; f < columns.size(); ++f) {
                    columns[f].push_back(doc[f]);
                }
            }
            PrintLine("flat_transposed", calcer.CalcFlatTransposed(columns));
        }

        // the same model from memory, on a second handle
        std::ifstream file(argv[1], std::ios::binary);
        const std::string bytes((std::istreambuf_iterator<char>(file)), std::istreambuf_iterator<char>());
        ModelCalcerWrapper fromMemory(bytes.data(), bytes.size());
        fromMemory.EnableGPUEvaluation(0);
        PrintLine("from_memory", fromMemory.Calc(floats, cats));

        // a wrong document is an exception with the library's message, and the handle keeps working
        try {
            calcer.Calc(std::vector<float>(), cats.empty() ? std::vector<std::string>() : cats[0]);
            std::printf("short_document accepted\n");
        } catch (const std::runtime_error& e) {
            std::printf("short_document refused\n");
        }
        PrintLine("after_error", calcer.Calc(floats, cats));
    } catch (const std::exception& e) {
        std::fprintf(stderr, "failed: %s\n", e.what());
        return 1;
    }
    return 0;
}
