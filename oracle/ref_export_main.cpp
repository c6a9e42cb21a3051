// Driver around a model that the reference holds as exported C++ code: the canonical outputs of its
// own export tests (catboost/python-package/ut/medium/canondata/test.test_cpp_export_*_CPU_/model.cpp,
// written by catboost/libs/model/model_export/cpp_exporter.cpp: the model's tables as static data plus
// the applier of model_export/resources/apply_catboost_model*.cpp). The file is compiled where it
// lies, named by -DMODEL_SOURCE; -DWITH_CATS=1 for the model with categorical features.
// Built by oracle/build_ref.sh into oracle/_ref/export_{cat,nocat}.
//
// TEST INFRASTRUCTURE ONLY.
//   export_* dump                  prints the model's tables as JSON
//   export_* apply IN.bin OUT.f64  IN: uint32 docs, then per doc FloatFeatureCount float32 and
//                                  CatFeatureCount int32 hashed values (looked up by value in the
//                                  model's own string -> hash table; any other value is an unknown
//                                  category); OUT: docs x Dimension float64 from ApplyCatboostModelMulti
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include MODEL_SOURCE

namespace {

void PrintFloats(const std::vector<float>& values) {
    std::printf("[");
    for (size_t i = 0; i < values.size(); ++i) {
        std::printf("%s%.9g", i ? ", " : "", values[i]);
    }
    std::printf("]");
}

template <typename T>
void PrintInts(const char* name, const T* values, size_t count) {
    std::printf("\"%s\": [", name);
    for (size_t i = 0; i < count; ++i) {
        std::printf("%s%lld", i ? ", " : "", static_cast<long long>(values[i]));
    }
    std::printf("],\n");
}

void PrintBorders(const char* name, const std::vector<std::vector<float>>& borders) {
    std::printf("\"%s\": [", name);
    for (size_t i = 0; i < borders.size(); ++i) {
        std::printf("%s", i ? ", " : "");
        PrintFloats(borders[i]);
    }
    std::printf("],\n");
}

int Dump() {
    const CatboostModel& m = CatboostModelStatic;
    size_t splits = 0;
    size_t leaves = 0;
    for (unsigned int t = 0; t < m.TreeCount; ++t) {
        splits += m.TreeDepth[t];
        leaves += size_t(1) << m.TreeDepth[t];
    }
    std::printf("{\n\"float_feature_count\": %u, \"cat_feature_count\": %u, \"binary_feature_count\": %u,\n",
                m.FloatFeatureCount, m.CatFeatureCount, m.BinaryFeatureCount);
    std::printf("\"dimension\": %u, \"scale\": %.17g,\n", m.Dimension, m.Scale);
    PrintBorders("float_feature_borders", m.FloatFeatureBorders);
    PrintInts("tree_depth", m.TreeDepth, m.TreeCount);
    PrintInts("tree_splits", m.TreeSplits, splits);
#if WITH_CATS
    PrintInts("tree_split_idxs", m.TreeSplitIdxs, splits);
    PrintInts("tree_split_feature_index", m.TreeSplitFeatureIndex, splits);
    PrintInts("tree_split_xor_mask", m.TreeSplitXorMask, splits);
#endif
    std::printf("\"biases\": [");
    for (unsigned int d = 0; d < m.Dimension; ++d) {
        std::printf("%s%.17g", d ? ", " : "", m.Biases[d]);
    }
    std::printf("],\n\"leaf_values\": [");
    for (size_t l = 0; l < leaves; ++l) {
        for (unsigned int d = 0; d < m.Dimension; ++d) {
            std::printf("%s%.17g", (l || d) ? ", " : "", m.LeafValues[l][d]);
        }
    }
    std::printf("]");
#if WITH_CATS
    std::printf(",\n");
    PrintInts("cat_features_index", m.CatFeaturesIndex, m.CatFeatureCount);
    PrintInts("one_hot_cat_feature_index", m.OneHotCatFeatureIndex.data(), m.OneHotCatFeatureIndex.size());
    std::printf("\"one_hot_hash_values\": [");
    for (size_t i = 0; i < m.OneHotHashValues.size(); ++i) {
        std::printf("%s[", i ? ", " : "");
        for (size_t j = 0; j < m.OneHotHashValues[i].size(); ++j) {
            std::printf("%s%d", j ? ", " : "", m.OneHotHashValues[i][j]);
        }
        std::printf("]");
    }
    std::printf("],\n");
    PrintBorders("ctr_feature_borders", m.CtrFeatureBorders);
    std::printf("\"cat_feature_hashes\": {");
    bool first = true;
    for (const auto& kv : CatFeatureHashes) {
        std::printf("%s\"%s\": %d", first ? "" : ", ", kv.first.c_str(), kv.second);
        first = false;
    }
    std::printf("},\n\"projections\": [");
    for (size_t p = 0; p < m.modelCtrs.CompressedModelCtrs.size(); ++p) {
        const auto& c = m.modelCtrs.CompressedModelCtrs[p];
        std::printf("%s{\"transposed_cat_feature_indexes\": [", p ? ",\n" : "\n");
        for (size_t i = 0; i < c.Projection.transposedCatFeatureIndexes.size(); ++i) {
            std::printf("%s%d", i ? ", " : "", c.Projection.transposedCatFeatureIndexes[i]);
        }
        std::printf("], \"binarized_indexes\": [");
        for (size_t i = 0; i < c.Projection.binarizedIndexes.size(); ++i) {
            const auto& b = c.Projection.binarizedIndexes[i];
            std::printf("%s[%u, %d, %u]", i ? ", " : "", b.BinIndex, b.CheckValueEqual ? 1 : 0, unsigned(b.Value));
        }
        std::printf("], \"ctrs\": [");
        for (size_t i = 0; i < c.ModelCtrs.size(); ++i) {
            const auto& ctr = c.ModelCtrs[i];
            std::printf("%s{\"base_hash\": \"%llu\", \"type\": %d, \"target_border_idx\": %d, \"prior_num\": %.9g, "
                        "\"prior_denom\": %.9g, \"shift\": %.9g, \"scale\": %.9g}",
                        i ? ", " : "", ctr.BaseHash, static_cast<int>(ctr.BaseCtrType), ctr.TargetBorderIdx,
                        ctr.PriorNum, ctr.PriorDenom, ctr.Shift, ctr.Scale);
        }
        std::printf("]}");
    }
    std::printf("],\n\"tables\": {");
    first = true;
    for (const auto& kv : m.modelCtrs.CtrData.LearnCtrs) {
        const auto& t = kv.second;
        std::printf("%s\n\"%llu\": {\"target_classes_count\": %d, \"counter_denominator\": %d, \"index\": [",
                    first ? "" : ",", kv.first, t.TargetClassesCount, t.CounterDenominator);
        first = false;
        bool firstKey = true;
        for (const auto& entry : t.IndexHashViewer) {
            std::printf("%s[\"%llu\", %u]", firstKey ? "" : ", ", entry.first, entry.second);
            firstKey = false;
        }
        std::printf("], \"mean_history\": [");
        for (size_t i = 0; i < t.CtrMeanHistory.size(); ++i) {
            std::printf("%s[%.9g, %d]", i ? ", " : "", t.CtrMeanHistory[i].Sum, t.CtrMeanHistory[i].Count);
        }
        std::printf("], \"total\": [");
        for (size_t i = 0; i < t.CtrTotal.size(); ++i) {
            std::printf("%s%d", i ? ", " : "", t.CtrTotal[i]);
        }
        std::printf("]}");
    }
    std::printf("}");
#endif
    std::printf("\n}\n");
    return 0;
}

int Apply(const char* inPath, const char* outPath) {
    const CatboostModel& m = CatboostModelStatic;
    std::FILE* in = std::fopen(inPath, "rb");
    std::FILE* out = std::fopen(outPath, "wb");
    if (!in || !out) {
        return 1;
    }
    unsigned int docs = 0;
    if (std::fread(&docs, 4, 1, in) != 1) {
        return 1;
    }
#if WITH_CATS
    std::unordered_map<int, std::string> stringOfHash;
    for (const auto& kv : CatFeatureHashes) {
        stringOfHash[kv.second] = kv.first;
    }
#endif
    std::vector<float> floats(m.FloatFeatureCount);
    std::vector<int> hashes(m.CatFeatureCount);
    for (unsigned int d = 0; d < docs; ++d) {
        if (std::fread(floats.data(), 4, floats.size(), in) != floats.size() ||
            std::fread(hashes.data(), 4, hashes.size(), in) != hashes.size()) {
            std::fprintf(stderr, "input ends early\n");
            return 1;
        }
#if WITH_CATS
        std::vector<std::string> cats;
        for (int h : hashes) {
            const auto it = stringOfHash.find(h);
            cats.push_back(it == stringOfHash.end() ? std::string("\x01 no such category") : it->second);
        }
        const std::vector<double> result = ApplyCatboostModelMulti(floats, cats);
#else
        const std::vector<double> result = ApplyCatboostModelMulti(floats);
#endif
        std::fwrite(result.data(), sizeof(double), result.size(), out);
    }
    std::fclose(in);
    std::fclose(out);
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc == 2 && std::strcmp(argv[1], "dump") == 0) {
        return Dump();
    }
    if (argc == 4 && std::strcmp(argv[1], "apply") == 0) {
        return Apply(argv[2], argv[3]);
    }
    std::fprintf(stderr, "usage: %s dump | apply IN.bin OUT.f64\n", argv[0]);
    return 2;
}
