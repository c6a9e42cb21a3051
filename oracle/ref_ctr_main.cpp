// Driver around the CTR calculator that the reference ships for exported models
// (catboost/libs/model/model_export/resources/ctr_structs.cpp and ctr_calcer.cpp: CalcHash, CalcCtrs with
// all six CTR types). Those two files are fragments without includes; they are compiled where they lie,
// under the includes below. Built by oracle/build_ref.sh into oracle/_ref/ctr_calc.
//
// TEST INFRASTRUCTURE ONLY. The model tables come from a file of 32-bit words (not from generated code):
//   ctr_calc IN.words OUT.f32
// IN:  projections, { cats, { cat position }*, bins, { bin index, check equal, value }*, ctrs,
//                     { table id, type, target border idx, prior num, prior denom, shift, scale }* }*
//      tables, { id, target classes, counter denominator, index size, { hash lo, hash hi, row }*,
//                means, { sum, count }*, totals, { total }* }*
//      docs, bins per doc, cats per doc, then per doc { bin }* { hashed cat }*
// OUT: docs x ctrs float32 values in the order CalcCtrs writes them.
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <unordered_map>
#include <vector>

#include <catboost/libs/model/model_export/resources/ctr_structs.cpp>
#include <catboost/libs/model/model_export/resources/ctr_calcer.cpp>

namespace {

struct TWords {
    std::vector<unsigned int> Data;
    size_t Pos = 0;
    unsigned int U() {
        if (Pos >= Data.size()) {
            std::fprintf(stderr, "input ends early\n");
            std::exit(1);
        }
        return Data[Pos++];
    }
    int I() {
        const unsigned int v = U();
        int r;
        std::memcpy(&r, &v, 4);
        return r;
    }
    float F() {
        const unsigned int v = U();
        float r;
        std::memcpy(&r, &v, 4);
        return r;
    }
};

}  // namespace

int main(int argc, char** argv) {
    if (argc != 3) {
        std::fprintf(stderr, "usage: ctr_calc IN.words OUT.f32\n");
        return 2;
    }
    TWords in;
    {
        std::FILE* f = std::fopen(argv[1], "rb");
        if (!f) {
            return 1;
        }
        unsigned int buf[4096];
        size_t got;
        while ((got = std::fread(buf, 4, 4096, f)) > 0) {
            in.Data.insert(in.Data.end(), buf, buf + got);
        }
        std::fclose(f);
    }
    TCatboostCPPExportModelCtrs model;
    model.UsedModelCtrsCount = 0;
    const unsigned int projections = in.U();
    for (unsigned int p = 0; p < projections; ++p) {
        TCatboostCPPExportCompressedModelCtr compressed;
        for (unsigned int n = in.U(); n > 0; --n) {
            compressed.Projection.transposedCatFeatureIndexes.push_back(in.I());
        }
        for (unsigned int n = in.U(); n > 0; --n) {
            TCatboostCPPExportBinFeatureIndexValue bin;
            bin.BinIndex = in.U();
            bin.CheckValueEqual = in.U() != 0;
            bin.Value = static_cast<unsigned char>(in.U());
            compressed.Projection.binarizedIndexes.push_back(bin);
        }
        for (unsigned int n = in.U(); n > 0; --n) {
            TCatboostCPPExportModelCtr ctr;
            ctr.BaseHash = in.U();
            ctr.BaseCtrType = static_cast<ECatboostCPPExportModelCtrType>(in.I());
            ctr.TargetBorderIdx = in.I();
            ctr.PriorNum = in.F();
            ctr.PriorDenom = in.F();
            ctr.Shift = in.F();
            ctr.Scale = in.F();
            compressed.ModelCtrs.push_back(ctr);
            ++model.UsedModelCtrsCount;
        }
        model.CompressedModelCtrs.push_back(compressed);
    }
    const unsigned int tables = in.U();
    for (unsigned int t = 0; t < tables; ++t) {
        const unsigned int id = in.U();
        TCatboostCPPExportCtrValueTable& table = model.CtrData.LearnCtrs[id];
        table.TargetClassesCount = in.I();
        table.CounterDenominator = in.I();
        for (unsigned int n = in.U(); n > 0; --n) {
            const unsigned long long lo = in.U();
            const unsigned long long hi = in.U();
            table.IndexHashViewer[lo | (hi << 32)] = in.U();
        }
        for (unsigned int n = in.U(); n > 0; --n) {
            TCatboostCPPExportCtrMeanHistory mean;
            mean.Sum = in.F();
            mean.Count = in.I();
            table.CtrMeanHistory.push_back(mean);
        }
        for (unsigned int n = in.U(); n > 0; --n) {
            table.CtrTotal.push_back(in.I());
        }
    }
    const unsigned int docs = in.U();
    const unsigned int binsPerDoc = in.U();
    const unsigned int catsPerDoc = in.U();
    std::FILE* out = std::fopen(argv[2], "wb");
    if (!out) {
        return 1;
    }
    std::vector<unsigned char> bins(binsPerDoc);
    std::vector<int> cats(catsPerDoc);
    std::vector<float> result(model.UsedModelCtrsCount);
    for (unsigned int d = 0; d < docs; ++d) {
        for (auto& b : bins) {
            b = static_cast<unsigned char>(in.U());
        }
        for (auto& c : cats) {
            c = in.I();
        }
        CalcCtrs(model, bins, cats, result);
        std::fwrite(result.data(), sizeof(float), result.size(), out);
    }
    std::fclose(out);
    return 0;
}
