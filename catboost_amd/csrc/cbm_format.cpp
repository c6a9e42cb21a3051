// .cbm reader / writer: "CBM1" + core size + flatbuffer TModelCore + trailing model parts (the reader
// takes the tables of the static CTR provider and refuses text / embedding parts; the writer emits none).
// Follows TFullModel::Save / Load (catboost/libs/model/model.cpp:1113-1228), the schemas
// catboost/libs/model/flatbuffers/model.fbs:22-54, features.fbs:5-75 and ctr_data.fbs:5-43 (vtable slot =
// field declaration order) and the size prefix of util/ysaveload.h:277-296.
#include "flatbuf.h"
#include "model.h"

#include <cstdio>
#include <fstream>

namespace cbamd {

namespace {

constexpr char kFormatString[] = "FlabuffersModel_v1";  // sic, model.cpp:53

// slots of TModelTrees (model.fbs:22-46)
enum ETreesSlot {
    TS_ApproxDimension = 0, TS_TreeSplits, TS_TreeSizes, TS_TreeStartOffsets, TS_CatFeatures, TS_FloatFeatures,
    TS_OneHotFeatures, TS_CtrFeatures, TS_LeafValues, TS_LeafWeights, TS_NonSymmetricStepNodes,
    TS_NonSymmetricNodeIdToLeafId, TS_TextFeatures, TS_EstimatedFeatures, TS_Scale, TS_Bias, TS_MultiBias,
    TS_RepackedBins, TS_EmbeddingFeatures
};

// TModelCtrBase / TFeatureCombination, ctr_data.fbs:15-19 and features.fbs:71-75
// (TModelCtrBase::FBDeserialize, TFeatureCombination::FBDeserialize, online_ctr.cpp:17-26, 72-95)
TModelCtrBase ReadCtrBase(const fb::TTable& t) {
    TModelCtrBase base;
    if (!t.Valid()) {
        return base;
    }
    const fb::TTable proj = t.Table(0);
    if (proj.Valid()) {
        base.Projection.CatFeatures = proj.Vector<int>(0);
        static_assert(sizeof(TFloatSplit) == 8 && sizeof(TOneHotSplit) == 8, "splits are two 4-byte fields");
        base.Projection.BinFeatures = proj.Vector<TFloatSplit>(1);
        base.Projection.OneHotFeatures = proj.Vector<TOneHotSplit>(2);
    }
    const int8_t type = t.Scalar<int8_t>(1, 0);
    CBAMD_ENSURE(type >= 0 && type <= 5, "unknown CTR type in model");
    base.CtrType = static_cast<ECtrType>(type);
    base.TargetBorderClassifierIdx = t.Scalar<int32_t>(2, 0);
    return base;
}

// TCtrFeature / TModelCtr, ctr_data.fbs:21-33 (TModelCtr::FBDeserialize, online_ctr.cpp:41-48)
TCtrFeature ReadCtrFeature(const fb::TTable& t) {
    TCtrFeature f;
    const fb::TTable ctr = t.Table(0);
    CBAMD_ENSURE(ctr.Valid(), "CTR feature without a CTR description");
    f.Ctr.Base = ReadCtrBase(ctr.Table(0));
    f.Ctr.TargetBorderIdx = ctr.Scalar<int32_t>(1, 0);
    f.Ctr.PriorNum = ctr.Scalar<float>(2, 0.f);
    f.Ctr.PriorDenom = ctr.Scalar<float>(3, 1.f);
    f.Ctr.Shift = ctr.Scalar<float>(4, 0.f);
    f.Ctr.Scale = ctr.Scalar<float>(5, 1.f);
    f.Borders = t.Vector<float>(1);
    return f;
}

// LoadSize of util/ysaveload.h:277-296: u32, or 0xffffffff followed by a u64
uint64_t ReadSize(const uint8_t* p, size_t size, size_t* pos) {
    CBAMD_ENSURE(*pos + 4 <= size, "Failed to read model part: file is truncated");
    uint32_t s32;
    std::memcpy(&s32, p + *pos, 4);
    *pos += 4;
    if (s32 != 0xffffffffu) {
        return s32;
    }
    CBAMD_ENSURE(*pos + 8 <= size, "Failed to read model part: file is truncated");
    uint64_t s64;
    std::memcpy(&s64, p + *pos, 8);
    *pos += 8;
    return s64;
}

// TCtrData::Load (ctr_data.cpp:24-34): a count, then per table a size and a flatbuffer whose
// root is TCtrValueTable (ctr_data.fbs:35-41; TCtrValueTable::LoadSolid, ctr_value_table.cpp:57-71)
void ReadStaticCtrProvider(const uint8_t* p, size_t size, size_t* pos, std::vector<TCtrValueTable>* tables) {
    const uint64_t count = ReadSize(p, size, pos);
    tables->clear();
    for (uint64_t i = 0; i < count; ++i) {
        const uint64_t len = ReadSize(p, size, pos);
        CBAMD_ENSURE(len >= 8 && len <= size - *pos, "Failed to read CTR value table: file is truncated");
        fb::TReader reader(p + *pos, static_cast<size_t>(len));
        const fb::TTable t = fb::GetRoot(reader);
        TCtrValueTable table;
        table.ModelCtrBase = ReadCtrBase(t.Table(0));
        table.IndexHashRaw = t.Vector<uint8_t>(1);
        table.CTRBlob = t.Vector<uint8_t>(2);
        table.CounterDenominator = t.Scalar<int32_t>(3, 0);
        table.TargetClassesCount = t.Scalar<int32_t>(4, 0);
        *pos += static_cast<size_t>(len);
        // a later table with the same key replaces an earlier one, as the hash map insert does
        bool replaced = false;
        for (auto& old : *tables) {
            if (old.ModelCtrBase == table.ModelCtrBase) {
                old = std::move(table);
                replaced = true;
                break;
            }
        }
        if (!replaced) {
            tables->push_back(std::move(table));
        }
    }
}

void ReadTrees(const fb::TTable& t, TModelTrees* trees) {
    *trees = TModelTrees();
    trees->ApproxDimension = t.Scalar<int32_t>(TS_ApproxDimension, 0);
    CBAMD_ENSURE(trees->ApproxDimension >= 1, "model approx dimension must be positive");
    // a dimension that neither the leaf values nor the bias can back is a damaged file; refusing it here
    // keeps a corrupted field from turning into gigabytes of bias
    CBAMD_ENSURE(static_cast<size_t>(trees->ApproxDimension) <=
                     std::max<size_t>({t.VectorLen(TS_LeafValues), t.VectorLen(TS_MultiBias), size_t(1)}),
                 "model approx dimension exceeds the leaf values and the bias the file holds");
    trees->TreeSplits = t.Vector<int>(TS_TreeSplits);
    trees->TreeSizes = t.Vector<int>(TS_TreeSizes);
    trees->TreeStartOffsets = t.Vector<int>(TS_TreeStartOffsets);
    for (const auto& c : t.Tables(TS_CatFeatures)) {  // features.fbs:20-25
        TCatFeature f;
        f.Index = c.Scalar<int32_t>(0, -1);
        f.FlatIndex = c.Scalar<int32_t>(1, -1);
        f.FeatureId = c.String(2);
        f.UsedInModel = c.Scalar<uint8_t>(3, 1) != 0;
        trees->CatFeatures.push_back(std::move(f));
    }
    for (const auto& c : t.Tables(TS_FloatFeatures)) {  // features.fbs:11-18
        TFloatFeature f;
        f.HasNans = c.Scalar<uint8_t>(0, 0) != 0;
        f.Index = c.Scalar<int32_t>(1, -1);
        f.FlatIndex = c.Scalar<int32_t>(2, -1);
        f.Borders = c.Vector<float>(3);
        f.FeatureId = c.String(4);
        const int8_t nan = c.Scalar<int8_t>(5, 0);
        CBAMD_ENSURE(nan >= 0 && nan <= 2, "unknown NaN value treatment in model");
        f.NanValueTreatment = static_cast<ENanValueTreatment>(nan);
        trees->FloatFeatures.push_back(std::move(f));
    }
    for (const auto& c : t.Tables(TS_OneHotFeatures)) {  // features.fbs:55-59
        TOneHotFeature f;
        f.CatFeatureIndex = c.Scalar<int32_t>(0, -1);
        f.Values = c.Vector<int>(1);
        f.StringValues = c.Strings(2);
        trees->OneHotFeatures.push_back(std::move(f));
    }
    for (const auto& c : t.Tables(TS_CtrFeatures)) {
        trees->CtrFeatures.push_back(ReadCtrFeature(c));
    }
    trees->TextFeatureCount = t.VectorLen(TS_TextFeatures);
    trees->EstimatedFeatureCount = t.VectorLen(TS_EstimatedFeatures);
    trees->EmbeddingFeatureCount = t.VectorLen(TS_EmbeddingFeatures);
    trees->LeafValues = t.Vector<double>(TS_LeafValues);
    trees->LeafWeights = t.Vector<double>(TS_LeafWeights);
    {
        static_assert(sizeof(TNonSymmetricTreeStepNode) == 4, "step node must be two u16");
        trees->NonSymmetricStepNodes = t.Vector<TNonSymmetricTreeStepNode>(TS_NonSymmetricStepNodes);
    }
    trees->NonSymmetricNodeIdToLeafId = t.Vector<uint32_t>(TS_NonSymmetricNodeIdToLeafId);
    // TModelTrees::SetScaleAndBias(fbObj), model.cpp:711-722
    const double scale = t.Scalar<double>(TS_Scale, 1.0);
    std::vector<double> bias = t.Vector<double>(TS_MultiBias);
    if (bias.empty()) {
        const double b = t.Scalar<double>(TS_Bias, 0.0);
        CBAMD_ENSURE(trees->ApproxDimension == 1 || b == 0,
                     "Inappropraite dimension of bias, should be " + std::to_string(trees->ApproxDimension) + " found 1");
        bias.assign(trees->ApproxDimension, b);
    }
    trees->SetScaleAndBias(scale, bias);
    // RepackedBins stored in the file are recomputed by UpdateRuntimeData (model.cpp:1227, 543-576).
}

size_t WriteFloatFeature(fb::TWriter& w, const TFloatFeature& f) {
    fb::TWriter::TTableBuilder b;
    if (f.HasNans) {
        b.Scalar<uint8_t>(0, 1);
    }
    if (f.Index != -1) {
        b.Scalar<int32_t>(1, f.Index);
    }
    if (f.FlatIndex != -1) {
        b.Scalar<int32_t>(2, f.FlatIndex);
    }
    b.Ref(3);
    if (!f.FeatureId.empty()) {
        b.Ref(4);
    }
    if (f.NanValueTreatment != ENanValueTreatment::AsIs) {
        b.Scalar<int8_t>(5, static_cast<int8_t>(f.NanValueTreatment));
    }
    auto pos = w.WriteTable(b);
    w.PatchRef(pos.RefPos(3), w.WriteVector(f.Borders));
    if (!f.FeatureId.empty()) {
        w.PatchRef(pos.RefPos(4), w.WriteString(f.FeatureId));
    }
    return pos.Table;
}

size_t WriteCatFeature(fb::TWriter& w, const TCatFeature& f) {
    fb::TWriter::TTableBuilder b;
    if (f.Index != -1) {
        b.Scalar<int32_t>(0, f.Index);
    }
    if (f.FlatIndex != -1) {
        b.Scalar<int32_t>(1, f.FlatIndex);
    }
    if (!f.FeatureId.empty()) {
        b.Ref(2);
    }
    if (!f.UsedInModel) {
        b.Scalar<uint8_t>(3, 0);
    }
    auto pos = w.WriteTable(b);
    if (!f.FeatureId.empty()) {
        w.PatchRef(pos.RefPos(2), w.WriteString(f.FeatureId));
    }
    return pos.Table;
}

size_t WriteOneHotFeature(fb::TWriter& w, const TOneHotFeature& f) {
    fb::TWriter::TTableBuilder b;
    if (f.CatFeatureIndex != -1) {
        b.Scalar<int32_t>(0, f.CatFeatureIndex);
    }
    b.Ref(1);
    if (!f.StringValues.empty()) {
        b.Ref(2);
    }
    auto pos = w.WriteTable(b);
    w.PatchRef(pos.RefPos(1), w.WriteVector(f.Values));
    if (!f.StringValues.empty()) {
        auto vec = w.WriteRefVector(f.StringValues.size());
        w.PatchRef(pos.RefPos(2), vec.first);
        for (size_t i = 0; i < f.StringValues.size(); ++i) {
            w.PatchRef(vec.second + 4 * i, w.WriteString(f.StringValues[i]));
        }
    }
    return pos.Table;
}

// TModelCtrBase with its TFeatureCombination (ctr_data.fbs:15-19, features.fbs:71-75)
size_t WriteCtrBase(fb::TWriter& w, const TModelCtrBase& base) {
    fb::TWriter::TTableBuilder b;
    b.Ref(0);
    if (base.CtrType != ECtrType::Borders) {
        b.Scalar<int8_t>(1, static_cast<int8_t>(base.CtrType));
    }
    if (base.TargetBorderClassifierIdx != 0) {
        b.Scalar<int32_t>(2, base.TargetBorderClassifierIdx);
    }
    auto pos = w.WriteTable(b);
    fb::TWriter::TTableBuilder pb;
    pb.Ref(0);
    pb.Ref(1);
    pb.Ref(2);
    auto proj = w.WriteTable(pb);
    w.PatchRef(pos.RefPos(0), proj.Table);
    w.PatchRef(proj.RefPos(0), w.WriteVector(base.Projection.CatFeatures));
    w.PatchRef(proj.RefPos(1), w.WriteVector(base.Projection.BinFeatures.data(), base.Projection.BinFeatures.size(), 8, 4));
    w.PatchRef(proj.RefPos(2),
               w.WriteVector(base.Projection.OneHotFeatures.data(), base.Projection.OneHotFeatures.size(), 8, 4));
    return pos.Table;
}

// TCtrFeature with its TModelCtr (ctr_data.fbs:21-33)
size_t WriteCtrFeature(fb::TWriter& w, const TCtrFeature& f) {
    fb::TWriter::TTableBuilder b;
    b.Ref(0);
    b.Ref(1);
    auto pos = w.WriteTable(b);
    fb::TWriter::TTableBuilder cb;
    cb.Ref(0);
    if (f.Ctr.TargetBorderIdx != 0) {
        cb.Scalar<int32_t>(1, f.Ctr.TargetBorderIdx);
    }
    if (f.Ctr.PriorNum != 0.f) {
        cb.Scalar<float>(2, f.Ctr.PriorNum);
    }
    if (f.Ctr.PriorDenom != 1.f) {
        cb.Scalar<float>(3, f.Ctr.PriorDenom);
    }
    if (f.Ctr.Shift != 0.f) {
        cb.Scalar<float>(4, f.Ctr.Shift);
    }
    if (f.Ctr.Scale != 1.f) {
        cb.Scalar<float>(5, f.Ctr.Scale);
    }
    auto ctr = w.WriteTable(cb);
    w.PatchRef(pos.RefPos(0), ctr.Table);
    w.PatchRef(ctr.RefPos(0), WriteCtrBase(w, f.Ctr.Base));
    w.PatchRef(pos.RefPos(1), w.WriteVector(f.Borders));
    return pos.Table;
}

// SaveSize of util/ysaveload.h:277-296
void AppendSize(std::string* out, uint64_t size) {
    if (size < 0xffffffffu) {
        const uint32_t s = static_cast<uint32_t>(size);
        out->append(reinterpret_cast<const char*>(&s), 4);
    } else {
        const uint32_t marker = 0xffffffffu;
        out->append(reinterpret_cast<const char*>(&marker), 4);
        out->append(reinterpret_cast<const char*>(&size), 8);
    }
}

// TCtrData::Save (ctr_data.cpp:9-22): the number of tables, then each as a size and a flatbuffer
// whose root is TCtrValueTable (TCtrValueTable::Save, ctr_value_table.cpp:16-48)
void AppendStaticCtrProvider(std::string* out, const std::vector<TCtrValueTable>& tables) {
    AppendSize(out, tables.size());
    for (const auto& table : tables) {
        fb::TWriter w;
        fb::TWriter::TTableBuilder b;
        b.Ref(0);
        b.Ref(1);
        b.Ref(2);
        if (table.CounterDenominator != 0) {
            b.Scalar<int32_t>(3, table.CounterDenominator);
        }
        if (table.TargetClassesCount != 0) {
            b.Scalar<int32_t>(4, table.TargetClassesCount);
        }
        auto pos = w.WriteTable(b);
        w.SetRoot(pos.Table);
        w.PatchRef(pos.RefPos(0), WriteCtrBase(w, table.ModelCtrBase));
        w.PatchRef(pos.RefPos(1), w.WriteVector(table.IndexHashRaw));
        w.PatchRef(pos.RefPos(2), w.WriteVector(table.CTRBlob));
        const auto& buf = w.Buffer();
        AppendSize(out, buf.size());
        out->append(reinterpret_cast<const char*>(buf.data()), buf.size());
    }
}

template <typename T, typename F>
void WriteTableVector(fb::TWriter& w, size_t refPos, const std::vector<T>& items, F writeOne) {
    auto vec = w.WriteRefVector(items.size());
    w.PatchRef(refPos, vec.first);
    for (size_t i = 0; i < items.size(); ++i) {
        w.PatchRef(vec.second + 4 * i, writeOne(w, items[i]));
    }
}

}  // namespace

void TFullModel::Load(const void* data, size_t size) {
    const uint8_t* p = static_cast<const uint8_t*>(data);
    CBAMD_ENSURE(size >= 8 && std::memcmp(p, "CBM1", 4) == 0, "Incorrect model file descriptor");
    uint64_t coreSize = 0;
    {
        uint32_t s32;
        std::memcpy(&s32, p + 4, 4);
        coreSize = s32;
    }
    size_t pos = 8;
    if (coreSize == 0xffffffffu) {
        CBAMD_ENSURE(size >= 16, "Failed to read model core size");
        std::memcpy(&coreSize, p + 8, 8);
        pos = 16;
    }
    CBAMD_ENSURE(coreSize <= size - pos, "Failed to read model core: file is truncated");
    fb::TReader reader(p + pos, static_cast<size_t>(coreSize));
    CBAMD_ENSURE(coreSize >= 8, "Flatbuffers model verification failed");
    const fb::TTable core = fb::GetRoot(reader);
    // TModelCore, model.fbs:48-54
    const std::string format = core.String(0);
    CBAMD_ENSURE(format == kFormatString, "Unsupported model format: " + format);
    ModelInfo.clear();
    for (const auto& kv : core.Tables(2)) {
        ModelInfo[kv.String(0)] = kv.String(1);
    }
    ModelPartIds = core.Strings(3);
    const fb::TTable treesTable = core.Table(1);
    if (treesTable.Valid()) {
        ReadTrees(treesTable, &Trees);
    } else {
        Trees = TModelTrees();
    }
    CtrTables.clear();
    size_t partPos = pos + static_cast<size_t>(coreSize);
    for (const auto& part : ModelPartIds) {
        // model.cpp:1201-1226 knows static ctr / text / embedding parts; this evaluator reads the first kind
        CBAMD_ENSURE(part == "static_provider_v1",
                     "Model part '" + std::string(part.c_str()) + "' (text or embedding data) is not supported by the HIP evaluator");
        ReadStaticCtrProvider(p, size, &partPos, &CtrTables);
    }
    EnsureSupported();
    Trees.UpdateRuntimeData();
}

void TFullModel::LoadFromFile(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    CBAMD_ENSURE(in.good(), "can't open \"" + path + "\"");
    std::vector<char> data((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    Load(data.data(), data.size());
}

std::string TFullModel::Save() const {
    const bool withCtrPart = !CtrTables.empty();
    fb::TWriter w;
    // TModelCore
    fb::TWriter::TTableBuilder coreB;
    coreB.Ref(0);
    coreB.Ref(1);
    if (!ModelInfo.empty()) {
        coreB.Ref(2);
    }
    if (withCtrPart) {
        coreB.Ref(3);
    }
    auto core = w.WriteTable(coreB);
    w.SetRoot(core.Table);
    w.PatchRef(core.RefPos(0), w.WriteString(kFormatString));

    // TModelTrees; FBSerialize writes Bias = 0 and the real bias into MultiBias (model.cpp:396-420)
    fb::TWriter::TTableBuilder tb;
    tb.Scalar<int32_t>(TS_ApproxDimension, Trees.ApproxDimension);
    for (int slot : {TS_TreeSplits, TS_TreeSizes, TS_TreeStartOffsets, TS_CatFeatures, TS_FloatFeatures,
                     TS_OneHotFeatures, TS_CtrFeatures, TS_LeafValues, TS_LeafWeights, TS_NonSymmetricStepNodes,
                     TS_NonSymmetricNodeIdToLeafId, TS_TextFeatures, TS_EstimatedFeatures, TS_MultiBias,
                     TS_RepackedBins, TS_EmbeddingFeatures}) {
        tb.Ref(slot);
    }
    if (Trees.Scale != 1.0) {
        tb.Scalar<double>(TS_Scale, Trees.Scale);
    }
    auto tp = w.WriteTable(tb);
    w.PatchRef(core.RefPos(1), tp.Table);
    w.PatchRef(tp.RefPos(TS_TreeSplits), w.WriteVector(Trees.TreeSplits));
    w.PatchRef(tp.RefPos(TS_TreeSizes), w.WriteVector(Trees.TreeSizes));
    w.PatchRef(tp.RefPos(TS_TreeStartOffsets), w.WriteVector(Trees.TreeStartOffsets));
    WriteTableVector(w, tp.RefPos(TS_CatFeatures), Trees.CatFeatures, WriteCatFeature);
    WriteTableVector(w, tp.RefPos(TS_FloatFeatures), Trees.FloatFeatures, WriteFloatFeature);
    WriteTableVector(w, tp.RefPos(TS_OneHotFeatures), Trees.OneHotFeatures, WriteOneHotFeature);
    WriteTableVector(w, tp.RefPos(TS_CtrFeatures), Trees.CtrFeatures, WriteCtrFeature);
    for (int slot : {TS_TextFeatures, TS_EstimatedFeatures, TS_EmbeddingFeatures}) {
        w.PatchRef(tp.RefPos(slot), w.WriteRefVector(0).first);
    }
    w.PatchRef(tp.RefPos(TS_LeafValues), w.WriteVector(Trees.LeafValues));
    w.PatchRef(tp.RefPos(TS_LeafWeights), w.WriteVector(Trees.LeafWeights));
    w.PatchRef(tp.RefPos(TS_NonSymmetricStepNodes),
               w.WriteVector(Trees.NonSymmetricStepNodes.data(), Trees.NonSymmetricStepNodes.size(), 4, 2));
    w.PatchRef(tp.RefPos(TS_NonSymmetricNodeIdToLeafId), w.WriteVector(Trees.NonSymmetricNodeIdToLeafId));
    w.PatchRef(tp.RefPos(TS_MultiBias), w.WriteVector(Trees.Bias));
    {
        // struct TRepackedBin {u16 FeatureIndex; u8 XorMask; u8 SplitIdx}, model.fbs:16-20
        static_assert(sizeof(TRepackedBin) == 4, "repacked bin must be 4 bytes");
        w.PatchRef(tp.RefPos(TS_RepackedBins), w.WriteVector(Trees.RepackedBins.data(), Trees.RepackedBins.size(), 4, 2));
    }
    if (!ModelInfo.empty()) {
        auto vec = w.WriteRefVector(ModelInfo.size());
        w.PatchRef(core.RefPos(2), vec.first);
        size_t i = 0;
        for (const auto& kv : ModelInfo) {  // std::map iterates in key order, as the `key` attribute requires
            fb::TWriter::TTableBuilder kb;
            kb.Ref(0);
            kb.Ref(1);
            auto kp = w.WriteTable(kb);
            w.PatchRef(vec.second + 4 * i, kp.Table);
            w.PatchRef(kp.RefPos(0), w.WriteString(kv.first));
            w.PatchRef(kp.RefPos(1), w.WriteString(kv.second));
            ++i;
        }
    }
    if (withCtrPart) {  // ModelPartIds, model.fbs:53 and model.cpp:1140-1161
        auto vec = w.WriteRefVector(1);
        w.PatchRef(core.RefPos(3), vec.first);
        w.PatchRef(vec.second, w.WriteString("static_provider_v1"));
    }
    const auto& buf = w.Buffer();
    std::string out;
    out.append("CBM1", 4);
    AppendSize(&out, buf.size());
    out.append(reinterpret_cast<const char*>(buf.data()), buf.size());
    if (withCtrPart) {
        AppendStaticCtrProvider(&out, CtrTables);
    }
    return out;
}

void TFullModel::SaveToFile(const std::string& path) const {
    const std::string data = Save();
    std::ofstream out(path, std::ios::binary);
    CBAMD_ENSURE(out.good(), "can't open \"" + path + "\" for writing");
    out.write(data.data(), static_cast<std::streamsize>(data.size()));
    CBAMD_ENSURE(out.good(), "failed to write \"" + path + "\"");
}

}  // namespace cbamd
