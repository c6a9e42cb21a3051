// JSON model import: the "json" model format of CatBoost read into the same tables as a .cbm file.
// Follows ConvertJsonToCatboostModel (catboost/libs/model/model_export/json_model_helpers.cpp:583-608)
// with its helpers GetObliviousModelTrees (:366-391), GetNonSymmetricModelTrees (:393-431),
// GetFeaturesInfo (:267-291), FloatFeatureFromJson (:180-189) and CatFeatureFromJson (:199-205).
// CTR features and their tables: CtrFeatureFromJson (:119-136), FeatureCombinationFromJson (:54-78) and
// CtrDataFromJson (:531-580); the json format does not carry TModelCtrBase::TargetBorderClassifierIdx (0 then).
#include "model.h"

#include <cerrno>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iterator>
#include <limits>
#include <memory>
#include <utility>

namespace cbamd {

namespace {

// ---- a small JSON reader: values keep the text of numbers, objects keep the order of their keys

struct TJson {
    enum EType { Null, Bool, Number, String, Array, Object };
    EType Type = Null;
    bool Flag = false;
    double Num = 0.0;
    std::string Text;  // string value, or the number as written
    std::vector<TJson> Items;
    std::vector<std::pair<std::string, TJson>> Fields;

    bool Has(const char* key) const { return Find(key) != nullptr; }
    const TJson* Find(const char* key) const {
        if (Type != Object) {
            return nullptr;
        }
        for (const auto& f : Fields) {
            if (f.first == key) {
                return &f.second;
            }
        }
        return nullptr;
    }
    const TJson& At(const char* key) const {
        const TJson* v = Find(key);
        CBAMD_ENSURE(v != nullptr, "JSON model: key \"" + key + "\" is missing");
        return *v;
    }
    const std::vector<TJson>& Array_(const char* what) const {
        CBAMD_ENSURE(Type == Array, "JSON model: " + what + " must be an array");
        return Items;
    }
    double Double(const char* what) const {
        CBAMD_ENSURE(Type == Number, "JSON model: " + what + " must be a number");
        return Num;
    }
    long long Integer(const char* what) const {
        CBAMD_ENSURE(Type == Number, "JSON model: " + what + " must be an integer");
        errno = 0;
        char* end = nullptr;
        const long long v = std::strtoll(Text.c_str(), &end, 10);
        if (errno == 0 && end != nullptr && *end == '\0') {
            return v;
        }
        CBAMD_ENSURE(std::isfinite(Num) && std::fabs(Num) < 9.0e18, "JSON model: " + what + " is out of range");
        return static_cast<long long>(Num);
    }
    int Int32(const char* what) const {
        const long long v = Integer(what);
        CBAMD_ENSURE(v >= std::numeric_limits<int>::min() && v <= std::numeric_limits<int>::max(),
                     "JSON model: " + what + " is out of range");
        return static_cast<int>(v);
    }
    const std::string& Str(const char* what) const {
        CBAMD_ENSURE(Type == String, "JSON model: " + what + " must be a string");
        return Text;
    }
    bool Boolean(const char* what) const {
        CBAMD_ENSURE(Type == Bool, "JSON model: " + what + " must be a boolean");
        return Flag;
    }
};

class TJsonParser {
public:
    TJsonParser(const char* data, size_t size) : P(data), End(data + size) {}

    TJson ParseDocument() {
        TJson v = ParseValue(0);
        SkipSpace();
        CBAMD_ENSURE(P == End, "JSON model: unexpected text after the document");
        return v;
    }

private:
    static constexpr int kMaxDepth = 4096;

    void SkipSpace() {
        while (P < End && (*P == ' ' || *P == '\t' || *P == '\n' || *P == '\r')) {
            ++P;
        }
    }
    [[noreturn]] void Fail(const char* what) const { throw TModelError(std::string("JSON model: ") + what); }

    TJson ParseValue(int depth) {
        if (depth > kMaxDepth) {
            Fail("nesting is too deep");
        }
        SkipSpace();
        if (P == End) {
            Fail("unexpected end of the document");
        }
        TJson v;
        const char c = *P;
        if (c == '{') {
            ++P;
            v.Type = TJson::Object;
            SkipSpace();
            if (P < End && *P == '}') {
                ++P;
                return v;
            }
            for (;;) {
                SkipSpace();
                if (P == End || *P != '"') {
                    Fail("object key expected");
                }
                std::string key = ParseString();
                SkipSpace();
                if (P == End || *P != ':') {
                    Fail("':' expected");
                }
                ++P;
                v.Fields.emplace_back(std::move(key), ParseValue(depth + 1));
                SkipSpace();
                if (P < End && *P == ',') {
                    ++P;
                    continue;
                }
                if (P < End && *P == '}') {
                    ++P;
                    return v;
                }
                Fail("',' or '}' expected");
            }
        }
        if (c == '[') {
            ++P;
            v.Type = TJson::Array;
            SkipSpace();
            if (P < End && *P == ']') {
                ++P;
                return v;
            }
            for (;;) {
                v.Items.push_back(ParseValue(depth + 1));
                SkipSpace();
                if (P < End && *P == ',') {
                    ++P;
                    continue;
                }
                if (P < End && *P == ']') {
                    ++P;
                    return v;
                }
                Fail("',' or ']' expected");
            }
        }
        if (c == '"') {
            v.Type = TJson::String;
            v.Text = ParseString();
            return v;
        }
        if (Literal("true")) {
            v.Type = TJson::Bool;
            v.Flag = true;
            return v;
        }
        if (Literal("false")) {
            v.Type = TJson::Bool;
            return v;
        }
        if (Literal("null")) {
            return v;
        }
        // numbers; the writer also emits nan / inf / -inf for such leaf values
        const char* begin = P;
        while (P < End && (std::strchr("+-.eE", *P) != nullptr || (*P >= '0' && *P <= '9') ||
                           (*P >= 'a' && *P <= 'z') || (*P >= 'A' && *P <= 'Z'))) {
            ++P;
        }
        if (P == begin) {
            Fail("unexpected character");
        }
        v.Type = TJson::Number;
        v.Text.assign(begin, P);
        char* end = nullptr;
        v.Num = std::strtod(v.Text.c_str(), &end);
        if (end == nullptr || *end != '\0') {
            Fail("malformed number");
        }
        return v;
    }

    bool Literal(const char* word) {
        const size_t n = std::strlen(word);
        if (static_cast<size_t>(End - P) >= n && std::memcmp(P, word, n) == 0) {
            P += n;
            return true;
        }
        return false;
    }

    static void AppendUtf8(std::string* out, uint32_t cp) {
        if (cp < 0x80) {
            out->push_back(static_cast<char>(cp));
        } else if (cp < 0x800) {
            out->push_back(static_cast<char>(0xC0 | (cp >> 6)));
            out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
        } else if (cp < 0x10000) {
            out->push_back(static_cast<char>(0xE0 | (cp >> 12)));
            out->push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
            out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
        } else {
            out->push_back(static_cast<char>(0xF0 | (cp >> 18)));
            out->push_back(static_cast<char>(0x80 | ((cp >> 12) & 0x3F)));
            out->push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
            out->push_back(static_cast<char>(0x80 | (cp & 0x3F)));
        }
    }

    uint32_t Hex4() {
        if (End - P < 4) {
            Fail("truncated \\u escape");
        }
        uint32_t v = 0;
        for (int i = 0; i < 4; ++i) {
            const char c = *P++;
            v <<= 4;
            if (c >= '0' && c <= '9') {
                v |= static_cast<uint32_t>(c - '0');
            } else if (c >= 'a' && c <= 'f') {
                v |= static_cast<uint32_t>(c - 'a' + 10);
            } else if (c >= 'A' && c <= 'F') {
                v |= static_cast<uint32_t>(c - 'A' + 10);
            } else {
                Fail("malformed \\u escape");
            }
        }
        return v;
    }

    std::string ParseString() {
        ++P;  // opening quote
        std::string out;
        for (;;) {
            if (P == End) {
                Fail("unterminated string");
            }
            const char c = *P++;
            if (c == '"') {
                return out;
            }
            if (c != '\\') {
                out.push_back(c);
                continue;
            }
            if (P == End) {
                Fail("unterminated string");
            }
            const char e = *P++;
            switch (e) {
                case '"': out.push_back('"'); break;
                case '\\': out.push_back('\\'); break;
                case '/': out.push_back('/'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'n': out.push_back('\n'); break;
                case 'r': out.push_back('\r'); break;
                case 't': out.push_back('\t'); break;
                case 'u': {
                    uint32_t cp = Hex4();
                    if (cp >= 0xD800 && cp < 0xDC00 && End - P >= 6 && P[0] == '\\' && P[1] == 'u') {
                        P += 2;
                        const uint32_t low = Hex4();
                        if (low >= 0xDC00 && low < 0xE000) {
                            cp = 0x10000 + ((cp - 0xD800) << 10) + (low - 0xDC00);
                        } else {
                            Fail("malformed surrogate pair");
                        }
                    }
                    AppendUtf8(&out, cp);
                    break;
                }
                default:
                    Fail("unknown escape in a string");
            }
        }
    }

    const char* P;
    const char* End;
};

// TJsonValue::GetStringRobust of a model_info value: strings as they are, anything else as JSON text
void WriteCompact(const TJson& v, std::string* out) {
    switch (v.Type) {
        case TJson::Null:
            *out += "null";
            break;
        case TJson::Bool:
            *out += v.Flag ? "true" : "false";
            break;
        case TJson::Number:
            *out += v.Text;
            break;
        case TJson::String: {
            out->push_back('"');
            for (const char c : v.Text) {
                if (c == '"' || c == '\\') {
                    out->push_back('\\');
                    out->push_back(c);
                } else if (c == '\n') {
                    *out += "\\n";
                } else if (c == '\t') {
                    *out += "\\t";
                } else if (c == '\r') {
                    *out += "\\r";
                } else {
                    out->push_back(c);
                }
            }
            out->push_back('"');
            break;
        }
        case TJson::Array:
            out->push_back('[');
            for (size_t i = 0; i < v.Items.size(); ++i) {
                if (i) {
                    out->push_back(',');
                }
                WriteCompact(v.Items[i], out);
            }
            out->push_back(']');
            break;
        case TJson::Object:
            out->push_back('{');
            for (size_t i = 0; i < v.Fields.size(); ++i) {
                if (i) {
                    out->push_back(',');
                }
                TJson key;
                key.Type = TJson::String;
                key.Text = v.Fields[i].first;
                WriteCompact(key, out);
                out->push_back(':');
                WriteCompact(v.Fields[i].second, out);
            }
            out->push_back('}');
            break;
    }
}

ENanValueTreatment NanTreatmentFromString(const std::string& s) {
    if (s == "AsIs") {
        return ENanValueTreatment::AsIs;
    }
    if (s == "AsFalse") {
        return ENanValueTreatment::AsFalse;
    }
    CBAMD_ENSURE(s == "AsTrue", "JSON model: unknown nan_value_treatment \"" + s + "\"");
    return ENanValueTreatment::AsTrue;
}

// json_model_helpers.cpp:366-391
void ReadObliviousTrees(const TJson& treesJson, TModelTrees* trees) {
    bool dimensionKnown = false;
    for (const TJson& tree : treesJson.Array_("oblivious_trees")) {
        const auto& leaves = tree.At("leaf_values").Array_("leaf_values");
        for (const TJson& leaf : leaves) {
            trees->LeafValues.push_back(leaf.Double("a leaf value"));
        }
        const auto& splits = tree.At("splits").Array_("splits");
        CBAMD_ENSURE(splits.size() < 31, "JSON model: unsupported tree depth");
        const size_t leafCount = size_t(1) << splits.size();
        CBAMD_ENSURE(!leaves.empty() && leaves.size() % leafCount == 0,
                     "JSON model: the number of leaf values does not match the tree's depth");
        const int dimension = static_cast<int>(leaves.size() / leafCount);
        CBAMD_ENSURE(!dimensionKnown || dimension == trees->ApproxDimension,
                     "JSON model: trees disagree about the approx dimension");
        trees->ApproxDimension = dimension;
        dimensionKnown = true;
        std::vector<int> binSplits;
        for (const TJson& split : splits) {
            binSplits.push_back(split.At("split_index").Int32("split_index"));
        }
        trees->AddBinTree(binSplits);
        if (const TJson* weights = tree.Find("leaf_weights")) {
            for (const TJson& w : weights->Array_("leaf_weights")) {
                trees->LeafWeights.push_back(w.Double("a leaf weight"));
            }
        }
    }
}

// json_model_helpers.cpp:393-431: nodes in pre-order; a leaf is a node without children whose value
// index goes into NonSymmetricNodeIdToLeafId
struct TNonSymmetricReader {
    TModelTrees* Trees;
    bool DimensionKnown = false;

    int ReadNode(const TJson& node, int depth) {
        CBAMD_ENSURE(depth < 4000, "JSON model: tree is too deep");
        const int nodeIdx = static_cast<int>(Trees->NonSymmetricStepNodes.size());
        Trees->NonSymmetricStepNodes.push_back({0, 0});
        if (const TJson* value = node.Find("value")) {
            CBAMD_ENSURE(Trees->LeafValues.size() < std::numeric_limits<uint32_t>::max(), "JSON model: too many leaf values");
            Trees->NonSymmetricNodeIdToLeafId.push_back(static_cast<uint32_t>(Trees->LeafValues.size()));
            Trees->TreeSplits.push_back(0);
            int dimension = 1;
            if (value->Type == TJson::Array) {
                dimension = static_cast<int>(value->Items.size());
                for (const TJson& v : value->Items) {
                    Trees->LeafValues.push_back(v.Double("a leaf value"));
                }
            } else {
                Trees->LeafValues.push_back(value->Double("a leaf value"));
            }
            CBAMD_ENSURE(dimension >= 1 && (!DimensionKnown || dimension == Trees->ApproxDimension),
                         "JSON model: leaves disagree about the approx dimension");
            Trees->ApproxDimension = dimension;
            DimensionKnown = true;
            if (const TJson* weight = node.Find("weight")) {
                Trees->LeafWeights.push_back(weight->Double("a leaf weight"));
            }
        } else {
            Trees->NonSymmetricNodeIdToLeafId.push_back(std::numeric_limits<uint32_t>::max());
            Trees->TreeSplits.push_back(node.At("split").At("split_index").Int32("split_index"));
            const int left = ReadNode(node.At("left"), depth + 1) - nodeIdx;
            const int right = ReadNode(node.At("right"), depth + 1) - nodeIdx;
            CBAMD_ENSURE(left > 0 && left <= 0xffff && right > 0 && right <= 0xffff, "JSON model: tree is too large");
            Trees->NonSymmetricStepNodes[nodeIdx].LeftSubtreeDiff = static_cast<uint16_t>(left);
            Trees->NonSymmetricStepNodes[nodeIdx].RightSubtreeDiff = static_cast<uint16_t>(right);
        }
        return nodeIdx;
    }
};

void ReadNonSymmetricTrees(const TJson& treesJson, TModelTrees* trees) {
    TNonSymmetricReader reader{trees};
    for (const TJson& tree : treesJson.Array_("trees")) {
        const size_t before = trees->NonSymmetricStepNodes.size();
        reader.ReadNode(tree, 0);
        trees->TreeStartOffsets.push_back(static_cast<int>(before));
        trees->TreeSizes.push_back(static_cast<int>(trees->NonSymmetricStepNodes.size() - before));
    }
}

// json_model_helpers.cpp:267-291
ECtrType CtrTypeFromString(const std::string& s) {  // ECtrType, catboost/private/libs/ctr_description/ctr_type.h
    static const char* const names[] = {"Borders", "Buckets", "BinarizedTargetMeanValue", "FloatTargetMeanValue",
                                        "Counter", "FeatureFreq"};
    for (int i = 0; i < 6; ++i) {
        if (s == names[i]) {
            return static_cast<ECtrType>(i);
        }
    }
    CBAMD_ENSURE(false, "JSON model: unknown CTR type \"" + s + "\"");
    return ECtrType::Borders;
}

// FeatureCombinationFromJson, json_model_helpers.cpp:54-78
TFeatureCombination ReadProjection(const TJson& elements) {
    TFeatureCombination projection;
    for (const TJson& v : elements.Array_("the elements of a CTR")) {
        const std::string& kind = v.At("combination_element").Str("combination_element");
        if (kind == "cat_feature_value") {
            projection.CatFeatures.push_back(v.At("cat_feature_index").Int32("cat_feature_index"));
        } else if (kind == "float_feature") {
            TFloatSplit split;
            split.FloatFeature = v.At("float_feature_index").Int32("float_feature_index");
            split.Split = static_cast<float>(v.At("border").Double("border"));
            projection.BinFeatures.push_back(split);
        } else {
            TOneHotSplit split;
            split.CatFeatureIdx = v.At("cat_feature_index").Int32("cat_feature_index");
            split.Value = v.At("value").Int32("value");
            projection.OneHotFeatures.push_back(split);
        }
    }
    return projection;
}

// CtrFeatureFromJson / ModelCtrFromJson, json_model_helpers.cpp:119-136
TCtrFeature ReadCtrFeature(const TJson& v) {
    TCtrFeature feature;
    feature.Ctr.Base.Projection = ReadProjection(v.At("elements"));
    feature.Ctr.Base.CtrType = CtrTypeFromString(v.At("ctr_type").Str("ctr_type"));
    feature.Ctr.TargetBorderIdx = v.At("target_border_idx").Int32("target_border_idx");
    feature.Ctr.PriorNum = static_cast<float>(v.At("prior_numerator").Double("prior_numerator"));
    feature.Ctr.PriorDenom = static_cast<float>(v.At("prior_denomerator").Double("prior_denomerator"));
    feature.Ctr.Shift = static_cast<float>(v.At("shift").Double("shift"));
    feature.Ctr.Scale = static_cast<float>(v.At("scale").Double("scale"));
    for (const TJson& b : v.At("borders").Array_("the borders of a CTR")) {
        feature.Borders.push_back(static_cast<float>(b.Double("a border")));
    }
    return feature;
}

void ReadFeaturesInfo(const TJson& info, TModelTrees* trees) {
    if (const TJson* floats = info.Find("float_features")) {
        for (const TJson& v : floats->Array_("float_features")) {
            TFloatFeature f;
            f.HasNans = v.At("has_nans").Boolean("has_nans");
            f.Index = v.At("feature_index").Int32("feature_index");
            f.FlatIndex = v.At("flat_feature_index").Int32("flat_feature_index");
            if (const TJson* borders = v.Find("borders")) {
                if (borders->Type != TJson::Null) {
                    for (const TJson& b : borders->Array_("borders")) {
                        f.Borders.push_back(static_cast<float>(b.Double("a border")));
                    }
                }
            }
            if (const TJson* id = v.Find("feature_id")) {
                f.FeatureId = id->Type == TJson::String ? id->Text : std::string();
            }
            f.NanValueTreatment = NanTreatmentFromString(v.At("nan_value_treatment").Str("nan_value_treatment"));
            trees->FloatFeatures.push_back(std::move(f));
        }
    }
    if (const TJson* cats = info.Find("categorical_features")) {
        for (const TJson& v : cats->Array_("categorical_features")) {
            TCatFeature c;
            c.Index = v.At("feature_index").Int32("feature_index");
            c.FlatIndex = v.At("flat_feature_index").Int32("flat_feature_index");
            if (const TJson* id = v.Find("feature_id")) {
                c.FeatureId = id->Type == TJson::String ? id->Text : std::string();
            }
            trees->CatFeatures.push_back(c);
            if (const TJson* values = v.Find("values")) {
                TOneHotFeature oh;
                oh.CatFeatureIndex = c.Index;
                for (const TJson& x : values->Array_("values")) {
                    oh.Values.push_back(x.Int32("a one-hot value"));
                }
                if (const TJson* names = v.Find("string_values")) {
                    if (names->Type == TJson::Array) {
                        for (const TJson& s : names->Items) {
                            oh.StringValues.push_back(s.Str("a one-hot string value"));
                        }
                    }
                }
                trees->OneHotFeatures.push_back(std::move(oh));
            }
        }
    }
    if (const TJson* ctrs = info.Find("ctrs")) {
        if (ctrs->Type == TJson::Array) {
            for (const TJson& v : ctrs->Items) {
                trees->CtrFeatures.push_back(ReadCtrFeature(v));
            }
        }
    }
}

// CtrDataFromJson, json_model_helpers.cpp:531-580: a map from the text of a {"type", "identifier"} object
// to {"hash_map": [hash as a decimal string, the row's values, ...], "hash_stride", "counter_denominator"}.
// Rows are numbered in the order of their hashes (TDenseIndexHashBuilder::AddIndex,
// catboost/libs/helpers/dense_hash_view.h:74-121: 2^k buckets at a load factor of at most one half,
// linear probing, a hash seen again keeps its row).
void ReadCtrData(const TJson& data, std::vector<TCtrValueTable>* tables) {
    if (data.Type != TJson::Object) {
        return;
    }
    for (const auto& entry : data.Fields) {
        TJsonParser keyParser(entry.first.data(), entry.first.size());
        const TJson key = keyParser.ParseDocument();
        TCtrValueTable table;
        table.ModelCtrBase.CtrType = CtrTypeFromString(key.At("type").Str("type"));
        table.ModelCtrBase.Projection = ReadProjection(key.At("identifier"));
        const ECtrType type = table.ModelCtrBase.CtrType;
        const bool mean = type == ECtrType::BinarizedTargetMeanValue || type == ECtrType::FloatTargetMeanValue;
        const bool counter = type == ECtrType::Counter || type == ECtrType::FeatureFreq;
        const long long stride = entry.second.At("hash_stride").Integer("hash_stride");
        const auto& items = entry.second.At("hash_map").Array_("hash_map");
        CBAMD_ENSURE(stride >= 2 && stride <= 65536 && items.size() % static_cast<size_t>(stride) == 0,
                     "JSON model: hash_map does not hold whole rows of hash_stride values");
        CBAMD_ENSURE(!mean || stride == 3, "JSON model: a mean CTR table has rows of a sum and a count");
        CBAMD_ENSURE(!counter || stride == 2, "JSON model: a counter CTR table has rows of one value");
        const size_t rows = items.size() / static_cast<size_t>(stride);
        const size_t values = static_cast<size_t>(stride) - 1;
        size_t buckets = 2;
        while (buckets < 2 * rows) {
            buckets *= 2;
        }
        CBAMD_ENSURE(buckets < (size_t(1) << 31), "JSON model: CTR table is too large");
        std::vector<uint64_t> hashes(buckets, ~uint64_t(0));
        std::vector<uint32_t> rowOf(buckets, 0);
        std::vector<uint32_t> blob(rows * (mean ? 2 : values), 0);
        if (counter) {
            table.CounterDenominator = entry.second.At("counter_denominator").Int32("counter_denominator");
        } else if (!mean) {
            table.TargetClassesCount = static_cast<int>(values);
        }
        uint32_t rowCount = 0;
        for (size_t r = 0; r < rows; ++r) {
            const TJson* item = &items[r * static_cast<size_t>(stride)];
            const std::string& text = item[0].Str("a hash of hash_map");
            errno = 0;
            char* end = nullptr;
            const unsigned long long hash = std::strtoull(text.c_str(), &end, 10);
            CBAMD_ENSURE(!text.empty() && text[0] != '-' && errno == 0 && end != nullptr && *end == '\0',
                         "JSON model: a hash of hash_map is not a 64-bit number");
            CBAMD_ENSURE(hash != ~0ull, "JSON model: a hash of hash_map has the value of an empty bucket");
            size_t z = hash & (buckets - 1);
            while (hashes[z] != ~uint64_t(0) && hashes[z] != hash) {
                z = (z + 1) & (buckets - 1);
            }
            if (hashes[z] == ~uint64_t(0)) {
                hashes[z] = hash;
                rowOf[z] = rowCount++;
            }
            const uint32_t row = rowOf[z];
            if (mean) {
                // the reference reads the sum with GetInteger (json_model_helpers.cpp:562): a sum that is
                // not a whole number becomes 0 there, and so it does here
                const double sum = item[1].Double("a sum of hash_map");
                const float kept = (std::isfinite(sum) && sum == std::floor(sum) && std::fabs(sum) < 9.0e18)
                                       ? static_cast<float>(static_cast<long long>(sum)) : 0.f;
                std::memcpy(&blob[2 * row], &kept, 4);
                blob[2 * row + 1] = static_cast<uint32_t>(item[2].Int32("a count of hash_map"));
            } else {
                for (size_t k = 0; k < values; ++k) {
                    blob[row * values + k] = static_cast<uint32_t>(item[1 + k].Int32("a value of hash_map"));
                }
            }
        }
        table.IndexHashRaw.resize(buckets * 12);
        for (size_t z = 0; z < buckets; ++z) {
            std::memcpy(&table.IndexHashRaw[12 * z], &hashes[z], 8);
            std::memcpy(&table.IndexHashRaw[12 * z + 8], &rowOf[z], 4);
        }
        blob.resize(static_cast<size_t>(rowCount) * (mean ? 2 : values));
        table.CTRBlob.resize(blob.size() * 4);
        if (!blob.empty()) {
            std::memcpy(table.CTRBlob.data(), blob.data(), table.CTRBlob.size());
        }
        tables->push_back(std::move(table));
    }
}

}  // namespace

void TFullModel::LoadFromJson(const void* data, size_t size) {
    TJsonParser parser(static_cast<const char*>(data), size);
    const TJson root = parser.ParseDocument();
    CBAMD_ENSURE(root.Type == TJson::Object, "JSON model: the document must be an object");
    *this = TFullModel();
    if (const TJson* info = root.Find("model_info")) {
        if (info->Type == TJson::Object) {
            for (const auto& kv : info->Fields) {
                std::string text;
                if (kv.second.Type == TJson::String) {
                    text = kv.second.Text;
                } else {
                    WriteCompact(kv.second, &text);
                }
                ModelInfo[kv.first] = text;
            }
        }
    }
    if (const TJson* oblivious = root.Find("oblivious_trees")) {
        ReadObliviousTrees(*oblivious, &Trees);
    } else {
        ReadNonSymmetricTrees(root.At("trees"), &Trees);
    }
    ReadFeaturesInfo(root.At("features_info"), &Trees);
    if (const TJson* ctrData = root.Find("ctr_data")) {
        ReadCtrData(*ctrData, &CtrTables);
        if (!CtrTables.empty()) {
            ModelPartIds.push_back("static_provider_v1");
        }
    }
    if (const TJson* sb = root.Find("scale_and_bias")) {
        const auto& items = sb->Array_("scale_and_bias");
        CBAMD_ENSURE(items.size() == 2, "JSON model: scale_and_bias must hold a scale and a bias");
        const double scale = items[0].Double("the scale");
        std::vector<double> bias;
        if (items[1].Type == TJson::Array) {
            for (const TJson& b : items[1].Items) {
                bias.push_back(b.Double("a bias value"));
            }
        } else {
            bias.push_back(items[1].Double("the bias"));  // files written before multi-dimensional biases
        }
        if (bias.size() == 1 && Trees.ApproxDimension > 1 && bias[0] == 0.0) {
            bias.assign(Trees.ApproxDimension, 0.0);
        }
        Trees.SetScaleAndBias(scale, bias);
    }
    EnsureSupported();
    Trees.UpdateRuntimeData();
}

void TFullModel::LoadFromJsonFile(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    CBAMD_ENSURE(in.good(), "can't open \"" + path + "\"");
    std::vector<char> data((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    LoadFromJson(data.data(), data.size());
}

}  // namespace cbamd
