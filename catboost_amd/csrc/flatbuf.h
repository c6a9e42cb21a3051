// Minimal FlatBuffers wire-format reader (bounds-checked) and writer: just what the .cbm
// model format needs (tables, scalars, strings, vectors of scalars / structs / tables / strings).
// Wire format facts used: a buffer starts with a u32 offset to the root table; a table starts
// with an i32 such that vtable = table - value; a vtable is {u16 vtable bytes, u16 table bytes,
// u16 field offset per slot (0 = absent)}; strings and vectors start with a u32 element count;
// every reference field holds a u32 distance forward from the field to its target.
#pragma once

#include "model.h"

#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

namespace cbamd::fb {

class TReader {
public:
    TReader(const uint8_t* data, size_t size) : Data(data), Size(size) {}

    template <typename T>
    T Read(size_t pos) const {
        Check(pos, sizeof(T));
        T v;
        std::memcpy(&v, Data + pos, sizeof(T));
        return v;
    }
    void Check(size_t pos, size_t len) const {
        CBAMD_ENSURE(pos <= Size && len <= Size - pos, "Flatbuffers model verification failed");
    }
    size_t Follow(size_t pos) const {  // reference field -> target position
        const uint32_t rel = Read<uint32_t>(pos);
        CBAMD_ENSURE(rel >= 4, "Flatbuffers model verification failed");
        const size_t target = pos + rel;
        Check(target, 4);
        return target;
    }
    const uint8_t* Ptr(size_t pos, size_t len) const {
        Check(pos, len);
        return Data + pos;
    }

private:
    const uint8_t* Data;
    size_t Size;
};

class TTable {
public:
    TTable() = default;
    TTable(const TReader* r, size_t pos) : R(r), Pos(pos) {
        const int32_t soff = R->Read<int32_t>(pos);
        const int64_t vt = static_cast<int64_t>(pos) - soff;
        CBAMD_ENSURE(vt >= 0, "Flatbuffers model verification failed");
        Vt = static_cast<size_t>(vt);
        VtSize = R->Read<uint16_t>(Vt);
        CBAMD_ENSURE(VtSize >= 4 && (VtSize & 1) == 0, "Flatbuffers model verification failed");
        R->Check(Vt, VtSize);
        TableSize = R->Read<uint16_t>(Vt + 2);
        R->Check(Pos, TableSize);
    }
    bool Valid() const { return R != nullptr; }

    size_t FieldPos(int slot) const {  // 0 when absent
        const size_t off = 4 + 2 * static_cast<size_t>(slot);
        if (off + 2 > VtSize) {
            return 0;
        }
        const uint16_t f = R->Read<uint16_t>(Vt + off);
        if (f == 0) {
            return 0;
        }
        CBAMD_ENSURE(f < TableSize, "Flatbuffers model verification failed");
        return Pos + f;
    }
    template <typename T>
    T Scalar(int slot, T def) const {
        const size_t p = FieldPos(slot);
        return p ? R->Read<T>(p) : def;
    }
    bool Has(int slot) const { return FieldPos(slot) != 0; }
    std::string String(int slot) const {
        const size_t p = FieldPos(slot);
        if (!p) {
            return std::string();
        }
        return StringAt(R->Follow(p));
    }
    TTable Table(int slot) const {
        const size_t p = FieldPos(slot);
        return p ? TTable(R, R->Follow(p)) : TTable();
    }
    // vector of scalars or fixed-size structs
    template <typename T>
    std::vector<T> Vector(int slot) const {
        std::vector<T> out;
        const size_t p = FieldPos(slot);
        if (!p) {
            return out;
        }
        const size_t v = R->Follow(p);
        const uint32_t n = R->Read<uint32_t>(v);
        const uint8_t* src = R->Ptr(v + 4, static_cast<size_t>(n) * sizeof(T));
        out.resize(n);
        if (n) {
            std::memcpy(out.data(), src, static_cast<size_t>(n) * sizeof(T));
        }
        return out;
    }
    size_t VectorLen(int slot) const {
        const size_t p = FieldPos(slot);
        return p ? R->Read<uint32_t>(R->Follow(p)) : 0;
    }
    std::vector<TTable> Tables(int slot) const {
        std::vector<TTable> out;
        const size_t p = FieldPos(slot);
        if (!p) {
            return out;
        }
        const size_t v = R->Follow(p);
        const uint32_t n = R->Read<uint32_t>(v);
        R->Check(v + 4, static_cast<size_t>(n) * 4);
        out.reserve(n);
        for (uint32_t i = 0; i < n; ++i) {
            out.emplace_back(R, R->Follow(v + 4 + 4 * static_cast<size_t>(i)));
        }
        return out;
    }
    std::vector<std::string> Strings(int slot) const {
        std::vector<std::string> out;
        const size_t p = FieldPos(slot);
        if (!p) {
            return out;
        }
        const size_t v = R->Follow(p);
        const uint32_t n = R->Read<uint32_t>(v);
        R->Check(v + 4, static_cast<size_t>(n) * 4);
        for (uint32_t i = 0; i < n; ++i) {
            out.push_back(StringAt(R->Follow(v + 4 + 4 * static_cast<size_t>(i))));
        }
        return out;
    }

private:
    std::string StringAt(size_t s) const {
        const uint32_t n = R->Read<uint32_t>(s);
        const uint8_t* src = R->Ptr(s + 4, n);
        return std::string(reinterpret_cast<const char*>(src), n);
    }
    const TReader* R = nullptr;
    size_t Pos = 0, Vt = 0;
    uint16_t VtSize = 0, TableSize = 0;
};

inline TTable GetRoot(const TReader& r) {
    return TTable(&r, r.Follow(0));
}

// Front-to-back writer: a table is emitted with zeroed reference fields, its children are
// emitted after it and the reference fields are patched with the forward distance.
class TWriter {
public:
    TWriter() { Buf.resize(4, 0); }  // root offset placeholder

    struct TField {
        int Slot;
        uint8_t Bytes[8];
        uint8_t Size;   // 1, 2, 4 or 8
        bool IsRef;     // u32 reference to patch later
    };

    class TTableBuilder {
    public:
        template <typename T>
        void Scalar(int slot, T v) {
            static_assert(sizeof(T) <= 8, "scalar too wide");
            TField f{};
            f.Slot = slot;
            f.Size = sizeof(T);
            f.IsRef = false;
            std::memcpy(f.Bytes, &v, sizeof(T));
            Fields.push_back(f);
        }
        void Ref(int slot) {
            TField f{};
            f.Slot = slot;
            f.Size = 4;
            f.IsRef = true;
            Fields.push_back(f);
        }
        std::vector<TField> Fields;
    };

    struct TTablePos {
        size_t Table = 0;
        std::vector<std::pair<int, size_t>> RefFieldPos;  // slot -> absolute position of the u32
        size_t RefPos(int slot) const {
            for (const auto& p : RefFieldPos) {
                if (p.first == slot) {
                    return p.second;
                }
            }
            return 0;
        }
    };

    // Emits vtable + table; returns where the table and its reference fields landed.
    TTablePos WriteTable(const TTableBuilder& b) {
        int maxSlot = -1;
        size_t maxAlign = 4;
        for (const auto& f : b.Fields) {
            maxSlot = std::max(maxSlot, f.Slot);
            maxAlign = std::max<size_t>(maxAlign, f.Size);
        }
        // field layout inside the table, largest first so that no padding is needed
        std::vector<const TField*> order;
        for (const auto& f : b.Fields) {
            order.push_back(&f);
        }
        std::stable_sort(order.begin(), order.end(), [](const TField* a, const TField* c) { return a->Size > c->Size; });
        std::vector<uint16_t> offsets(maxSlot + 1, 0);
        // soffset occupies [0, 4); the first field must start at a multiple of its size
        size_t cur = 4;
        std::vector<size_t> fieldOff(order.size());
        for (size_t i = 0; i < order.size(); ++i) {
            cur = (cur + order[i]->Size - 1) / order[i]->Size * order[i]->Size;
            fieldOff[i] = cur;
            offsets[order[i]->Slot] = static_cast<uint16_t>(cur);
            cur += order[i]->Size;
        }
        const size_t tableSize = cur;
        const size_t vtSize = 4 + 2 * offsets.size();
        // vtable, 2-aligned; then the table at a multiple of maxAlign
        Align(2);
        const size_t vtPos = Buf.size();
        PutU16(static_cast<uint16_t>(vtSize));
        PutU16(static_cast<uint16_t>(tableSize));
        for (uint16_t o : offsets) {
            PutU16(o);
        }
        Align(maxAlign);
        TTablePos pos;
        pos.Table = Buf.size();
        Buf.resize(Buf.size() + tableSize, 0);
        const int32_t soff = static_cast<int32_t>(pos.Table - vtPos);
        std::memcpy(&Buf[pos.Table], &soff, 4);
        for (size_t i = 0; i < order.size(); ++i) {
            const size_t at = pos.Table + fieldOff[i];
            if (order[i]->IsRef) {
                pos.RefFieldPos.emplace_back(order[i]->Slot, at);
            } else {
                std::memcpy(&Buf[at], order[i]->Bytes, order[i]->Size);
            }
        }
        return pos;
    }

    void PatchRef(size_t fieldPos, size_t target) {
        const uint32_t rel = static_cast<uint32_t>(target - fieldPos);
        std::memcpy(&Buf[fieldPos], &rel, 4);
    }
    void SetRoot(size_t table) { PatchRef(0, table); }

    size_t WriteString(const std::string& s) {
        Align(4);
        const size_t pos = Buf.size();
        PutU32(static_cast<uint32_t>(s.size()));
        Buf.insert(Buf.end(), s.begin(), s.end());
        Buf.push_back(0);
        return pos;
    }

    // vector of scalars / structs with element alignment `align`
    size_t WriteVector(const void* data, size_t count, size_t elemSize, size_t align) {
        // the u32 count sits right before the first element; the element must be aligned
        Align(4);
        while ((Buf.size() + 4) % std::max<size_t>(align, 4) != 0) {
            Buf.push_back(0);
        }
        const size_t pos = Buf.size();
        PutU32(static_cast<uint32_t>(count));
        const uint8_t* p = static_cast<const uint8_t*>(data);
        if (count) {
            Buf.insert(Buf.end(), p, p + count * elemSize);
        }
        return pos;
    }
    template <typename T>
    size_t WriteVector(const std::vector<T>& v) {
        return WriteVector(v.data(), v.size(), sizeof(T), alignof(T));
    }

    // vector of `count` references; returns (vector position, position of element 0)
    std::pair<size_t, size_t> WriteRefVector(size_t count) {
        Align(4);
        const size_t pos = Buf.size();
        PutU32(static_cast<uint32_t>(count));
        const size_t first = Buf.size();
        Buf.resize(Buf.size() + 4 * count, 0);
        return {pos, first};
    }

    std::vector<uint8_t>& Buffer() { return Buf; }

private:
    void Align(size_t a) {
        while (Buf.size() % a != 0) {
            Buf.push_back(0);
        }
    }
    void PutU16(uint16_t v) {
        const size_t p = Buf.size();
        Buf.resize(p + 2);
        std::memcpy(&Buf[p], &v, 2);
    }
    void PutU32(uint32_t v) {
        const size_t p = Buf.size();
        Buf.resize(p + 4);
        std::memcpy(&Buf[p], &v, 4);
    }
    std::vector<uint8_t> Buf;
};

}  // namespace cbamd::fb
