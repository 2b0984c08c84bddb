// GGUF directory reader and MoE expert-tensor binding for the host side of the
// gfx950 library: what stands between a model file and the device pointers the
// C ABI takes.
//
// Mirrors, by name and by check:
//   GGUFFile / parse / tensor / tensorRange    rust/crates/lev-gguf/src/lib.rs:11-19 (bounds), 94-112 (block
//                                              layouts), 137-176 (values), 407-486 (parse);
//                                              Sources/LeviathanCore/GGUF.swift:96-176, 203-300
//   MoEModelBinding::bind / offsets            Sources/LeviathanCore/MoEModelBinding.swift:95-214
//
// Every count and length is bounded before allocation, tensor extents are
// checked against the file length, offsets against the alignment, and no
// weight byte is read by the parser.  Header-only, no device code.
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

namespace leviathan {

struct GGUFError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// GgmlType::block_layout, lev-gguf/src/lib.rs:94-112: (elements, bytes) per block; false for unknown ids.
inline bool ggufBlockLayout(uint32_t type, uint64_t &elems, uint64_t &bytes) {
    switch (type) {
    case 0: elems = 1, bytes = 4; return true;              // F32
    case 1: case 30: elems = 1, bytes = 2; return true;     // F16, BF16
    case 2: elems = 32, bytes = 18; return true;            // Q4_0
    case 3: elems = 32, bytes = 20; return true;
    case 6: elems = 32, bytes = 22; return true;
    case 7: elems = 32, bytes = 24; return true;
    case 8: elems = 32, bytes = 34; return true;
    case 9: elems = 32, bytes = 36; return true;
    case 10: elems = 256, bytes = 84; return true;
    case 11: elems = 256, bytes = 110; return true;
    case 12: elems = 256, bytes = 144; return true;         // Q4_K
    case 13: elems = 256, bytes = 176; return true;
    case 14: elems = 256, bytes = 210; return true;         // Q6_K
    case 15: elems = 256, bytes = 292; return true;
    default: return false;
    }
}

// One metadata value.  Scalars keep their bits in `bits` (sign-extended for
// signed types, IEEE bits for floats, 0/1 for bool); strings in `str`; arrays
// of up to kKeptArrayLen elements in `items`, longer ones only as (type, length).
struct GGUFValue {
    uint32_t type = 0;
    uint64_t bits = 0;
    std::string str;
    uint32_t elemType = 0;
    uint64_t length = 0;
    bool kept = true;
    std::vector<GGUFValue> items;

    // Value::as_u64, lib.rs:155-167
    bool asU64(uint64_t &out) const {
        switch (type) {
        case 0: case 2: case 4: case 10: out = bits; return true;
        case 1: case 3: case 5: case 11:
            if ((int64_t)bits < 0) return false;
            out = bits;
            return true;
        default: return false;
        }
    }
};

struct GGUFTensorInfo {
    std::string name;
    std::vector<uint64_t> dims;
    uint32_t ggmlType = 0;
    uint64_t offset = 0;      // relative to the data section
    uint64_t byteSize = 0;
};

struct GGUFSkippedArray {
    uint32_t elemType;
    uint64_t length, elementsAt;   // absolute offset of the first element
};

class GGUFFile {
public:
    static constexpr uint64_t kMaxKV = 1ull << 16, kMaxTensors = 1ull << 20, kMaxString = 1ull << 24;
    static constexpr uint32_t kMaxDims = 8;
    static constexpr uint64_t kKeptArrayLen = 64, kDefaultAlignment = 32;

    uint32_t version = 0;
    uint64_t alignment = kDefaultAlignment, dataOffset = 0, fileLen = 0;
    std::map<std::string, GGUFValue> metadata;
    std::map<std::string, GGUFSkippedArray> skippedArrays;
    std::vector<GGUFTensorInfo> tensors;

    // parse(), lib.rs:407-486.  `data` needs to hold the directory only;
    // `fileLen` is the length of the whole file.
    static GGUFFile parse(const uint8_t *data, size_t size, uint64_t fileLen) {
        Cursor c{data, size, 0};
        GGUFFile g;
        g.fileLen = fileLen;
        uint8_t magic[4];
        c.take(magic, 4);
        if (std::memcmp(magic, "GGUF", 4) != 0) throw GGUFError("missing GGUF magic");
        g.version = c.u32();
        if (g.version < 2 || g.version > 3) throw GGUFError("unsupported version " + std::to_string(g.version));
        const uint64_t tensorCount = c.u64(), kvCount = c.u64();
        if (tensorCount > kMaxTensors) throw GGUFError("tensor count exceeds the bound");
        if (kvCount > kMaxKV) throw GGUFError("metadata count exceeds the bound");
        for (uint64_t i = 0; i < kvCount; ++i) {
            const std::string key = c.string();
            const uint32_t ty = c.u32();
            const uint64_t elementsAt = c.pos + 12;   // an array starts with element type (4) and length (8)
            GGUFValue v = c.value(ty);
            if (ty == 9 && !v.kept) g.skippedArrays[key] = {v.elemType, v.length, elementsAt};
            if (!g.metadata.emplace(key, std::move(v)).second) throw GGUFError("duplicate metadata key " + key);
        }
        std::set<std::string> names;
        g.tensors.reserve((size_t)tensorCount);
        for (uint64_t i = 0; i < tensorCount; ++i) {
            GGUFTensorInfo t;
            t.name = c.string();
            const uint32_t nd = c.u32();
            if (nd == 0 || nd > kMaxDims) throw GGUFError("tensor " + t.name + ": bad dimension count");
            for (uint32_t d = 0; d < nd; ++d) t.dims.push_back(c.u64());
            t.ggmlType = c.u32();
            t.offset = c.u64();
            if (!names.insert(t.name).second) throw GGUFError("duplicate tensor name " + t.name);
            g.tensors.push_back(std::move(t));
        }
        auto al = g.metadata.find("general.alignment");
        if (al != g.metadata.end()) {
            uint64_t a = 0;
            if (!al->second.asU64(a) || a == 0 || (a & (a - 1)) != 0)
                throw GGUFError("general.alignment is not a positive power of two");
            g.alignment = a;
        }
        g.dataOffset = (c.pos + g.alignment - 1) / g.alignment * g.alignment;
        if (g.dataOffset > fileLen) throw GGUFError("tensor data section starts past end of file");
        for (GGUFTensorInfo &t : g.tensors) {
            if (!byteSize(t, t.byteSize))
                throw GGUFError("tensor " + t.name + ": unsupported or inconsistent size");
            for (uint64_t d : t.dims)
                if (d == 0) throw GGUFError("tensor " + t.name + ": zero dimension");
            if (t.offset % g.alignment != 0) throw GGUFError("tensor " + t.name + ": offset not aligned");
            uint64_t start, end;
            if (__builtin_add_overflow(g.dataOffset, t.offset, &start) ||
                __builtin_add_overflow(start, t.byteSize, &end) || end > fileLen)
                throw GGUFError("tensor " + t.name + ": extent exceeds file length");
        }
        return g;
    }

    // GgufFile::open, lib.rs:217-221: reads the directory (grown on demand), never the weights.
    static GGUFFile open(const std::string &path) {
        FILE *f = std::fopen(path.c_str(), "rb");
        if (!f) throw GGUFError("cannot open " + path);
        std::fseek(f, 0, SEEK_END);
        const long len = std::ftell(f);
        if (len < 0) {
            std::fclose(f);
            throw GGUFError("cannot size " + path);
        }
        std::vector<uint8_t> head;
        size_t want = 1u << 20;
        for (;;) {
            if (want > (size_t)len) want = (size_t)len;
            head.resize(want);
            std::fseek(f, 0, SEEK_SET);
            if (std::fread(head.data(), 1, want, f) != want) {
                std::fclose(f);
                throw GGUFError("short read on " + path);
            }
            try {
                GGUFFile g = parse(head.data(), head.size(), (uint64_t)len);
                std::fclose(f);
                return g;
            } catch (const Truncated &) {
                if (want == (size_t)len) {
                    std::fclose(f);
                    throw GGUFError("truncated directory in " + path);
                }
                want *= 4;
            } catch (...) {
                std::fclose(f);
                throw;
            }
        }
    }

    // TensorInfo::byte_size, lib.rs:187-201
    static bool byteSize(const GGUFTensorInfo &t, uint64_t &out) {
        uint64_t elems, bytes, n = 1;
        if (!ggufBlockLayout(t.ggmlType, elems, bytes)) return false;
        for (uint64_t d : t.dims)
            if (__builtin_mul_overflow(n, d, &n)) return false;
        if (n % elems != 0) return false;
        return !__builtin_mul_overflow(n / elems, bytes, &out);
    }

    const GGUFTensorInfo *tensor(const std::string &name) const {
        for (const GGUFTensorInfo &t : tensors)
            if (t.name == name) return &t;
        return nullptr;
    }
    // tensorRange, GGUF.swift:141-174: absolute [start, end) in the file (checked at parse).
    void tensorRange(const GGUFTensorInfo &t, uint64_t &start, uint64_t &end) const {
        start = dataOffset + t.offset;
        end = start + t.byteSize;
    }
    // metadataUInt / metadataString, GGUF.swift:110-130
    uint64_t metadataUInt(const std::string &key) const {
        auto it = metadata.find(key);
        uint64_t v = 0;
        if (it == metadata.end()) throw GGUFError("missing metadata " + key);
        if (it->second.asU64(v)) return v;
        if (it->second.type == 1 || it->second.type == 3 || it->second.type == 5 || it->second.type == 11) return 0;
        throw GGUFError("missing metadata " + key + " (not an integer)");
    }
    const std::string &metadataString(const std::string &key) const {
        auto it = metadata.find(key);
        if (it == metadata.end() || it->second.type != 8) throw GGUFError("missing metadata " + key);
        return it->second.str;
    }

private:
    struct Truncated : GGUFError {
        Truncated() : GGUFError("truncated") {}
    };
    struct Cursor {
        const uint8_t *data;
        size_t size;
        uint64_t pos;
        void take(void *out, uint64_t n) {
            if (n > size - pos) throw Truncated();
            if (out) std::memcpy(out, data + pos, (size_t)n);
            pos += n;
        }
        uint32_t u32() {
            uint32_t v;
            take(&v, 4);
            return v;
        }
        uint64_t u64() {
            uint64_t v;
            take(&v, 8);
            return v;
        }
        std::string string() {
            const uint64_t n = u64();
            if (n > kMaxString) throw GGUFError("string length exceeds the bound");
            std::string s((size_t)n, '\0');
            take(n ? &s[0] : nullptr, n);
            if (!validUtf8(s)) throw GGUFError("string is not valid utf-8");
            return s;
        }
        static int scalarSize(uint32_t ty) {
            switch (ty) {
            case 0: case 1: case 7: return 1;
            case 2: case 3: return 2;
            case 4: case 5: case 6: return 4;
            case 10: case 11: case 12: return 8;
            default: return 0;
            }
        }
        GGUFValue scalar(uint32_t ty) {
            GGUFValue v;
            v.type = ty;
            if (ty == 8) {
                v.str = string();
                return v;
            }
            const int n = scalarSize(ty);
            if (!n) throw GGUFError("unsupported value type " + std::to_string(ty));
            uint64_t raw = 0;
            take(&raw, (uint64_t)n);
            if (ty == 1) raw = (uint64_t)(int64_t)(int8_t)raw;
            if (ty == 3) raw = (uint64_t)(int64_t)(int16_t)raw;
            if (ty == 5) raw = (uint64_t)(int64_t)(int32_t)raw;
            if (ty == 7) raw = raw != 0;
            v.bits = raw;
            return v;
        }
        GGUFValue value(uint32_t ty) {
            if (ty != 9) return scalar(ty);
            GGUFValue v;
            v.type = 9;
            v.elemType = u32();
            v.length = u64();
            if (v.elemType == 9) throw GGUFError("nested arrays are not supported");
            if (v.length <= kKeptArrayLen) {
                for (uint64_t i = 0; i < v.length; ++i) v.items.push_back(scalar(v.elemType));
                return v;
            }
            v.kept = false;
            if (v.elemType == 8) {
                for (uint64_t i = 0; i < v.length; ++i) {
                    const uint64_t n = u64();
                    if (n > kMaxString) throw GGUFError("string length exceeds the bound");
                    take(nullptr, n);
                }
            } else {
                const int n = scalarSize(v.elemType);
                uint64_t total;
                if (!n) throw GGUFError("unsupported array element type " + std::to_string(v.elemType));
                if (__builtin_mul_overflow(v.length, (uint64_t)n, &total)) throw GGUFError("array byte length overflows");
                take(nullptr, total);
            }
            return v;
        }
    };
    static bool validUtf8(const std::string &s) {
        size_t i = 0;
        const size_t n = s.size();
        while (i < n) {
            const unsigned char c = (unsigned char)s[i];
            size_t len;
            uint32_t cp;
            if (c < 0x80) { i += 1; continue; }
            if ((c & 0xE0) == 0xC0) len = 2, cp = c & 0x1Fu;
            else if ((c & 0xF0) == 0xE0) len = 3, cp = c & 0x0Fu;
            else if ((c & 0xF8) == 0xF0) len = 4, cp = c & 0x07u;
            else return false;
            if (i + len > n) return false;
            for (size_t k = 1; k < len; ++k) {
                const unsigned char d = (unsigned char)s[i + k];
                if ((d & 0xC0) != 0x80) return false;
                cp = (cp << 6) | (d & 0x3Fu);
            }
            if ((len == 2 && cp < 0x80) || (len == 3 && cp < 0x800) || (len == 4 && cp < 0x10000) ||
                cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF))
                return false;
            i += len;
        }
        return true;
    }
};

// Checked binding of the routed-expert tensors of every layer to the file
// (MoEModelBinding.bind, MoEModelBinding.swift:95-168; the graph capture it also
// checks is not part of this library).  Offsets are absolute file offsets,
// which are buffer offsets when the file is resident from offset 0.
struct MoEModelBinding {
    static constexpr int64_t kMaxLayers = 128, kMaxExperts = 4096, kMaxTopK = 64, kMaxDim = 8192;
    int64_t fileByteCount = 0, layerCount = 0, expertCount = 0, topK = 0, hidden = 0, inter = 0, gateUpOut = 0;
    int64_t guStride = 0, dnStride = 0;                   // bytes per expert slice
    std::vector<int64_t> guTensorStarts, dnTensorStarts;  // per layer

    static MoEModelBinding bind(const GGUFFile &file, const std::string &arch = "gemma4") {
        MoEModelBinding b;
        if (file.metadataString("general.architecture") != arch)
            throw GGUFError("general.architecture is not " + arch);
        b.fileByteCount = (int64_t)file.fileLen;
        b.layerCount = metaInt(file, arch + ".block_count", kMaxLayers);
        b.expertCount = metaInt(file, arch + ".expert_count", kMaxExperts);
        b.topK = metaInt(file, arch + ".expert_used_count", kMaxTopK);
        b.hidden = metaInt(file, arch + ".embedding_length", kMaxDim);
        b.inter = metaInt(file, arch + ".expert_feed_forward_length", kMaxDim);
        b.gateUpOut = 2 * b.inter;
        if (b.topK > b.expertCount) throw GGUFError("topK exceeds expert_count");
        int64_t guFamily = 0, dnFamily = 0;
        for (const GGUFTensorInfo &t : file.tensors) {
            guFamily += hasSuffix(t.name, ".ffn_gate_up_exps.weight");
            dnFamily += hasSuffix(t.name, ".ffn_down_exps.weight");
        }
        if (guFamily != b.layerCount || dnFamily != b.layerCount)
            throw GGUFError("expert tensor families do not match block_count");
        b.guStride = sliceStride(b.hidden, b.gateUpOut);
        b.dnStride = sliceStride(b.inter, b.hidden);
        for (int64_t layer = 0; layer < b.layerCount; ++layer) {
            for (int isGU = 1; isGU >= 0; --isGU) {
                const std::string name = "blk." + std::to_string(layer) +
                                         (isGU ? ".ffn_gate_up_exps.weight" : ".ffn_down_exps.weight");
                const GGUFTensorInfo *t = file.tensor(name);
                if (!t) throw GGUFError("tensor " + name + " missing");
                const std::vector<uint64_t> want =
                    isGU ? std::vector<uint64_t>{(uint64_t)b.hidden, (uint64_t)b.gateUpOut, (uint64_t)b.expertCount}
                         : std::vector<uint64_t>{(uint64_t)b.inter, (uint64_t)b.hidden, (uint64_t)b.expertCount};
                if (t->ggmlType != 2 || t->dims != want) throw GGUFError(name + ": not Q4_0 of the expected shape");
                uint64_t start, end;
                file.tensorRange(*t, start, end);
                const int64_t stride = isGU ? b.guStride : b.dnStride;
                int64_t bytes;
                if (__builtin_mul_overflow(stride, b.expertCount, &bytes) || (int64_t)(end - start) != bytes)
                    throw GGUFError(name + ": extent is not expert_count whole slices");
                (isGU ? b.guTensorStarts : b.dnTensorStarts).push_back((int64_t)start);
            }
        }
        return b;
    }

    // offsets(forLayer:expertIds:), MoEModelBinding.swift:174-214: slot order kept, exactly topK distinct ids.
    void offsets(int64_t layer, const std::vector<int64_t> &expertIds, std::vector<uint64_t> &gu,
                 std::vector<uint64_t> &dn) const {
        if (layer < 0 || layer >= layerCount) throw GGUFError("layer outside the model");
        if (topK <= 0 || (int64_t)expertIds.size() != topK) throw GGUFError("route does not have exactly topK ids");
        std::set<int64_t> seen;
        gu.clear();
        dn.clear();
        for (int64_t id : expertIds) {
            if (id < 0 || id >= expertCount) throw GGUFError("expert id outside the model");
            if (!seen.insert(id).second) throw GGUFError("duplicate expert id");
            gu.push_back(slice(guTensorStarts[(size_t)layer], guStride, id));
            dn.push_back(slice(dnTensorStarts[(size_t)layer], dnStride, id));
        }
    }

    // sliceStride, MoEModelBinding.swift:283-291: whole Q4_0 rows of one expert
    static int64_t sliceStride(int64_t inDim, int64_t outDim) {
        int64_t rowBytes, stride;
        if (inDim <= 0 || outDim <= 0 || inDim % 32 != 0 || __builtin_mul_overflow(inDim / 32, (int64_t)18, &rowBytes) ||
            __builtin_mul_overflow(rowBytes, outDim, &stride))
            throw GGUFError("invalid Q4_0 slice dims");
        return stride;
    }

private:
    uint64_t slice(int64_t start, int64_t stride, int64_t id) const {
        int64_t off, abs, end, famBytes, famEnd;
        if (start < 0 || stride <= 0 || stride % 18 != 0 || __builtin_mul_overflow(id, stride, &off) ||
            __builtin_add_overflow(start, off, &abs) || __builtin_add_overflow(abs, stride, &end) ||
            __builtin_mul_overflow(stride, expertCount, &famBytes) || __builtin_add_overflow(start, famBytes, &famEnd) ||
            end > famEnd || end > fileByteCount)
            throw GGUFError("expert slice outside its tensor or the file");
        return (uint64_t)abs;
    }
    static bool hasSuffix(const std::string &s, const std::string &suf) {
        return s.size() >= suf.size() && s.compare(s.size() - suf.size(), suf.size(), suf) == 0;
    }
    static int64_t metaInt(const GGUFFile &f, const std::string &key, int64_t cap) {
        const uint64_t raw = f.metadataUInt(key);
        if (raw == 0 || raw > (uint64_t)cap) throw GGUFError(key + " outside 1..." + std::to_string(cap));
        return (int64_t)raw;
    }
};

}  // namespace leviathan
