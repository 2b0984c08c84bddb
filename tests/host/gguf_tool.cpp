// Prints the canonical dump of a GGUF directory as read by the C++ host
// reader (the same text form oracle/gguf.py prints), or the MoE expert binding.
//   gguf_tool dump <file>      exit 0 + dump, or exit 2 + "error: ..." when the reader rejects the file
//   gguf_tool bind <file>      exit 0 + binding lines, or exit 2
// No device is touched.
#include <cstdio>
#include <string>

#include "leviathan_gguf.hpp"

using namespace leviathan;

static std::string hex(const std::string &s) {
    static const char *d = "0123456789abcdef";
    std::string o;
    for (unsigned char c : s) {
        o.push_back(d[c >> 4]);
        o.push_back(d[c & 15]);
    }
    return o.empty() ? "-" : o;
}

static std::string repr(const GGUFValue &v) {
    if (v.type == 8) return hex(v.str);
    if (v.type == 9) {
        std::string o = "[" + std::to_string(v.elemType) + " " + std::to_string(v.length);
        if (!v.kept) return o + " skipped]";
        for (const GGUFValue &x : v.items) o += " " + repr(x);
        return o + "]";
    }
    const bool is_signed = v.type == 1 || v.type == 3 || v.type == 5 || v.type == 11;
    return is_signed ? std::to_string((long long)v.bits) : std::to_string((unsigned long long)v.bits);
}

int main(int argc, char **argv) {
    if (argc != 3) {
        std::fprintf(stderr, "usage: gguf_tool dump|bind <file>\n");
        return 1;
    }
    const std::string mode = argv[1];
    try {
        GGUFFile g = GGUFFile::open(argv[2]);
        if (mode == "dump") {
            std::printf("version %u\nalignment %llu\ndata_offset %llu\nfile_len %llu\n", g.version,
                        (unsigned long long)g.alignment, (unsigned long long)g.dataOffset,
                        (unsigned long long)g.fileLen);
            for (const auto &kv : g.metadata)   // std::map: byte-wise key order, as sorted() on bytes
                std::printf("kv %s %u %s\n", hex(kv.first).c_str(), kv.second.type, repr(kv.second).c_str());
            for (const auto &kv : g.skippedArrays)
                std::printf("skipped %s %u %llu %llu\n", hex(kv.first).c_str(), kv.second.elemType,
                            (unsigned long long)kv.second.length, (unsigned long long)kv.second.elementsAt);
            for (const GGUFTensorInfo &t : g.tensors) {
                std::string dims;
                for (size_t i = 0; i < t.dims.size(); ++i) dims += (i ? "," : "") + std::to_string(t.dims[i]);
                std::printf("tensor %s %u %s %llu %llu\n", hex(t.name).c_str(), t.ggmlType, dims.c_str(),
                            (unsigned long long)t.offset, (unsigned long long)t.byteSize);
            }
            return 0;
        }
        if (mode == "bind") {
            MoEModelBinding b = MoEModelBinding::bind(g);
            std::printf("layers %lld experts %lld topk %lld hidden %lld inter %lld gu_stride %lld dn_stride %lld\n",
                        (long long)b.layerCount, (long long)b.expertCount, (long long)b.topK, (long long)b.hidden,
                        (long long)b.inter, (long long)b.guStride, (long long)b.dnStride);
            for (int64_t l = 0; l < b.layerCount; ++l)
                std::printf("layer %lld gu %lld dn %lld\n", (long long)l, (long long)b.guTensorStarts[(size_t)l],
                            (long long)b.dnTensorStarts[(size_t)l]);
            // the route 0, 1, ... topK-1 reversed, to show slot order is kept
            std::vector<int64_t> ids;
            for (int64_t k = b.topK; k-- > 0;) ids.push_back(k);
            std::vector<uint64_t> gu, dn;
            b.offsets(b.layerCount - 1, ids, gu, dn);
            for (size_t k = 0; k < ids.size(); ++k)
                std::printf("slot %zu id %lld gu %llu dn %llu\n", k, (long long)ids[k], (unsigned long long)gu[k],
                            (unsigned long long)dn[k]);
            return 0;
        }
        std::fprintf(stderr, "unknown mode %s\n", mode.c_str());
        return 1;
    } catch (const GGUFError &e) {
        std::printf("error: %s\n", e.what());
        return 2;
    }
}
