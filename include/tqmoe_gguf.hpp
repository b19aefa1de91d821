// GGUF expert-bank ingestion for the tqmoe library, header-only and host-only.
//
// A mixture-of-experts checkpoint stores every expert of a projection in ONE 3-D tensor [cols, rows, n_experts]
// (ffn_gate_exps / ffn_up_exps / ffn_down_exps). Its bytes are expert after expert, rows in order, so the whole tensor
// is exactly the stacked block stream [n_experts * rows][cols] that tqmoe_bank_load reads, and one expert is a
// contiguous span of it. This header gives the reader and the slicer the names and the fail-closed behaviour of the
// reference's (src/core/gguf.hpp:71-91, gguf.cpp:116-200; tests/moe_experts.cpp is the model for the tests):
//
//   tqmoe_hip::gguf_open(path)            header, metadata alignment, tensor table (name -> type, ne, offset, bytes)
//   tqmoe_hip::gguf_block_layout(type..)  weights and bytes per block of a GGUF type
//   tqmoe_hip::gguf_expert_count(t)       ne[2] of a 3-D tensor, else 0
//   tqmoe_hip::gguf_expert_slice(t, i, n) descriptor of expert i: ne reduced to [cols, rows], offset / bytes of its span;
//                                         throws std::runtime_error on any inconsistency (a wrong slice would silently
//                                         read a neighbouring expert's weights)
//   tqmoe_hip::gguf_expert_bank(f, name)  what tqmoe_bank_load needs for the whole tensor: type, experts, rows, cols,
//                                         file offset and byte count of the block stream
//
// The caller copies the span to the device (the engine's Upload) and calls tqmoe_bank_load; nothing here touches a GPU.
#pragma once
#include <cstdint>
#include <cstdio>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace tqmoe_hip {

struct GgufTensor {
    uint32_t type = 0;
    std::vector<uint64_t> ne;   // ne[0] = cols (fastest), ne[1] = rows, ne[2] = experts
    uint64_t offset = 0;        // absolute file offset of the first byte
    uint64_t bytes = 0;
};

struct GgufFile {
    std::string path;
    uint32_t version = 0;
    uint64_t alignment = 32, data_offset = 0;
    std::map<std::string, GgufTensor> tensors;
    // the bytes of a tensor or of a slice
    std::vector<char> read(const GgufTensor & t) const {
        std::vector<char> out(t.bytes);
        FILE * f = std::fopen(path.c_str(), "rb");
        if (!f) throw std::runtime_error(path + ": cannot open");
        const bool ok = std::fseek(f, long(t.offset), SEEK_SET) == 0 && std::fread(out.data(), 1, out.size(), f) == out.size();
        std::fclose(f);
        if (!ok) throw std::runtime_error(path + ": short read");
        return out;
    }
};

// weights per block and bytes per block of the GGUF types an expert bank can have (gguf.cpp:116-152)
inline bool gguf_block_layout(uint32_t type, uint64_t & elems, uint64_t & bytes) {
    switch (type) {
        case 0: elems = 1; bytes = 4; return true;            // F32
        case 1: case 30: elems = 1; bytes = 2; return true;   // F16, BF16
        case 2: elems = 32; bytes = 18; return true;          // Q4_0
        case 3: elems = 32; bytes = 20; return true;          // Q4_1
        case 6: elems = 32; bytes = 22; return true;          // Q5_0
        case 7: elems = 32; bytes = 24; return true;          // Q5_1
        case 8: elems = 32; bytes = 34; return true;          // Q8_0
        case 10: elems = 256; bytes = 84; return true;        // Q2_K
        case 11: elems = 256; bytes = 110; return true;       // Q3_K
        case 12: elems = 256; bytes = 144; return true;       // Q4_K
        case 13: elems = 256; bytes = 176; return true;       // Q5_K
        case 14: elems = 256; bytes = 210; return true;       // Q6_K
        case 16: elems = 256; bytes = 66; return true;        // IQ2_XXS
        case 17: elems = 256; bytes = 74; return true;        // IQ2_XS
        case 18: elems = 256; bytes = 98; return true;        // IQ3_XXS
        case 19: elems = 256; bytes = 50; return true;        // IQ1_S
        case 20: elems = 32; bytes = 18; return true;         // IQ4_NL
        case 21: elems = 256; bytes = 110; return true;       // IQ3_S
        case 22: elems = 256; bytes = 82; return true;        // IQ2_S
        case 23: elems = 256; bytes = 136; return true;       // IQ4_XS
        case 323: elems = 128; bytes = 76; return true;       // NVFP4G
    }
    return false;
}

inline uint64_t gguf_expert_count(const GgufTensor & t) { return t.ne.size() == 3 ? t.ne[2] : 0; }

// One expert of a 3-D expert tensor [cols, rows, n_experts] as a 2-D tensor view of its own (the job of the reference's
// gguf_expert_slice, src/core/gguf.hpp:77-91). Fails closed: a tensor that is not 3-D, an empty expert axis, an index past
// it, a type without a block layout, rows that do not end on a block boundary (a row is what the loaders read, so the
// check is per row, not per expert), sizes that overflow 64 bits, or a byte count that disagrees with the one recorded
// when the file was opened all throw std::runtime_error naming the tensor.
struct ExpertGeometry { uint64_t experts, cols, rows, bytes_each; };
inline ExpertGeometry gguf_expert_geometry(const GgufTensor & t, const std::string & name) {
    auto fail = [&](const std::string & why) -> ExpertGeometry { throw std::runtime_error(name + ": " + why); };
    if (t.ne.size() != 3) return fail("expected a 3-D tensor [cols, rows, experts], found " + std::to_string(t.ne.size()) + " dimension(s)");
    ExpertGeometry g{t.ne[2], t.ne[0], t.ne[1], 0};
    if (g.experts == 0) return fail("the expert axis is empty");
    uint64_t block_elems = 0, block_bytes = 0;
    if (!gguf_block_layout(t.type, block_elems, block_bytes)) return fail("GGUF type " + std::to_string(t.type) + " has no block layout here");
    if (g.cols == 0 || g.rows == 0) return fail("an expert matrix of " + std::to_string(g.rows) + " x " + std::to_string(g.cols) + " holds nothing");
    if (g.cols % block_elems)
        return fail("rows of " + std::to_string(g.cols) + " weights do not end on the " + std::to_string(block_elems) + "-weight blocks of type " +
                    std::to_string(t.type));
    uint64_t row_bytes = 0, each = 0, all = 0;
    if (__builtin_mul_overflow(g.cols / block_elems, block_bytes, &row_bytes) || __builtin_mul_overflow(row_bytes, g.rows, &each) ||
        __builtin_mul_overflow(each, g.experts, &all))
        return fail("tensor size overflows 64 bits");
    if (all != t.bytes)
        return fail(std::to_string(g.experts) + " experts of " + std::to_string(each) + " bytes make " + std::to_string(all) + " bytes, the file records " +
                    std::to_string(t.bytes));
    g.bytes_each = each;
    return g;
}
inline GgufTensor gguf_expert_slice(const GgufTensor & t, uint64_t idx, const std::string & name) {
    const ExpertGeometry g = gguf_expert_geometry(t, name);
    if (idx >= g.experts) throw std::runtime_error(name + ": expert " + std::to_string(idx) + " requested, the tensor holds " + std::to_string(g.experts));
    GgufTensor view;
    view.type = t.type;
    view.ne = {g.cols, g.rows};
    view.bytes = g.bytes_each;
    view.offset = t.offset + idx * g.bytes_each;
    return view;
}

namespace gguf_detail {
struct Reader {
    FILE * f;
    const std::string & path;
    void raw(void * p, size_t n) { if (std::fread(p, 1, n, f) != n) throw std::runtime_error(path + ": truncated GGUF header"); }
    template <class T> T get() { T v; raw(&v, sizeof v); return v; }
    std::string str() {
        const uint64_t n = get<uint64_t>();
        if (n > (uint64_t(1) << 24)) throw std::runtime_error(path + ": implausible string length in GGUF header");
        std::string s(n, '\0');
        if (n) raw(&s[0], n);
        return s;
    }
    static size_t scalar_bytes(uint32_t t) {
        switch (t) { case 0: case 1: case 7: return 1; case 2: case 3: return 2; case 4: case 5: case 6: return 4; case 10: case 11: case 12: return 8; }
        return 0;
    }
    // skips a metadata value; returns it as u64 when it is an unsigned / signed integer scalar (for general.alignment)
    bool value(uint32_t type, uint64_t & as_int) {
        if (type == 8) { str(); return false; }
        if (type == 9) {
            const uint32_t et = get<uint32_t>();
            const uint64_t n = get<uint64_t>();
            for (uint64_t i = 0; i < n; ++i) { uint64_t dummy; value(et, dummy); }
            return false;
        }
        const size_t b = scalar_bytes(type);
        if (!b) throw std::runtime_error(path + ": unknown GGUF metadata type " + std::to_string(type));
        uint64_t v = 0;
        raw(&v, b);   // little-endian host
        as_int = v;
        return type == 0 || type == 1 || type == 2 || type == 3 || type == 4 || type == 5 || type == 10 || type == 11;
    }
};
}  // namespace gguf_detail

inline GgufFile gguf_open(const std::string & path) {
    FILE * fp = std::fopen(path.c_str(), "rb");
    if (!fp) throw std::runtime_error(path + ": cannot open");
    GgufFile out;
    out.path = path;
    try {
        gguf_detail::Reader r{fp, path};
        char magic[4];
        r.raw(magic, 4);
        if (magic[0] != 'G' || magic[1] != 'G' || magic[2] != 'U' || magic[3] != 'F') throw std::runtime_error(path + ": not a GGUF file");
        out.version = r.get<uint32_t>();
        if (out.version < 2 || out.version > 3) throw std::runtime_error(path + ": unsupported GGUF version " + std::to_string(out.version));
        const uint64_t n_tensors = r.get<uint64_t>(), n_kv = r.get<uint64_t>();
        for (uint64_t i = 0; i < n_kv; ++i) {
            const std::string key = r.str();
            const uint32_t type = r.get<uint32_t>();
            uint64_t v = 0;
            if (r.value(type, v) && key == "general.alignment" && v) out.alignment = v;
        }
        std::vector<std::pair<std::string, GgufTensor>> infos;
        for (uint64_t i = 0; i < n_tensors; ++i) {
            std::pair<std::string, GgufTensor> e;
            e.first = r.str();
            const uint32_t nd = r.get<uint32_t>();
            if (nd > 4) throw std::runtime_error(path + ": tensor " + e.first + " has " + std::to_string(nd) + " dimensions");
            for (uint32_t d = 0; d < nd; ++d) e.second.ne.push_back(r.get<uint64_t>());
            e.second.type = r.get<uint32_t>();
            e.second.offset = r.get<uint64_t>();   // relative to the data section until fixed below
            infos.push_back(e);
        }
        const uint64_t at = uint64_t(std::ftell(fp));
        out.data_offset = (at + out.alignment - 1) / out.alignment * out.alignment;
        std::fseek(fp, 0, SEEK_END);
        const uint64_t file_bytes = uint64_t(std::ftell(fp));
        for (auto & e : infos) {
            uint64_t blk = 0, bpb = 0, n = 1;
            for (uint64_t d : e.second.ne) n *= d;
            if (gguf_block_layout(e.second.type, blk, bpb)) {
                if (n % blk) throw std::runtime_error("GGUF tensor " + e.first + ": " + std::to_string(n) + " elements is not a multiple of the " + std::to_string(blk) +
                                                      "-element block of type " + std::to_string(e.second.type));
                e.second.bytes = n / blk * bpb;
            }
            e.second.offset += out.data_offset;
            if (e.second.offset + e.second.bytes > file_bytes) throw std::runtime_error("GGUF tensor " + e.first + " runs past the end of " + path);
            out.tensors[e.first] = e.second;
        }
    } catch (...) {
        std::fclose(fp);
        throw;
    }
    std::fclose(fp);
    return out;
}

// What tqmoe_bank_load needs for a whole expert tensor: the stacked block stream is the tensor's bytes as they lie.
struct GgufExpertBank { uint32_t type; int32_t experts, rows, cols; uint64_t offset, bytes; };
inline GgufExpertBank gguf_expert_bank(const GgufFile & f, const std::string & name) {
    const auto it = f.tensors.find(name);
    if (it == f.tensors.end()) throw std::runtime_error(f.path + ": no tensor " + name);
    const GgufTensor & t = it->second;
    gguf_expert_slice(t, 0, name);   // every consistency check of the slicer
    if (t.ne[0] > 0x7FFFFFFF || t.ne[1] > 0x7FFFFFFF || t.ne[2] > 0x7FFFFFFF) throw std::runtime_error(name + ": dimensions beyond 2^31");
    return GgufExpertBank{t.type, int32_t(t.ne[2]), int32_t(t.ne[1]), int32_t(t.ne[0]), t.offset, t.bytes};
}

}  // namespace tqmoe_hip
