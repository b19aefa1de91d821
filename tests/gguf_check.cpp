// Host check of include/tqmoe_gguf.hpp on the synthetic GGUF file tests/test_gguf.py writes. The property under test is
// the one the reference's tests/moe_experts.cpp is about: slicing a stacked expert tensor must hand back each expert's
// own bytes (a wrong stride reads a neighbour), and every inconsistent descriptor must be refused.
// usage: gguf_check <file> <cols> <rows> <experts>
// The file holds "experts.f32" (element value = expert * 10000 + row * 100 + col) and "experts.q2k" (every byte of expert
// e is 0xE0 + e). One line per check; the exit code is the number of failed checks.
#include <cstdlib>
#include <cstring>
#include <functional>

#include "tqmoe_gguf.hpp"

using namespace tqmoe_hip;

static int failed = 0;
static void report(const char * what, bool ok) {
    std::printf("   %s %s\n", ok ? "ok  " : "FAIL", what);
    failed += ok ? 0 : 1;
}
static bool refused(const std::function<void()> & f) {
    try { f(); } catch (const std::runtime_error &) { return true; }
    return false;
}

int main(int argc, char ** argv) {
    if (argc < 5) return 100;
    const uint64_t cols = std::strtoull(argv[2], nullptr, 10), rows = std::strtoull(argv[3], nullptr, 10), experts = std::strtoull(argv[4], nullptr, 10);
    const GgufFile file = gguf_open(argv[1]);

    // ---- fp32 tensor: every element names its expert, row and column
    const GgufTensor & plain = file.tensors.at("experts.f32");
    report("fp32 tensor: three dimensions, cols x rows x experts", plain.ne == std::vector<uint64_t>{cols, rows, experts});
    report("fp32 tensor: expert count", gguf_expert_count(plain) == experts);
    const std::vector<char> everything = file.read(plain);
    report("fp32 tensor: bytes of the whole tensor", everything.size() == cols * rows * experts * sizeof(float));
    bool shape = true, bytes = true, values = true;
    for (uint64_t e = 0; e < experts; ++e) {
        const GgufTensor one = gguf_expert_slice(plain, e, "experts.f32");
        shape = shape && one.ne == std::vector<uint64_t>{cols, rows} && one.bytes == cols * rows * sizeof(float) && one.type == plain.type;
        const std::vector<char> data = file.read(one);
        bytes = bytes && data.size() == one.bytes && !std::memcmp(data.data(), everything.data() + e * one.bytes, one.bytes);
        if (data.size() != one.bytes) break;
        float first, last;
        std::memcpy(&first, data.data(), 4);
        std::memcpy(&last, data.data() + one.bytes - 4, 4);
        values = values && first == float(e * 10000) && last == float(e * 10000 + (rows - 1) * 100 + (cols - 1));
    }
    report("fp32 slices: 2-D views of one expert's size", shape);
    report("fp32 slices: the bytes of the expert's own span of the tensor", bytes);
    report("fp32 slices: first and last value carry the slice's expert number", values);

    // ---- Q2_K tensor: block format, every byte names its expert
    const GgufTensor & blocks = file.tensors.at("experts.q2k");
    bool own = gguf_expert_count(blocks) == experts;
    for (uint64_t e = 0; e < experts && own; ++e) {
        const GgufTensor one = gguf_expert_slice(blocks, e, "experts.q2k");
        own = one.bytes == cols * rows / 256 * 84;
        for (char c : file.read(one)) own = own && uint8_t(c) == uint8_t(0xE0 + e);
    }
    report("Q2_K slices: 84 bytes per 256 weights, all of them the expert's own", own);
    const GgufExpertBank bank = gguf_expert_bank(file, "experts.q2k");
    report("Q2_K bank: the whole tensor as one stacked bank", bank.type == 10 && uint64_t(bank.experts) == experts && uint64_t(bank.rows) == rows &&
                                                                   uint64_t(bank.cols) == cols && bank.offset == blocks.offset && bank.bytes == blocks.bytes);

    // ---- descriptors that must be refused (built here, no file behind them)
    GgufTensor sound;
    sound.type = 0;
    sound.ne = {cols, rows, experts};
    sound.offset = 0;
    sound.bytes = cols * rows * experts * 4;
    auto slice_refused = [](GgufTensor t, uint64_t idx) { return refused([&] { gguf_expert_slice(t, idx, "t"); }); };
    report("accepted: a consistent descriptor", !slice_refused(sound, 0) && !slice_refused(sound, experts - 1));
    report("refused: the index one past the last expert", slice_refused(sound, experts));
    report("refused: an index far past the end", slice_refused(sound, experts + 100));
    { GgufTensor t = sound; t.ne = {cols, rows}; report("refused: a 2-D tensor", slice_refused(t, 0)); }
    { GgufTensor t = sound; t.ne = {cols, rows, experts, 2}; report("refused: a 4-D tensor", slice_refused(t, 0)); }
    { GgufTensor t = sound; t.ne = {cols, rows, 0}; report("refused: an empty expert axis", slice_refused(t, 0)); }
    { GgufTensor t = sound; t.bytes += 4; report("refused: a byte count other than experts x expert size", slice_refused(t, 0)); }
    { GgufTensor t = sound; t.type = 9999; report("refused: a type without a block layout", slice_refused(t, 0)); }
    {
        GgufTensor t;   // Q2_K rows of 100 weights: no whole number of 256-weight blocks
        t.type = 10; t.ne = {100, 7, experts}; t.offset = 0; t.bytes = 100 * 7 * experts;
        report("refused: rows that do not end on a block boundary", slice_refused(t, 0));
    }
    {
        GgufTensor t;   // 128 x 2 weights fill one Q2_K block per expert, but a row of 128 does not: rows are what loaders read
        t.type = 10; t.ne = {128, 2, experts}; t.offset = 0; t.bytes = 84 * experts;
        report("refused: an expert of whole blocks whose rows are not", slice_refused(t, 0));
    }
    {
        GgufTensor t = sound;   // sizes whose product leaves 64 bits
        t.ne = {uint64_t(1) << 40, uint64_t(1) << 30, 4};
        t.bytes = 0;
        report("refused: dimensions whose byte count overflows", slice_refused(t, 0));
    }
    report("refused: a file that does not exist", refused([&] { gguf_open(std::string(argv[1]) + ".missing"); }));
    return failed;
}
