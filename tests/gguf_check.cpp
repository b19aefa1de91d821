// Host check of include/tqmoe_gguf.hpp against a synthetic GGUF file written by tests/test_gguf.py: the cases of the
// reference's tests/moe_experts.cpp (every slice must read ITS OWN expert; inconsistencies must throw).
// usage: gguf_check <file> <cols> <rows> <experts>   tensors: experts.f32 (value e * 10000 + r * 100 + c), experts.q2k
// (every byte of expert e is 0xE0 + e). Prints one line per check; exit code = number of failures.
#include <cstdlib>
#include <cstring>

#include "tqmoe_gguf.hpp"

using namespace tqmoe_hip;

static int failures = 0;
static void check(bool ok, const char * what) {
    std::printf("   %s %s\n", ok ? "ok  " : "FAIL", what);
    if (!ok) ++failures;
}
static bool throws(const GgufTensor & t, uint64_t idx) {
    try { gguf_expert_slice(t, idx, "t"); return false; } catch (const std::runtime_error &) { return true; }
}

int main(int argc, char ** argv) {
    if (argc < 5) return 100;
    const uint64_t COLS = std::strtoull(argv[2], nullptr, 10), ROWS = std::strtoull(argv[3], nullptr, 10), N_EXP = std::strtoull(argv[4], nullptr, 10);
    const GgufFile f = gguf_open(argv[1]);
    const GgufTensor & t = f.tensors.at("experts.f32");
    check(gguf_expert_count(t) == N_EXP, "expert count");
    check(t.ne.size() == 3 && t.ne[0] == COLS && t.ne[1] == ROWS && t.ne[2] == N_EXP, "tensor dims are [COLS][ROWS][N_EXP]");
    const std::vector<char> whole = f.read(t);
    check(whole.size() == COLS * ROWS * N_EXP * 4, "whole tensor byte count");
    bool all_ok = true, values_ok = true;
    for (uint64_t e = 0; e < N_EXP; ++e) {
        const GgufTensor s = gguf_expert_slice(t, e, "experts.f32");
        if (s.ne.size() != 2 || s.ne[0] != COLS || s.ne[1] != ROWS || s.bytes != COLS * ROWS * 4) { all_ok = false; break; }
        const std::vector<char> got = f.read(s);
        if (got.size() != s.bytes || std::memcmp(got.data(), whole.data() + e * s.bytes, s.bytes) != 0) { all_ok = false; break; }
        const float * v = reinterpret_cast<const float *>(got.data());
        if (v[0] != float(e * 10000) || v[COLS * ROWS - 1] != float(e * 10000 + (ROWS - 1) * 100 + (COLS - 1))) values_ok = false;
    }
    check(all_ok, "every slice is byte-identical to its own expert span");
    check(values_ok, "sliced values identify the correct expert (first and last element)");
    const GgufTensor & q = f.tensors.at("experts.q2k");
    bool q_ok = gguf_expert_count(q) == N_EXP;
    for (uint64_t e = 0; e < N_EXP && q_ok; ++e) {
        const GgufTensor s = gguf_expert_slice(q, e, "experts.q2k");
        if (s.bytes != COLS * ROWS / 256 * 84) { q_ok = false; break; }
        for (char c : f.read(s)) if (uint8_t(c) != uint8_t(0xE0 + e)) { q_ok = false; break; }
    }
    check(q_ok, "each Q2_K slice reads exactly its own expert's bytes");
    const GgufExpertBank b = gguf_expert_bank(f, "experts.q2k");
    check(b.type == 10 && uint64_t(b.experts) == N_EXP && uint64_t(b.rows) == ROWS && uint64_t(b.cols) == COLS && b.bytes == q.bytes && b.offset == q.offset,
          "bank descriptor of the whole tensor");
    // fail-closed behaviour
    GgufTensor good;
    good.type = 0; good.ne = {COLS, ROWS, N_EXP}; good.offset = 0; good.bytes = COLS * ROWS * N_EXP * 4;
    check(!throws(good, 0), "a consistent descriptor does not throw");
    check(throws(good, N_EXP), "index == n_experts throws");
    check(throws(good, N_EXP + 100), "index far out of range throws");
    GgufTensor two_d = good; two_d.ne = {COLS, ROWS};
    check(throws(two_d, 0), "2-D tensor throws");
    GgufTensor zero_exp = good; zero_exp.ne = {COLS, ROWS, 0};
    check(throws(zero_exp, 0), "zero experts throws");
    GgufTensor bad_bytes = good; bad_bytes.bytes = good.bytes + 4;
    check(throws(bad_bytes, 0), "byte-count mismatch throws");
    GgufTensor bad_block; bad_block.type = 10; bad_block.ne = {100, 7, N_EXP}; bad_block.offset = 0; bad_block.bytes = 100 * 7 * N_EXP;
    check(throws(bad_block, 0), "per-expert count not block-aligned throws");
    GgufTensor four_d = good; four_d.ne = {COLS, ROWS, N_EXP, 2};
    check(throws(four_d, 0), "4-D tensor throws");
    GgufTensor bad_type = good; bad_type.type = 9999;
    check(throws(bad_type, 0), "unknown type throws");
    bool no_file = false;
    try { gguf_open(std::string(argv[1]) + ".missing"); } catch (const std::runtime_error &) { no_file = true; }
    check(no_file, "a missing file throws");
    return failures;
}
