// Drives include/tqmoe_adapter.hpp the way the reference's engine would: through a base class with the expert virtuals
// of tqllm::WeightFormat, called by base pointer. The base below restates those virtuals' signatures
// (src/formats/weight/weight_format.hpp:22-28, 51-73) with stand-in element types, so that the `override`s of
// tqmoe_hip::ExpertOverrides only compile if they match; then one decode product pair, one decode product with a row per
// assignment, the two grouped products over counts / groups / capacity, the int8 grouped product on the reference's own
// operands (both activation modes) and moe_group with the reference's seven arguments run on the GPU, and their results are
// written out for tests/test_gpu_adapter.py, which compares them with the oracle.
//
// usage: adapter_check <dir>   reads <dir>/meta.txt (type experts rows cols n topk capacity) and the arrays
// gate.bin, up.bin (GGUF blocks), x.bin (fp16 [n][cols]), ids.bin (int32 [n][topk]), counts.bin, groups.bin, and for the int8
// product xq1.bin / xq2.bin (int8 [n][cols], natural order: quantised per block / per token), xs1.bin / xs2.bin (fp32
// [n][cols / 32]: a scale per block / the token's scale repeated), xsum.bin (int16 [n][cols / 32][2]); writes yg.bin, yu.bin, y1.bin (bf16 [n * topk][rows]), act.bin (fp16), yd.bin
// (bf16), dg.bin / du.bin / dg1.bin (bf16: expert_matvec_dedup2 and expert_matvec_dedup over maps built by moe_dedup_maps), yi1.bin / yi2.bin (bf16: the int8 product in modes 1 and 2; absent when the format has none), ycap.bin (bf16: expert_gemm
// with a capacity below the largest count), mg_counts.bin / mg_groups.bin (int32: moe_group)
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <fstream>
#include <string>
#include <vector>

#include "tqmoe_adapter.hpp"

struct __half { uint16_t bits; };
struct __nv_bfloat16 { uint16_t bits; };
using cudaStream_t = hipStream_t;

namespace tqllm {
struct WeightFormat;
struct Mat {
    const void * p = nullptr;
    uint32_t type = 30;
    int rows = 0, cols = 0;
    const void * aux = nullptr;
    const WeightFormat * fmt = nullptr;
};
struct WeightFormat {
    virtual ~WeightFormat() = default;
    virtual bool expert_gemm(const Mat &, const __half *, __nv_bfloat16 *, int, const int *, const int *, int, int, int, bool, cudaStream_t) const { return false; }
    virtual bool expert_gemm_i8(const Mat &, const int8_t *, const float *, const int16_t *, __nv_bfloat16 *, int, const int *, const int *, int, int, int, bool,
                                cudaStream_t, int) const { return false; }
    virtual bool expert_gemm_gateup(const Mat &, const Mat &, const __half *, __half *, int, const int *, const int *, int, int, int, cudaStream_t) const { return false; }
    virtual bool has_expert_matvec() const { return false; }
    virtual void expert_matvec(const Mat &, const __half *, __nv_bfloat16 *, int, const int *, int, int, bool, cudaStream_t) const {}
    virtual void expert_matvec2(const Mat &, const Mat &, const __half *, __nv_bfloat16 *, __nv_bfloat16 *, int, const int *, int, int, cudaStream_t) const {}
    virtual int u4h_id() const { return -1; }
    virtual bool has_expert_dedup() const { return u4h_id() >= 0; }
    virtual void expert_matvec_dedup(const Mat &, const __half *, __nv_bfloat16 *, int, const int *, int, cudaStream_t) const {}
    virtual void expert_matvec_dedup2(const Mat &, const Mat &, const __half *, __nv_bfloat16 *, __nv_bfloat16 *, int, const int *, int, cudaStream_t) const {}
};
}  // namespace tqllm

struct HipExperts final : tqmoe_hip::ExpertOverrides<tqllm::WeightFormat, tqllm::Mat, __half, __nv_bfloat16, cudaStream_t> {};

static void hip(hipError_t rc, const char * what) {
    if (rc != hipSuccess) { std::fprintf(stderr, "%s: %s\n", what, hipGetErrorString(rc)); std::exit(2); }
}
static std::vector<char> slurp(const std::string & path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) { std::fprintf(stderr, "cannot read %s\n", path.c_str()); std::exit(2); }
    return std::vector<char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}
static void * to_device(const std::vector<char> & h) {
    void * d = nullptr;
    hip(hipMalloc(&d, h.size()), "hipMalloc");
    hip(hipMemcpy(d, h.data(), h.size(), hipMemcpyHostToDevice), "hipMemcpy");
    return d;
}
static void * device_zeros(size_t bytes) {
    void * d = nullptr;
    hip(hipMalloc(&d, bytes), "hipMalloc");
    hip(hipMemset(d, 0, bytes), "hipMemset");
    return d;
}
static void dump(const std::string & path, const void * dev, size_t bytes) {
    std::vector<char> h(bytes);
    hip(hipMemcpy(h.data(), dev, bytes, hipMemcpyDeviceToHost), "hipMemcpy back");
    std::ofstream(path, std::ios::binary).write(h.data(), std::streamsize(bytes));
}

int main(int argc, char ** argv) {
    if (argc < 2) return 100;
    const std::string dir = argv[1];
    unsigned type;
    int experts, rows, cols, n, topk, capacity;
    {
        std::ifstream meta(dir + "/meta.txt");
        meta >> type >> experts >> rows >> cols >> n >> topk >> capacity;
        if (!meta) { std::fprintf(stderr, "bad meta.txt\n"); return 2; }
    }
    const int A = n * topk;
    try {
        HipExperts fmt;
        const tqllm::WeightFormat * base = &fmt;
        // banks: WeightFormat::load's job, with the library's loader on the uploaded GGUF bytes
        tqllm::Mat mats[2];
        const char * names[2] = {"/gate.bin", "/up.bin"};
        for (int i = 0; i < 2; ++i) {
            size_t cb = 0, ab = 0;
            tqmoe_error e = tqmoe_hip::fresh();
            tqmoe_hip::check(tqmoe_bank_layout(type, int64_t(experts) * rows, cols, &cb, &ab, &e), e);
            void * staged = to_device(slurp(dir + names[i]));
            void * codes = device_zeros(cb), * aux = device_zeros(ab);
            tqmoe_hip::ExpertFormat::load(type, staged, experts, rows, cols, codes, aux, nullptr, nullptr);
            mats[i].p = codes; mats[i].aux = aux; mats[i].type = type; mats[i].rows = experts * rows; mats[i].cols = cols; mats[i].fmt = base;
        }
        const __half * x = static_cast<const __half *>(to_device(slurp(dir + "/x.bin")));
        const int * ids = static_cast<const int *>(to_device(slurp(dir + "/ids.bin")));
        const int * counts = static_cast<const int *>(to_device(slurp(dir + "/counts.bin")));
        const int * groups = static_cast<const int *>(to_device(slurp(dir + "/groups.bin")));
        size_t sb = tqmoe_hip::expert_scratch_bytes(cols, A, A, experts, 1);
        sb = std::max(sb, tqmoe_expert_matvec_dedup_scratch_bytes(A, rows, cols, TQMOE_BF16, 1));
        fmt.set_scratch(device_zeros(sb), sb);
        fmt.max_assignments = A;

        if (!base->has_expert_matvec()) return 3;
        const size_t ybytes = size_t(A) * rows * 2;
        __nv_bfloat16 * yg = static_cast<__nv_bfloat16 *>(device_zeros(ybytes)), * yu = static_cast<__nv_bfloat16 *>(device_zeros(ybytes));
        __nv_bfloat16 * y1 = static_cast<__nv_bfloat16 *>(device_zeros(ybytes)), * yd = static_cast<__nv_bfloat16 *>(device_zeros(ybytes));
        __half * act = static_cast<__half *>(device_zeros(ybytes));
        base->expert_matvec2(mats[0], mats[1], x, yg, yu, rows, ids, n, topk, nullptr);
        base->expert_matvec(mats[0], x, y1, rows, ids, n, topk, false, nullptr);
        if (!base->expert_gemm_gateup(mats[0], mats[1], x, act, rows, counts, groups, capacity, experts, topk, nullptr)) return 4;
        if (!base->expert_gemm(mats[1], x, yd, rows, counts, groups, capacity, experts, topk, false, nullptr)) return 5;
        // the int8 grouped product on the rows the reference's activation quantiser leaves, both modes; `false` = no such kernel
        {
            const int8_t * xq = static_cast<const int8_t *>(to_device(slurp(dir + "/xq1.bin"))), * xq2 = static_cast<const int8_t *>(to_device(slurp(dir + "/xq2.bin")));
            const float * xs1 = static_cast<const float *>(to_device(slurp(dir + "/xs1.bin"))), * xs2 = static_cast<const float *>(to_device(slurp(dir + "/xs2.bin")));
            const int16_t * xsum = static_cast<const int16_t *>(to_device(slurp(dir + "/xsum.bin")));
            __nv_bfloat16 * yi = static_cast<__nv_bfloat16 *>(device_zeros(ybytes));
            if (base->expert_gemm_i8(mats[1], xq, xs1, xsum, yi, rows, counts, groups, capacity, experts, topk, false, nullptr, 1)) {
                hip(hipDeviceSynchronize(), "synchronize");
                dump(dir + "/yi1.bin", yi, ybytes);
                hip(hipMemset(yi, 0, ybytes), "hipMemset");
                if (!base->expert_gemm_i8(mats[1], xq2, xs2, xsum, yi, rows, counts, groups, capacity, experts, topk, false, nullptr, 2)) return 7;
                hip(hipDeviceSynchronize(), "synchronize");
                dump(dir + "/yi2.bin", yi, ybytes);
            }
            if (base->expert_gemm_i8(mats[1], xq, xs2, xsum, yi, rows, counts, groups, capacity, experts, topk, false, nullptr, 3)) return 8;   // the v3 modes: not here
        }
        // a capacity below the largest count: the lists are cut at the capacity, and so must the products be (no row of another
        // expert's list, no row twice)
        {
            __nv_bfloat16 * ycap = static_cast<__nv_bfloat16 *>(device_zeros(ybytes));
            std::vector<char> gh = slurp(dir + "/groups.bin");
            const int cap2 = 3;
            std::vector<int> cut(size_t(experts) * cap2);
            for (int e = 0; e < experts; ++e) for (int j = 0; j < cap2; ++j) cut[size_t(e) * cap2 + j] = reinterpret_cast<const int *>(gh.data())[size_t(e) * capacity + j];
            const int * groups2 = static_cast<const int *>(to_device(std::vector<char>(reinterpret_cast<const char *>(cut.data()), reinterpret_cast<const char *>(cut.data() + cut.size()))));
            if (!base->expert_gemm(mats[1], x, ycap, rows, counts, groups2, cap2, experts, topk, false, nullptr)) return 9;
            hip(hipDeviceSynchronize(), "synchronize");
            dump(dir + "/ycap.bin", ycap, ybytes);
        }
        // the decode grouping maps built on the device (moe_dedup_maps, every expert in its own bank slot) and the pair of products
        // over them: the rows must be those of expert_matvec2 over the ids
        if (A <= 1024) {
            if (!base->has_expert_dedup()) return 11;
            std::vector<int> ident(experts);
            for (int e = 0; e < experts; ++e) ident[e] = e;
            const int * slot_of = static_cast<const int *>(to_device(std::vector<char>(reinterpret_cast<const char *>(ident.data()), reinterpret_cast<const char *>(ident.data() + experts))));
            int * gu = static_cast<int *>(device_zeros(size_t(A) * tqmoe_hip::kDedupStride * 4)), * dn = static_cast<int *>(device_zeros(size_t(A) * tqmoe_hip::kDedupStride * 4));
            tqmoe_hip::moe_dedup_maps(ids, slot_of, A, topk, nullptr, gu, dn, A, nullptr);
            __nv_bfloat16 * dg = static_cast<__nv_bfloat16 *>(device_zeros(ybytes)), * du = static_cast<__nv_bfloat16 *>(device_zeros(ybytes));
            base->expert_matvec_dedup2(mats[0], mats[1], x, dg, du, rows, gu, A, nullptr);
            hip(hipDeviceSynchronize(), "synchronize");
            dump(dir + "/dg.bin", dg, ybytes);
            dump(dir + "/du.bin", du, ybytes);
            hip(hipMemset(dg, 0, ybytes), "hipMemset");
            base->expert_matvec_dedup(mats[0], x, dg, rows, gu, A, nullptr);
            hip(hipDeviceSynchronize(), "synchronize");
            dump(dir + "/dg1.bin", dg, ybytes);
        }
        // moe_group with the reference's seven arguments (moe_kernels.cuh:29): counts [experts], groups [experts][n]
        {
            int * mc = static_cast<int *>(device_zeros(size_t(experts) * 4));
            std::vector<char> fill(size_t(experts) * n * 4, char(0xFF));
            int * mg = static_cast<int *>(to_device(fill));
            tqmoe_hip::moe_group(ids, mc, mg, experts, n, topk, nullptr);
            hip(hipDeviceSynchronize(), "synchronize");
            dump(dir + "/mg_counts.bin", mc, size_t(experts) * 4);
            dump(dir + "/mg_groups.bin", mg, size_t(experts) * n * 4);
        }
        hip(hipDeviceSynchronize(), "synchronize");
        dump(dir + "/yg.bin", yg, ybytes);
        dump(dir + "/yu.bin", yu, ybytes);
        dump(dir + "/y1.bin", y1, ybytes);
        dump(dir + "/act.bin", act, ybytes);
        dump(dir + "/yd.bin", yd, ybytes);
        // a bad shape must throw std::invalid_argument, as the reference's entry points do (quant.cu:72-74)
        bool threw = false;
        try { base->expert_matvec(mats[0], x, y1, rows, ids, 0, topk, false, nullptr); } catch (const std::invalid_argument &) { threw = true; }
        if (!threw) return 6;
        // lists for another number of experts than the bank holds: refused, not read past the arrays
        threw = false;
        try { base->expert_gemm(mats[1], x, yd, rows, counts, groups, capacity, experts - 1, topk, false, nullptr); } catch (const std::invalid_argument &) { threw = true; }
        if (!threw) return 10;
    } catch (const std::exception & ex) {
        std::fprintf(stderr, "adapter_check: %s\n", ex.what());
        return 1;
    }
    std::printf("adapter_check ok\n");
    return 0;
}
