// A C++ host that drives the library the way the reference's llm.c benchmark does
// (example_llmc_rope.cu:132-144 and :243-316): the packed (B, T, 3*NH, HS) fp32 tensor comes from
// sideaware_malloc, the table from the runtime's own allocator, the op header is the one-line
// `#include "<file>"` resolved in the working directory, the kernel runs in place through
// sideaware_elementwise with every optional argument zero, and the result is held against the CPU
// oracle with llm.c's tolerance rule.  Forward, then backward of the forward's output.
//
// usage: llmc_rope_host <fwd_header_file> <bwd_header_file> B T NH HS
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/sideaware.h"

extern "C" {
void oracle_freqs_cis(float* freqs_cis, int dim, int end, float theta, int use_scaled);
void oracle_rope_forward_qkv_f32(float* out, const float* inp, const float* freqs_cis, int B, int T, int Nq,
                                 int Nkv, int head_dim);
void oracle_rope_backward_qkv_f32(float* dinp, const float* dout, const float* freqs_cis, int B, int T, int Nq,
                                  int Nkv, int head_dim);
size_t oracle_validate_f32(const float* got, const float* ref, size_t n, float tolerance);
}

#define HIP_OK(call)                                                                              \
    do {                                                                                          \
        hipError_t e_ = (call);                                                                   \
        if (e_ != hipSuccess) {                                                                   \
            std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                \
            return 10;                                                                            \
        }                                                                                         \
    } while (0)

static int run_in_place(int kernel, float* d_inout, const float* d_freqs, size_t bytes) {
    sideaware_elementwise(kernel, bytes, d_inout, nullptr, nullptr, nullptr, d_inout, d_freqs, nullptr, nullptr,
                          nullptr, 0, 0, 0, 0, nullptr);
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

static size_t differing_bits(const float* a, const float* b, size_t n) {
    size_t bad = 0;
    for (size_t i = 0; i < n; i++) {
        uint32_t x, y;
        std::memcpy(&x, a + i, 4);
        std::memcpy(&y, b + i, 4);
        bad += x != y;
    }
    return bad;
}

int main(int argc, char** argv) {
    if (argc != 7) {
        std::fprintf(stderr, "usage: %s fwd_header bwd_header B T NH HS\n", argv[0]);
        return 2;
    }
    const std::string fwd = std::string("#include \"") + argv[1] + "\"\n";
    const std::string bwd = std::string("#include \"") + argv[2] + "\"\n";
    const int B = std::atoi(argv[3]), T = std::atoi(argv[4]), NH = std::atoi(argv[5]), HS = std::atoi(argv[6]);
    const size_t n = (size_t)B * T * 3 * NH * HS, bytes = n * sizeof(float);

    // CPU side: inputs in [-1, 1) from a fixed linear congruential generator, the table with
    // Llama-3.1 scaling as the reference's main() asks for it (theta 10000, use_scaled 1)
    std::vector<float> inp(n), out(n), dinp(n), got(n), freqs((size_t)T * HS);
    uint32_t state = 12345u;
    for (size_t i = 0; i < n; i++) {
        state = state * 1664525u + 1013904223u;
        inp[i] = (float)(state >> 8) * (2.0f / 16777216.0f) - 1.0f;
    }
    oracle_freqs_cis(freqs.data(), HS, T, 10000.0f, 1);
    oracle_rope_forward_qkv_f32(out.data(), inp.data(), freqs.data(), B, T, NH, NH, HS);
    oracle_rope_backward_qkv_f32(dinp.data(), out.data(), freqs.data(), B, T, NH, NH, HS);

    HIP_OK(hipSetDevice(0));
    float *d_inout = nullptr, *d_freqs = nullptr;
    if (sideaware_malloc((void**)&d_inout, bytes) != 0 || !d_inout) {
        std::fprintf(stderr, "sideaware_malloc failed: %s\n", sideaware_last_error());
        return 3;
    }
    if ((uintptr_t)d_inout % (2u << 20)) return 4;                    // large regions are 2 MiB aligned
    HIP_OK(hipMalloc((void**)&d_freqs, freqs.size() * sizeof(float)));
    HIP_OK(hipMemcpy(d_freqs, freqs.data(), freqs.size() * sizeof(float), hipMemcpyHostToDevice));

    sideaware_write_sass("isa.txt");
    const int k_fwd = sideaware_create_kernel(fwd.c_str());
    const int k_bwd = sideaware_create_kernel(bwd.c_str());
    if (k_fwd < 1 || k_bwd < 1 || k_fwd == k_bwd || sideaware_create_kernel(fwd.c_str()) != k_fwd) return 5;

    // in place: restore the input before every call, as the reference's loop does
    for (int round = 0; round < 2; round++) {
        HIP_OK(hipMemcpy(d_inout, inp.data(), bytes, hipMemcpyHostToDevice));
        if (run_in_place(k_fwd, d_inout, d_freqs, bytes)) return 6;
        HIP_OK(hipMemcpy(got.data(), d_inout, bytes, hipMemcpyDeviceToHost));
        size_t faults = oracle_validate_f32(got.data(), out.data(), n, 1e-5f);
        size_t bits = differing_bits(got.data(), out.data(), n);
        std::printf("forward round %d: %zu faults, %zu values differ in any bit\n", round, faults, bits);
        if (faults || bits) return 7;
    }
    HIP_OK(hipMemcpy(d_inout, out.data(), bytes, hipMemcpyHostToDevice));
    if (run_in_place(k_bwd, d_inout, d_freqs, bytes)) return 6;
    HIP_OK(hipMemcpy(got.data(), d_inout, bytes, hipMemcpyDeviceToHost));
    {
        size_t faults = oracle_validate_f32(got.data(), dinp.data(), n, 1e-5f);
        size_t bits = differing_bits(got.data(), dinp.data(), n);
        std::printf("backward: %zu faults, %zu values differ in any bit\n", faults, bits);
        if (faults || bits) return 8;
    }
    if (sideaware_last_error()[0]) {
        std::fprintf(stderr, "library error: %s\n", sideaware_last_error());
        return 9;
    }
    if (sideaware_free(d_inout) != 0) return 11;
    HIP_OK(hipFree(d_freqs));
    std::printf("llmc rope host ok\n");
    return 0;
}
