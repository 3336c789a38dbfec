// Standalone C++ functional test of the C ABI (no Python, no torch), shaped after the reference's
// own native test (test/unit_test.cpp:219-331): fp32 data from rand(), token counts
// {513, 1257, 127, 778, 10024, 3} x hidden {1024, 508, 124}, every output compared with a CPU
// reference at atol 1e-4, one "validation:" line per case.
//
// Differences: one GPU holds all nranks partial buffers (nranks separate hipMalloc allocations);
// the CPU reference is the oracle's restatement of allreduce_rmsnorm_ref (oracle/tde_oracle.c),
// linked as a checker only; residual_out is additionally required to be bit-exact against the
// oracle's rank-order restatement.
//
// Build: python tests/native/build_native.py   (produces tests/native/unit_test_abi; links libtde_hip.so, built before
//        it by python torch_dist_ext_amd/_build.py)
// Run:   tests/native/unit_test_abi            (exit code 0 = every case validated)
#include <hip/hip_runtime.h>

#include <cmath>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "tde_abi.h"

extern "C" {
int tdo_unit_test_ref(const float *allreduce_in, const float *residual_in, const float *gamma, int64_t size, int64_t hidden,
                      int nranks, float *residual_out, float *norm_out, float eps);
int tdo_reduce_rms(int dtype, int nranks, int64_t tokens, int64_t hidden, const void *const *parts, const void *residual_in,
                   const void *gamma, float eps, int quant, int sumsq_mode, void *residual_out, void *norm_out,
                   uint8_t *q_out, float *scale_out);
}

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));            \
            std::exit(2);                                                                     \
        }                                                                                     \
    } while (0)

static bool run_case(int nranks, int tokens, int hidden, float eps, float atol) {
    const int64_t size = (int64_t)tokens * hidden;
    std::vector<float> parts((size_t)nranks * size), residual(size), gamma(hidden);
    for (auto &v : parts) v = rand() / (float)INT_MAX;
    for (auto &v : residual) v = rand() / (float)INT_MAX;
    for (auto &v : gamma) v = rand() / (float)INT_MAX;

    std::vector<void *> d_parts(nranks);
    void *d_res = nullptr, *d_gamma = nullptr, *d_res_out = nullptr, *d_norm = nullptr;
    for (int r = 0; r < nranks; ++r) {
        HIP_OK(hipMalloc(&d_parts[r], size * sizeof(float)));
        HIP_OK(hipMemcpy(d_parts[r], parts.data() + (size_t)r * size, size * sizeof(float), hipMemcpyHostToDevice));
    }
    HIP_OK(hipMalloc(&d_res, size * sizeof(float)));
    HIP_OK(hipMalloc(&d_res_out, size * sizeof(float)));
    HIP_OK(hipMalloc(&d_norm, size * sizeof(float)));
    HIP_OK(hipMalloc(&d_gamma, hidden * sizeof(float)));
    HIP_OK(hipMemcpy(d_res, residual.data(), size * sizeof(float), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_gamma, gamma.data(), hidden * sizeof(float), hipMemcpyHostToDevice));

    tde_problem p{};
    p.dtype = TDE_F32;
    p.nranks = nranks;
    p.tokens = tokens;
    p.hidden = hidden;
    p.eps = eps;
    tde_buffers b{};
    for (int r = 0; r < nranks; ++r) b.partial[r] = d_parts[r];
    b.residual_in = d_res;
    b.residual_out = d_res_out;
    b.norm_out = d_norm;
    b.gamma = d_gamma;
    tde_plan_out plan{};
    int st = tde_plan(&p, &plan);
    if (st == TDE_OK) st = tde_reduce_rms(&p, &b, nullptr);
    if (st != TDE_OK) {
        std::fprintf(stderr, "tde_reduce_rms: %s (hip %d)\n", tde_status_string(st), tde_last_hip_error());
        std::exit(2);
    }
    HIP_OK(hipDeviceSynchronize());

    std::vector<float> res_out(size), norm_out(size), res_ref(size), norm_ref(size), res_exact(size), norm_exact(size);
    HIP_OK(hipMemcpy(res_out.data(), d_res_out, size * sizeof(float), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(norm_out.data(), d_norm, size * sizeof(float), hipMemcpyDeviceToHost));
    tdo_unit_test_ref(parts.data(), residual.data(), gamma.data(), size, hidden, nranks, res_ref.data(), norm_ref.data(), eps);
    std::vector<const void *> host_parts(nranks);
    for (int r = 0; r < nranks; ++r) host_parts[r] = parts.data() + (size_t)r * size;
    tdo_reduce_rms(/*f32*/ 2, nranks, tokens, hidden, host_parts.data(), residual.data(), gamma.data(), eps, 0, /*f64 sumsq*/ 1,
                   res_exact.data(), norm_exact.data(), nullptr, nullptr);

    bool ok = true;
    for (int64_t i = 0; i < size && ok; ++i) {
        if (std::isnan(res_out[i]) || std::fabs(res_out[i] - res_ref[i]) > atol) ok = false;
        if (std::isnan(norm_out[i]) || std::fabs(norm_out[i] - norm_ref[i]) > atol) ok = false;
        if (std::memcmp(&res_out[i], &res_exact[i], sizeof(float)) != 0) ok = false; // rank-order sum, bit for bit
        if (std::fabs(norm_out[i] - norm_exact[i]) > 4e-6f * std::fabs(norm_exact[i]) + 1e-30f) ok = false;
    }
    for (auto ptr : d_parts) HIP_OK(hipFree(ptr));
    HIP_OK(hipFree(d_res));
    HIP_OK(hipFree(d_res_out));
    HIP_OK(hipFree(d_norm));
    HIP_OK(hipFree(d_gamma));
    std::printf("nranks:%d num_tokens:%d hidden_dim:%d block:%d grid:%d validation:%d\n", nranks, tokens, hidden,
                plan.block_threads, plan.grid_blocks, ok ? 1 : 0);
    std::fflush(stdout);
    return ok;
}

int main() {
    int ngpus = 0;
    HIP_OK(hipGetDeviceCount(&ngpus));
    if (ngpus < 1) {
        std::fprintf(stderr, "no GPU\n");
        return 2;
    }
    HIP_OK(hipSetDevice(0));
    std::printf("abi version:%d\n", tde_abi_version());
    const int tokens[] = {513, 1257, 127, 778, 10024, 3};
    const int hidden[] = {1024, 512 - 4, 124};
    const int ranks[] = {8, 4, 2};
    bool all = true;
    int k = 0;
    for (int t : tokens)
        for (int h : hidden) all = run_case(ranks[k++ % 3], t, h, 1e-6f, 1e-4f) && all;
    // argument errors come back as status codes, never as aborts
    tde_problem bad{};
    bad.dtype = TDE_F32;
    bad.nranks = 3;
    bad.tokens = 1;
    bad.hidden = 4;
    tde_plan_out plan{};
    all = (tde_plan(&bad, &plan) == TDE_ENRANKS) && all;
    std::printf("all:%d\n", all ? 1 : 0);
    return all ? 0 : 1;
}
