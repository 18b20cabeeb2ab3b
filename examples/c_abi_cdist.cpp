// The C ABI without Python: an L1 distance matrix and a Laplace kernel matrix
// computed by libkermac_amd.so from a plain HIP host program, checked against a
// double-precision loop on the host.
//
//   hipcc --offload-arch=gfx950 -O2 -Iinclude examples/c_abi_cdist.cpp \
//         -Lkermac_amd/_lib -lkermac_amd -Wl,-rpath,$PWD/kermac_amd/_lib -o c_abi_cdist
//   ./c_abi_cdist [M N K]
//
// (python -m kermac_amd._build builds it as kermac_amd/_lib/c_abi_cdist.)
// Exit status 0 = results within rtol 1e-5 of the host loop.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "kermac_amd.h"

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t status_ = (call);                                                          \
        if (status_ != hipSuccess) {                                                          \
            std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(status_));       \
            return 2;                                                                         \
        }                                                                                     \
    } while (0)

#define KMC_OK_OR_RETURN(call)                                                                \
    do {                                                                                      \
        int status_ = (call);                                                                 \
        if (status_ != KMC_OK) {                                                              \
            std::fprintf(stderr, "%s failed with status %d: %s\n", #call, status_, kmc_last_error()); \
            return 2;                                                                         \
        }                                                                                     \
    } while (0)

static float next_uniform(unsigned long long &state)
{
    state = state * 6364136223846793005ULL + 1442695040888963407ULL;
    return static_cast<float>((state >> 40) & 0xffffff) / 16777216.0f * 2.0f - 1.0f;
}

int main(int argc, char **argv)
{
    const int M = argc > 3 ? std::atoi(argv[1]) : 1000;
    const int N = argc > 3 ? std::atoi(argv[2]) : 700;
    const int K = argc > 3 ? std::atoi(argv[3]) : 96;
    std::printf("kermac_amd C ABI version %d, M=%d N=%d K=%d\n", kmc_abi_version(), M, N, K);

    // K-major panels: a_store[K][M], b_store[K][N], out_store[N][M].
    std::vector<float> a(static_cast<size_t>(K) * M), b(static_cast<size_t>(K) * N), out(static_cast<size_t>(N) * M);
    unsigned long long state = 12345;
    for (float &v : a) v = next_uniform(state);
    for (float &v : b) v = next_uniform(state);

    float *d_a = nullptr, *d_b = nullptr, *d_out = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_a), a.size() * sizeof(float)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_b), b.size() * sizeof(float)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_out), out.size() * sizeof(float)));
    HIP_OK(hipMemcpy(d_a, a.data(), a.size() * sizeof(float), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_b, b.data(), b.size() * sizeof(float), hipMemcpyHostToDevice));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    kmc_build_kernel_params params;
    std::memset(&params, 0, sizeof(params));
    params.inner_operator = KMC_OP_DIFF;
    params.inner_power = KMC_POW_ABS;
    params.outer_power = KMC_POW_NOOP;
    params.kernel_type = KMC_KERNEL_NONE;
    params.a_majorness = KMC_COL_MAJOR;   // m is the contiguous index of a_store
    params.b_majorness = KMC_COL_MAJOR;
    params.m = M; params.n = N; params.k = K; params.l = 1;
    params.a = d_a; params.a_ld = M;
    params.b = d_b; params.b_ld = N;
    params.c = d_out; params.c_ld = M;
    params.epsilon = 1e-5f;

    int failures = 0;
    for (int pass = 0; pass < 2; pass++) {
        const bool laplace = pass == 1;
        const float bandwidth = 0.25f * K;
        if (laplace) {
            params.kernel_type = KMC_KERNEL_LAPLACE;
            params.bandwidth_value = bandwidth;   // by value: the pointer stays NULL
        }
        hipEvent_t start, stop;
        HIP_OK(hipEventCreate(&start));
        HIP_OK(hipEventCreate(&stop));
        KMC_OK_OR_RETURN(kmc_build_kernel(&params, stream));   // warm-up
        HIP_OK(hipEventRecord(start, stream));
        KMC_OK_OR_RETURN(kmc_build_kernel(&params, stream));
        HIP_OK(hipEventRecord(stop, stream));
        HIP_OK(hipStreamSynchronize(stream));
        float ms = 0.0f;
        HIP_OK(hipEventElapsedTime(&ms, start, stop));
        HIP_OK(hipMemcpy(out.data(), d_out, out.size() * sizeof(float), hipMemcpyDeviceToHost));

        double worst = 0.0;
        for (int n = 0; n < N; n += 7)
            for (int m = 0; m < M; m += 3) {
                double truth = 0.0;
                for (int k = 0; k < K; k++)
                    truth += std::fabs(static_cast<double>(b[static_cast<size_t>(k) * N + n]) - a[static_cast<size_t>(k) * M + m]);
                if (laplace) truth = std::exp(-(truth < 1e-5 ? 0.0 : truth) / bandwidth);
                const double got = out[static_cast<size_t>(n) * M + m];
                const double rel = std::fabs(got - truth) / (std::fabs(truth) + 1e-300);
                if (rel > worst) worst = rel;
            }
        std::printf("%s: %.3f ms, max relative error on the sampled entries %.2e\n",
                    laplace ? "laplace kernel (bandwidth K/4)" : "L1 distance", ms, worst);
        if (!(worst <= 1e-5)) failures++;
    }

    // An invalid argument is reported through the status and kmc_last_error().
    params.inner_power = 99;
    const int status = kmc_build_kernel(&params, stream);
    std::printf("inner_power = 99 -> status %d (%s)\n", status, kmc_last_error());
    if (status != KMC_ERR_INVALID_ARGUMENT) failures++;

    HIP_OK(hipStreamDestroy(stream));
    HIP_OK(hipFree(d_a));
    HIP_OK(hipFree(d_b));
    HIP_OK(hipFree(d_out));
    std::printf(failures ? "FAILED\n" : "ok\n");
    return failures ? 1 : 0;
}
