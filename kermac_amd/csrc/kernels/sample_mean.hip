// kmc_sample_mean: the mean point of (a sample of) the rows of an operand panel, the
// centre that the matrix-core kernels subtract from both operands while they stage them
// (|a|^2 + |b|^2 - 2 a.b cancels in proportion to the norms, and the norms that matter are
// those around the centre).  Up to 4096 rows are averaged exactly as given; of a longer panel
// 16 runs of 256 consecutive rows, evenly spaced from the first row to the last.  The sums run
// in a fixed order, so the same panel always gives the same centre.  The result is padded with
// zeros to a multiple of GRAM_CENTRE_PAD floats, as the kernels expect it.
#include <hip/hip_runtime.h>

#include "../host/host_common.hpp"
#include "build_kernel.hpp"
#include "launch.hpp"

namespace kmc {

struct SampleMeanArgs {
    const float *x; i64 ld, bs;
    int rows, k, k_padded;
    float *mean; i64 mean_bs;
    int samples;         // rows that are averaged
};

constexpr int SM_MAX_SAMPLES = 4096;
constexpr int SM_RUN = 256;
constexpr int SM_RUNS = SM_MAX_SAMPLES / SM_RUN;

__device__ __forceinline__ i64 sampled_row(const SampleMeanArgs &args, int s)
{
    if (args.rows <= SM_MAX_SAMPLES) return s;
    const int run = s / SM_RUN;
    return (i64)run * (args.rows - SM_RUN) / (SM_RUNS - 1) + (s - run * SM_RUN);
}

// k contiguous (row-major panel): a workgroup owns 64 k, four groups of lanes share the rows.
__global__ __launch_bounds__(256) void sample_mean_rows(const SampleMeanArgs args)
{
    __shared__ float partial[4][64];
    const int kk = threadIdx.x & 63, group = threadIdx.x >> 6;
    const int k = blockIdx.x * 64 + kk;
    const float *x = args.x + blockIdx.y * args.bs;
    float sum = 0.0f;
    if (k < args.k)
        for (int s = group; s < args.samples; s += 4) sum += x[sampled_row(args, s) * args.ld + k];
    partial[group][kk] = sum;
    __syncthreads();
    if (group == 0 && k < args.k_padded) {
        const float total = ((partial[0][kk] + partial[1][kk]) + partial[2][kk]) + partial[3][kk];
        args.mean[blockIdx.y * args.mean_bs + k] = (k < args.k && args.samples > 0) ? total / (float)args.samples : 0.0f;
    }
}

// rows contiguous (K-major panel): a wave owns one k, its lanes take consecutive rows.
__global__ __launch_bounds__(256) void sample_mean_columns(const SampleMeanArgs args)
{
    __shared__ float partial[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int k = blockIdx.x * 4 + wave;
    const float *x = args.x + blockIdx.y * args.bs;
    float sum = 0.0f;
    if (k < args.k)
        for (int s = lane; s < args.samples; s += 64) sum += x[(i64)k * args.ld + sampled_row(args, s)];
    partial[wave][lane] = sum;
    __syncthreads();
    if (lane == 0 && k < args.k_padded) {
        float total = 0.0f;
        for (int j = 0; j < 64; j++) total += partial[wave][j];
        args.mean[blockIdx.y * args.mean_bs + k] = (k < args.k && args.samples > 0) ? total / (float)args.samples : 0.0f;
    }
}

}  // namespace kmc

extern "C" int kmc_sample_mean(const float *x, int32_t majorness, int32_t rows, int32_t k, int64_t ld, int64_t bs, int32_t l,
                               float *mean, int64_t mean_bs, void *stream)
{
    using kmc_host::fail;
    if (majorness != KMC_COL_MAJOR && majorness != KMC_ROW_MAJOR)
        return fail(KMC_ERR_INVALID_ARGUMENT, "majorness %d is not a kmc_majorness", majorness);
    if (rows < 0 || k < 0 || l < 0 || ld < 0 || bs < 0 || mean_bs < 0)
        return fail(KMC_ERR_INVALID_ARGUMENT, "negative extent or stride");
    if (l > 65535) return fail(KMC_ERR_INVALID_ARGUMENT, "batch count %d exceeds 65535", l);
    const int k_padded = (k + kmc::GRAM_CENTRE_PAD - 1) / kmc::GRAM_CENTRE_PAD * kmc::GRAM_CENTRE_PAD;
    if (k == 0 || l == 0) return KMC_OK;
    if (!mean || (rows > 0 && !x)) return fail(KMC_ERR_INVALID_ARGUMENT, "null pointer");
    if (l > 1 && mean_bs < k_padded)
        return fail(KMC_ERR_INVALID_ARGUMENT, "mean_bs = %lld is smaller than k padded to %d", static_cast<long long>(mean_bs), k_padded);
    int status = kmc_host::require_gfx950();
    if (status != KMC_OK) return status;
    kmc::SampleMeanArgs args;
    args.x = x; args.ld = ld; args.bs = bs;
    args.rows = rows; args.k = k; args.k_padded = k_padded;
    args.mean = mean; args.mean_bs = mean_bs;
    args.samples = rows < kmc::SM_MAX_SAMPLES ? rows : kmc::SM_MAX_SAMPLES;
    hipError_t e;
    if (majorness == KMC_ROW_MAJOR)
        e = kmc_host::launch(kmc::sample_mean_rows, dim3(k_padded / 64, l), dim3(256), static_cast<hipStream_t>(stream), args);
    else
        e = kmc_host::launch(kmc::sample_mean_columns, dim3(k_padded / 4, l), dim3(256), static_cast<hipStream_t>(stream), args);
    if (e != hipSuccess) return kmc_host::fail_hip(e, "sample_mean launch");
    return KMC_OK;
}
