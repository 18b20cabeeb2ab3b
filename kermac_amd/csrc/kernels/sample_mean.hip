// kmc_sample_mean: the mean point of (a sample of) the rows of an operand panel, the
// centre that the matrix-core kernels subtract from both operands while they stage them
// (|a|^2 + |b|^2 - 2 a.b cancels in proportion to the norms, and the norms that matter are
// those around the centre).  Up to 4096 rows are averaged exactly as given; of a longer panel
// 16 runs of 256 consecutive rows, evenly spaced from the first row to the last.  The sums run
// in a fixed order, so the same panel always gives the same centre.  The result is padded with
// zeros to a multiple of GRAM_CENTRE_PAD floats, as the kernels expect it, and followed by a
// flag: 1 when subtracting the centre is worth its cost, 0 when the centre is so close to the
// origin, measured against the spread of the sampled rows around it (|c|^2 <= spread^2 / 64), that
// the norms -- and with them the cancellation -- would change by less than 2 %.  The matrix-core
// kernels then skip the subtraction for that batch entry.  Layout per batch entry:
// [centre, padded][flag, 63 unused floats][variance per k, padded] = 2 * padded + 64 floats.
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

// mean of squares minus square of mean, per k, goes behind the centre and its flag
__device__ __forceinline__ float *variance_of(const SampleMeanArgs &args, int batch)
{
    return args.mean + batch * args.mean_bs + args.k_padded + GRAM_CENTRE_PAD;
}

constexpr int SM_MAX_SAMPLES = 4096;
constexpr int SM_RUN = 256;
constexpr int SM_RUNS = SM_MAX_SAMPLES / SM_RUN;

__device__ __forceinline__ i64 sampled_row(const SampleMeanArgs &args, int s)
{
    if (args.rows <= SM_MAX_SAMPLES) return s;
    const int run = s / SM_RUN;
    return (i64)run * (args.rows - SM_RUN) / (SM_RUNS - 1) + (s - run * SM_RUN);
}

// k contiguous (row-major panel): a workgroup owns 64 k, its 16 waves share the rows, and a wave
// has eight rows under way at once (eight sums per lane, added in a fixed order at the end): the
// panel's rows lie K floats apart, so the time is that of the loads' latency, not of their bytes.
constexpr int SM_ROW_WAVES = 16;
constexpr int SM_ROW_UNROLL = 8;

__global__ __launch_bounds__(64 * SM_ROW_WAVES) void sample_mean_rows(const SampleMeanArgs args)
{
    __shared__ float partial[SM_ROW_WAVES][64];
    __shared__ float partial_squares[SM_ROW_WAVES][64];
    const int kk = threadIdx.x & 63, group = threadIdx.x >> 6;
    const int k = blockIdx.x * 64 + kk;
    const float *x = args.x + blockIdx.y * args.bs;
    float sum[SM_ROW_UNROLL], squares[SM_ROW_UNROLL];
#pragma unroll
    for (int u = 0; u < SM_ROW_UNROLL; ++u) sum[u] = squares[u] = 0.0f;
    if (k < args.k) {
        int s = group;
        for (; s + (SM_ROW_UNROLL - 1) * SM_ROW_WAVES < args.samples; s += SM_ROW_UNROLL * SM_ROW_WAVES) {
            float v[SM_ROW_UNROLL];
#pragma unroll
            for (int u = 0; u < SM_ROW_UNROLL; ++u) v[u] = x[sampled_row(args, s + u * SM_ROW_WAVES) * args.ld + k];
#pragma unroll
            for (int u = 0; u < SM_ROW_UNROLL; ++u) {
                sum[u] += v[u];
                squares[u] += v[u] * v[u];
            }
        }
        for (; s < args.samples; s += SM_ROW_WAVES) {
            const float v = x[sampled_row(args, s) * args.ld + k];
            sum[0] += v;
            squares[0] += v * v;
        }
    }
    float mine = 0.0f, mine_squares = 0.0f;
#pragma unroll
    for (int u = 0; u < SM_ROW_UNROLL; ++u) {
        mine += sum[u];
        mine_squares += squares[u];
    }
    partial[group][kk] = mine;
    partial_squares[group][kk] = mine_squares;
    __syncthreads();
    if (group == 0 && k < args.k_padded) {
        float total = 0.0f, total_squares = 0.0f;
#pragma unroll
        for (int w = 0; w < SM_ROW_WAVES; ++w) {
            total += partial[w][kk];
            total_squares += partial_squares[w][kk];
        }
        const bool live = k < args.k && args.samples > 0;
        const float mean = live ? total / (float)args.samples : 0.0f;
        args.mean[blockIdx.y * args.mean_bs + k] = mean;
        variance_of(args, blockIdx.y)[k] = live ? fmaxf(total_squares / (float)args.samples - mean * mean, 0.0f) : 0.0f;
    }
}

// rows contiguous (K-major panel): a wave owns one k, its lanes take consecutive rows.
__global__ __launch_bounds__(256) void sample_mean_columns(const SampleMeanArgs args)
{
    __shared__ float partial[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int k = blockIdx.x * 4 + wave;
    const float *x = args.x + blockIdx.y * args.bs;
    __shared__ float partial_squares[4][64];
    float sum = 0.0f, squares = 0.0f;
    if (k < args.k) {
        // eight loads under way per lane, added in the order of the rows: the sampled rows of a long panel lie far apart,
        // and one load at a time made this launch 20 us of waiting (4096 rows: 64 round trips) where it now takes a few
        constexpr int IN_FLIGHT = 8;
        for (int first = lane; first < args.samples; first += 64 * IN_FLIGHT) {
            float v[IN_FLIGHT];
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; u++) {
                const int s = first + 64 * u;
                v[u] = s < args.samples ? x[(i64)k * args.ld + sampled_row(args, s)] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < IN_FLIGHT; u++)
                if (first + 64 * u < args.samples) {
                    sum += v[u];
                    squares += v[u] * v[u];
                }
        }
    }
    partial[wave][lane] = sum;
    partial_squares[wave][lane] = squares;
    __syncthreads();
    if (lane == 0 && k < args.k_padded) {
        float total = 0.0f, total_squares = 0.0f;
        for (int j = 0; j < 64; j++) {
            total += partial[wave][j];
            total_squares += partial_squares[wave][j];
        }
        const bool live = k < args.k && args.samples > 0;
        const float mean = live ? total / (float)args.samples : 0.0f;
        args.mean[blockIdx.y * args.mean_bs + k] = mean;
        variance_of(args, blockIdx.y)[k] = live ? fmaxf(total_squares / (float)args.samples - mean * mean, 0.0f) : 0.0f;
    }
}

// One workgroup per batch entry: |c|^2 against the summed variance, both added in a fixed order.
__global__ __launch_bounds__(256) void centre_flag(const SampleMeanArgs args)
{
    __shared__ float norms[256], spreads[256];
    const float *centre = args.mean + blockIdx.x * args.mean_bs;
    const float *variance = variance_of(args, blockIdx.x);
    float norm = 0.0f, spread = 0.0f;
    for (int k = threadIdx.x; k < args.k; k += 256) {
        norm += centre[k] * centre[k];
        spread += variance[k];
    }
    norms[threadIdx.x] = norm;
    spreads[threadIdx.x] = spread;
    __syncthreads();
    for (int width = 128; width > 0; width >>= 1) {
        if ((int)threadIdx.x < width) {
            norms[threadIdx.x] += norms[threadIdx.x + width];
            spreads[threadIdx.x] += spreads[threadIdx.x + width];
        }
        __syncthreads();
    }
    if (threadIdx.x < GRAM_CENTRE_PAD) {
        // not-a-number data: keep the subtraction (the comparison is false), the repair decides
        const bool needless = norms[0] <= spreads[0] * (1.0f / 64.0f);
        args.mean[blockIdx.x * args.mean_bs + args.k_padded + threadIdx.x] = (threadIdx.x == 0 && !needless) ? 1.0f : 0.0f;
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
    if (l > 1 && mean_bs < 2 * k_padded + kmc::GRAM_CENTRE_PAD)
        return fail(KMC_ERR_INVALID_ARGUMENT, "mean_bs = %lld is smaller than 2 * %d + %d", static_cast<long long>(mean_bs), k_padded,
                    kmc::GRAM_CENTRE_PAD);
    int status = kmc_host::require_gfx950();
    if (status != KMC_OK) return status;
    kmc::SampleMeanArgs args;
    args.x = x; args.ld = ld; args.bs = bs;
    args.rows = rows; args.k = k; args.k_padded = k_padded;
    args.mean = mean; args.mean_bs = mean_bs;
    args.samples = rows < kmc::SM_MAX_SAMPLES ? rows : kmc::SM_MAX_SAMPLES;
    hipError_t e;
    if (majorness == KMC_ROW_MAJOR)
        e = kmc_host::launch(kmc::sample_mean_rows, dim3(k_padded / 64, l), dim3(64 * kmc::SM_ROW_WAVES), static_cast<hipStream_t>(stream), args);
    else
        e = kmc_host::launch(kmc::sample_mean_columns, dim3(k_padded / 4, l), dim3(256), static_cast<hipStream_t>(stream), args);
    if (e != hipSuccess) return kmc_host::fail_hip(e, "sample_mean launch");
    e = kmc_host::launch(kmc::centre_flag, dim3(l), dim3(256), static_cast<hipStream_t>(stream), args);
    if (e != hipSuccess) return kmc_host::fail_hip(e, "centre_flag launch");
    return KMC_OK;
}
