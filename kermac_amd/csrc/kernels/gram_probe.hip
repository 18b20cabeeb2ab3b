// The sample of the result that is taken in front of a matrix-core launch for squared differences.
//
// |a|^2 + |b|^2 - 2 a.b cancels for pairs of near-duplicate points; a 128 x 128 part of the result that holds
// such a pair is stamped by the matrix-core kernel and recomputed by the direct kernel behind it.  Data that
// has such pairs in every part (points drawn around a few centres, in any order) would pay for both kernels.
// This kernel looks first, at the operands as the caller holds them: BK_SAMPLE_TILES tiles of the result over
// the batch, 16 consecutive rows of each operand from each, their 256 pairs over up to 128 of the k (8 runs of
// 16 spread over the contraction), judged by the matrix-core kernels' own criterion on those k -- near-duplicates
// fail it on any subset of k.  A workgroup owns one sampled tile and one word of the result, which it writes
// whole: nothing is accumulated across workgroups, so nothing has to be cleared and the order of the workgroups
// does not matter.  build_kernel.hpp's sample_leaves_it_to_the_direct_kernel turns the words into the decision,
// inside the matrix-core kernels.  The reference has no counterpart (it has no matrix-core path).
#include <hip/hip_runtime.h>

#include "../host/host_common.hpp"
#include "../host/dispatch_rules.hpp"
#include "build_kernel.hpp"
#include "launch.hpp"

static_assert(kmc::BK_SAMPLE_TILES == kmc_rules::SAMPLE_TILES && kmc::BK_SAMPLE_LEAVE_PER_16384 == kmc_rules::SAMPLE_LEAVE_PER_16384 &&
                  kmc::BK_SAMPLE_BYTES == KMC_SAMPLE_BYTES,
              "the table of dispatch rules, the header and the kernels' constants must say the same");

namespace kmc {

constexpr int GP_RUNS = 8;                     // runs of 16 consecutive k
constexpr int GP_K = GP_RUNS * BK_TILE_K;      // k per pair
constexpr int GP_THREADS = BK_SAMPLE_ROWS * BK_SAMPLE_ROWS;

struct GramProbeArgs {
    const float *a, *b;
    i64 a_ld, a_bs, b_ld, b_bs;
    int a_k_contiguous, b_k_contiguous;
    int m, n, k, l;
    const float *centre; i64 centre_bs;        // as in BuildKernelArgs; the flag sits behind the padded centre
    float trust;
    unsigned *sample;                          // [BK_SAMPLE_TILES]
};

__device__ __forceinline__ float probe_element(const float *x, i64 ld, int k_contiguous, int row, int k)
{
    return k_contiguous ? x[(i64)row * ld + k] : x[(i64)k * ld + row];
}

__global__ __launch_bounds__(GP_THREADS) void gram_probe_operands(const GramProbeArgs args)
{
    __shared__ float rows_a[GP_K][BK_SAMPLE_ROWS + 1];      // + 1: no bank is hit twice whichever way the rows are loaded
    __shared__ float rows_b[GP_K][BK_SAMPLE_ROWS + 1];
    __shared__ unsigned below_in_tile;
    const int t = threadIdx.x;
    if (t == 0) below_in_tile = 0u;
    unsigned h = (unsigned)blockIdx.x * 2654435761u + 0x9e3779b9u;
    h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 13;
    const int batch = (int)(h % (unsigned)args.l);
    h = h * 0x7feb352du + 0x1234567u; h ^= h >> 16;
    const int m0 = (int)(h % (unsigned)((args.m + BK_TILE_M - 1) / BK_TILE_M)) * BK_TILE_M + (int)((h >> 20) & 7u) * BK_SAMPLE_ROWS;
    h = h * 0x7feb352du + 0x1234567u; h ^= h >> 16;
    const int n0 = (int)(h % (unsigned)((args.n + BK_TILE_N - 1) / BK_TILE_N)) * BK_TILE_N + (int)((h >> 20) & 7u) * BK_SAMPLE_ROWS;

    const float *a = args.a + batch * args.a_bs, *b = args.b + batch * args.b_bs;
    const int k_padded = (args.k + GRAM_CENTRE_PAD - 1) / GRAM_CENTRE_PAD * GRAM_CENTRE_PAD;
    const float *centre = args.centre ? args.centre + batch * args.centre_bs : nullptr;
    if (centre && centre[k_padded] == 0.0f) centre = nullptr;        // the flag: this batch entry is taken as it is

    // Lane t fetches, for each run, one value of a and one of b: 16 rows x 16 k per run, along whichever
    // direction is contiguous.  Rows beyond the panel repeat its last row (a pair counted twice biases nothing
    // that matters here); k beyond the contraction contributes nothing.
    const int slices = (args.k + BK_TILE_K - 1) / BK_TILE_K;
    const int runs = slices < GP_RUNS ? slices : GP_RUNS;
    const int row_a = args.a_k_contiguous ? t / BK_TILE_K : t % BK_SAMPLE_ROWS, k_a = args.a_k_contiguous ? t % BK_TILE_K : t / BK_SAMPLE_ROWS;
    const int row_b = args.b_k_contiguous ? t / BK_TILE_K : t % BK_SAMPLE_ROWS, k_b = args.b_k_contiguous ? t % BK_TILE_K : t / BK_SAMPLE_ROWS;
    const int m = min(m0 + row_a, args.m - 1), n = min(n0 + row_b, args.n - 1);
    float va[GP_RUNS], vb[GP_RUNS];
#pragma unroll
    for (int r = 0; r < GP_RUNS; r++) {
        const int first = (int)((i64)r * slices / runs) * BK_TILE_K;
        const int ka = first + k_a, kb = first + k_b;
        const bool exists = r < runs;
        va[r] = exists && ka < args.k ? probe_element(a, args.a_ld, args.a_k_contiguous, m, ka) - (centre ? centre[ka] : 0.0f) : 0.0f;
        vb[r] = exists && kb < args.k ? probe_element(b, args.b_ld, args.b_k_contiguous, n, kb) - (centre ? centre[kb] : 0.0f) : 0.0f;
    }
#pragma unroll
    for (int r = 0; r < GP_RUNS; r++) {
        rows_a[r * BK_TILE_K + k_a][row_a] = va[r];
        rows_b[r * BK_TILE_K + k_b][row_b] = vb[r];
    }
    __syncthreads();
    const int i = t % BK_SAMPLE_ROWS, j = t / BK_SAMPLE_ROWS;      // this lane's pair: row i of a, row j of b
    float d2 = 0.0f, norms = 0.0f;
#pragma unroll 8
    for (int q = 0; q < GP_K; q++) {
        const float x = rows_a[q][i], y = rows_b[q][j];
        d2 += (y - x) * (y - x);
        norms += x * x + y * y;
    }
    if (!(d2 >= args.trust * norms)) atomicAdd(&below_in_tile, 1u);
    __syncthreads();
    if (t == 0) args.sample[blockIdx.x] = below_in_tile | (below_in_tile > 0u ? 0x10000u : 0u);
}

}  // namespace kmc

namespace kmc_host {

// Fills sample[0 .. BK_SAMPLE_TILES) for the problem of `p` (squared differences; m, n, k, l at least 1).
hipError_t launch_gram_probe(const kmc_build_kernel_params *p, const kmc::BuildKernelArgs &args, unsigned *sample, hipStream_t stream)
{
    kmc::GramProbeArgs probe;
    probe.a = p->a; probe.b = p->b;
    probe.a_ld = p->a_ld; probe.a_bs = p->a_bs; probe.b_ld = p->b_ld; probe.b_bs = p->b_bs;
    probe.a_k_contiguous = p->a_majorness == KMC_COL_MAJOR ? 0 : 1;
    probe.b_k_contiguous = p->b_majorness == KMC_COL_MAJOR ? 0 : 1;
    probe.m = args.m; probe.n = args.n; probe.k = args.k; probe.l = args.l;
    probe.centre = args.centre; probe.centre_bs = args.centre_bs;
    probe.trust = args.gram_trust;
    probe.sample = sample;
    return launch(kmc::gram_probe_operands, dim3(kmc::BK_SAMPLE_TILES), dim3(kmc::GP_THREADS), stream, probe);
}

}  // namespace kmc_host
