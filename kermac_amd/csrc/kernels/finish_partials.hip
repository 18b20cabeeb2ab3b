// Second step of a contraction that was cut over k: the partial sums of the slices
// are added in slice order and the result goes through the epilogue of the fused
// pairwise-reduction kernel (outer power, epsilon mask, kernel function, regularised
// diagonal: include/build_a_kernel.cuh:374-447 of the reference).  Element-wise, one
// lane per four consecutive m; where one row of the result has fewer than 128 such
// lanes, the lanes of a workgroup also divide the slices among themselves (lane group g
// adds slices g, g + G, g + 2 G, ... in that order, then group 0 adds the groups' sums in
// group order: a fixed order for a given shape, so results repeat bit for bit).
#include <hip/hip_runtime.h>

#include "launch.hpp"
#include "build_kernel.hpp"

namespace kmc {

struct FinishArgs {
    BuildKernelArgs kernel;     // m, n, l, c / c_ld / c_bs, epilogue parameters
    const float *partials;      // (slice, batch, n, m), m contiguous
    i64 partial_ld, partial_bs, partial_slice;
    int slices;
    int vec;                    // partials and c allow 128-bit access
    int quad_lanes;             // lanes along m per workgroup: 256 / groups, a power of two
    int groups;                 // lane groups that share the slices of one quad of m
};

// One row n of the result for this workgroup's lanes.
__device__ __forceinline__ void finish_row(const FinishArgs &fa, float4 *group_sums, int batch, int n, float p_outer,
                                           float neg_gamma, float regularization)
{
    const BuildKernelArgs &args = fa.kernel;
    const int quad = threadIdx.x & (fa.quad_lanes - 1);
    const int group = threadIdx.x / fa.quad_lanes;
    const int m = (blockIdx.x * fa.quad_lanes + quad) * 4;
    const bool live = m < args.m;
    const int valid = live ? min(4, args.m - m) : 0;

    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const float *src = fa.partials + batch * fa.partial_bs + (i64)n * fa.partial_ld + m;
    if (live) {
        // Eight loads in flight, added in slice order (the order of the sum is fixed).
        const i64 step = fa.groups * fa.partial_slice;
        const float *at = src + group * fa.partial_slice;
        const int mine = (fa.slices - group + fa.groups - 1) / fa.groups;   // slices group, group + G, ...
        int s = 0;
        for (; s + 8 <= mine; s += 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = load4_guarded(at + (s + u) * step, valid, fa.vec);
#pragma unroll
            for (int u = 0; u < 8; u++) {
                sum[0] += v[u].x; sum[1] += v[u].y; sum[2] += v[u].z; sum[3] += v[u].w;
            }
        }
        for (; s < mine; s++) {
            const float4 v = load4_guarded(at + s * step, valid, fa.vec);
            sum[0] += v.x; sum[1] += v.y; sum[2] += v.z; sum[3] += v.w;
        }
    }
    if (fa.groups > 1) {   // uniform over the launch
        group_sums[threadIdx.x] = make_float4(sum[0], sum[1], sum[2], sum[3]);
        __syncthreads();
        if (group == 0) {
            for (int g = 1; g < fa.groups; g++) {
                const float4 v = group_sums[g * fa.quad_lanes + quad];
                sum[0] += v.x; sum[1] += v.y; sum[2] += v.z; sum[3] += v.w;
            }
        }
        __syncthreads();   // the next row of this workgroup writes group_sums again
    }
    if (!live || group != 0) return;

    const int outer_power = args.outer_power;
    const int kernel_type = args.kernel_type;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        sum[i] = epilogue_value(sum[i], outer_power, kernel_type, p_outer, neg_gamma, args.epsilon);
        if (kernel_type != KERNEL_NONE && regularization != 0.0f && args.reg_off_x + m + i == args.reg_off_y + n)
            sum[i] = 1.0f + regularization;
    }

    float *dst = args.c + batch * args.c_bs + (i64)n * args.c_ld + m;
    if (fa.vec && valid == 4) {
        *reinterpret_cast<float4 *>(dst) = make_float4(sum[0], sum[1], sum[2], sum[3]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (i < valid) dst[i] = sum[i];
    }
}

// Grid: x = blocks of lanes along m, y = rows n (a workgroup strides over n by the grid
// height, so n may exceed the 65535 a grid dimension can hold), z = batch.
__global__ __launch_bounds__(256) void finish_partials(const FinishArgs fa)
{
    const BuildKernelArgs &args = fa.kernel;
    __shared__ float4 group_sums[256];
    const int batch = blockIdx.z;
    float p_outer = 0.0f, neg_gamma = 0.0f, regularization = 0.0f;
    if (args.outer_power == POW_POW) p_outer = args.p_outer ? args.p_outer[batch * args.p_outer_bs] : args.p_outer_value;
    if (args.kernel_type != KERNEL_NONE) {
        const float bw = args.bandwidth ? args.bandwidth[batch * args.bandwidth_bs] : args.bandwidth_value;
        neg_gamma = kernel_neg_gamma(args.kernel_type, bw);
        regularization = args.regularization ? args.regularization[batch * args.regularization_bs]
                                             : args.regularization_value;
    }
    for (int n = blockIdx.y; n < args.n; n += gridDim.y) finish_row(fa, group_sums, batch, n, p_outer, neg_gamma, regularization);
}

}  // namespace kmc

namespace kmc_host {

hipError_t launch_finish_partials(const kmc::BuildKernelArgs &kernel, const float *partials, int64_t partial_ld,
                                  int64_t partial_bs, int64_t partial_slice, int slices, int vec, hipStream_t stream)
{
    kmc::FinishArgs fa;
    fa.kernel = kernel;
    fa.partials = partials;
    fa.partial_ld = partial_ld; fa.partial_bs = partial_bs; fa.partial_slice = partial_slice;
    fa.slices = slices;
    fa.vec = vec;
    // A row of fewer than 128 quads of m leaves lanes for sharing the slices (at least 8 each).
    const int quads = (kernel.m + 3) / 4;
    fa.quad_lanes = 256;
    while (fa.quad_lanes > 1 && fa.quad_lanes / 2 >= quads && slices >= 8 * (512 / fa.quad_lanes)) fa.quad_lanes /= 2;
    fa.groups = 256 / fa.quad_lanes;
    const dim3 grid((quads + fa.quad_lanes - 1) / fa.quad_lanes, kernel.n < 65535 ? kernel.n : 65535, kernel.l);
    return launch(kmc::finish_partials, grid, dim3(256), stream, fa);
}

}  // namespace kmc_host
