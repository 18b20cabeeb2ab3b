// Second step of a contraction that was cut over k: the partial sums of the slices
// are added in slice order and the result goes through the epilogue of the fused
// pairwise-reduction kernel (outer power, epsilon mask, kernel function, regularised
// diagonal: include/build_a_kernel.cuh:374-447 of the reference).  Element-wise, one
// lane per four consecutive m.
#include <hip/hip_runtime.h>

#include "build_kernel.hpp"

namespace kmc {

struct FinishArgs {
    BuildKernelArgs kernel;     // m, n, l, c / c_ld / c_bs, epilogue parameters
    const float *partials;      // (slice, batch, n, m), m contiguous
    i64 partial_ld, partial_bs, partial_slice;
    int slices;
    int vec;                    // partials and c allow 128-bit access
};

__global__ __launch_bounds__(256) void finish_partials(const FinishArgs fa)
{
    const BuildKernelArgs &args = fa.kernel;
    const int batch = blockIdx.z;
    const int n = blockIdx.y;
    const int m = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (m >= args.m) return;
    const int valid = min(4, args.m - m);

    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const float *src = fa.partials + batch * fa.partial_bs + (i64)n * fa.partial_ld + m;
    // Eight loads in flight, added in slice order (the order of the sum is fixed).
    int s = 0;
    for (; s + 8 <= fa.slices; s += 8) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = load4_guarded(src + (s + u) * fa.partial_slice, valid, fa.vec);
#pragma unroll
        for (int u = 0; u < 8; u++) {
            sum[0] += v[u].x; sum[1] += v[u].y; sum[2] += v[u].z; sum[3] += v[u].w;
        }
    }
    for (; s < fa.slices; s++) {
        const float4 v = load4_guarded(src + s * fa.partial_slice, valid, fa.vec);
        sum[0] += v.x; sum[1] += v.y; sum[2] += v.z; sum[3] += v.w;
    }

    const int outer_power = args.outer_power;
    const int kernel_type = args.kernel_type;
    float p_outer = 0.0f, neg_gamma = 0.0f, regularization = 0.0f;
    if (outer_power == POW_POW) p_outer = args.p_outer ? args.p_outer[batch * args.p_outer_bs] : args.p_outer_value;
    if (kernel_type != KERNEL_NONE) {
        const float bw = args.bandwidth ? args.bandwidth[batch * args.bandwidth_bs] : args.bandwidth_value;
        neg_gamma = kernel_neg_gamma(kernel_type, bw);
        regularization = args.regularization ? args.regularization[batch * args.regularization_bs]
                                             : args.regularization_value;
    }
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
    const dim3 grid((kernel.m + 1023) / 1024, kernel.n, kernel.l);
    hipLaunchKernelGGL(kmc::finish_partials, grid, dim3(256), 0, stream, fa);
    return hipGetLastError();
}

}  // namespace kmc_host
