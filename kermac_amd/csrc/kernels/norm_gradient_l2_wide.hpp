// The gradient of the L2 norm as one matrix product on the fp16 matrix instruction.
//
//   e[o][n][m] = sum_k c[o][k] a[k][m] (d[n][m] - b[n][k])
//              = (d[n][m] - s[n]) g[m][o] - sum_k p[o N + n][k] a[k][m],
//   g[m][o] = sum_k a[k][m] c[o][k],   p[o N + n][k] = c[o][k] (b[n][k] - s[n]),
//
// for any shift s[n]; with s[n] the mean of row n of b both terms are as small as the data allows
// (a common offset of d and b, which the difference d - b never sees, would otherwise be multiplied
// out and cancelled).  The second term is a product of an (O N) x K matrix with a K x M one: the
// rows of p and the columns of a are split into two fp16 pieces per value with a scale per row,
// exactly as the squared-difference route does it (gram_f16_wide.hpp), and the same kernel walks
// the pieces (GW_EPILOGUE_GRADIENT_L2: three piece products per 16 k); its epilogue fetches d and g
// and stores e.  Where the fp32 kernels build c a (d - b) value by value on the vector ALU and
// contract it on the fp32 matrix instruction, this route has no work per (o, n, m, k) outside the
// matrix instruction.  Error of the product from the pieces below 3 * 2^-22 sum_k |c a (b - s)|;
// g and the rest are fp32.
//
// This header: the kernels that prepare p, s and the transposed c (g itself comes from
// kmc_matrix_times_coefficients with a as the stored panel).
#pragma once

#include <hip/hip_runtime.h>

namespace kmc {

using i64 = long long;

struct GradientL2PrepareArgs {
    const float *b; i64 b_ld, b_bs;          // [n][k], k contiguous
    const float *c; i64 c_ld, c_bs;          // [o][k], k contiguous
    float *products; i64 products_ld, products_bs;   // [o n_rows + n][k]
    float *shift; i64 shift_bs;              // [n]
    float *c_transposed; i64 c_transposed_ld, c_transposed_bs;   // [k][o]
    int n, o, k;
};

constexpr int GL2_THREADS = 256;
constexpr int GL2_OUTPUTS = 4;       // rows of p per workgroup

// One workgroup per row n of b and four outputs: the mean of the row (sums in a fixed order, the
// same in every workgroup of the row), then the rows of p that belong to it.
__global__ __launch_bounds__(GL2_THREADS) void gradient_l2_products(const GradientL2PrepareArgs args)
{
    __shared__ float partial[GL2_THREADS];
    const int n = blockIdx.x, batch = blockIdx.z;
    const int o_begin = blockIdx.y * GL2_OUTPUTS;
    const int o_end = o_begin + GL2_OUTPUTS < args.o ? o_begin + GL2_OUTPUTS : args.o;
    const float *b_row = args.b + batch * args.b_bs + (i64)n * args.b_ld;
    float sum = 0.0f;
    for (int k = threadIdx.x; k < args.k; k += GL2_THREADS) sum += b_row[k];
    partial[threadIdx.x] = sum;
    __syncthreads();
    for (int width = GL2_THREADS / 2; width > 0; width >>= 1) {
        if ((int)threadIdx.x < width) partial[threadIdx.x] += partial[threadIdx.x + width];
        __syncthreads();
    }
    const float mean = partial[0] / (float)args.k;
    // not-a-number or infinite rows: no shift (the product then carries them as the fp32 kernels would)
    const float shift = (mean - mean == 0.0f) ? mean : 0.0f;
    if (threadIdx.x == 0 && blockIdx.y == 0) args.shift[batch * args.shift_bs + n] = shift;
    const float *c = args.c + batch * args.c_bs;
    float *products = args.products + batch * args.products_bs;
    for (int k = threadIdx.x; k < args.k; k += GL2_THREADS) {
        const float centred = b_row[k] - shift;
        for (int o = o_begin; o < o_end; ++o)
            products[((i64)o * args.n + n) * args.products_ld + k] = c[(i64)o * args.c_ld + k] * centred;
    }
}

// g = the sum of `parts` partial products, in their order (kmc_matrix_times_coefficients with n_splits)
struct GradientL2SumArgs {
    const float *partial;
    float *sum;
    i64 count, stride;
    int parts;
};

__global__ __launch_bounds__(GL2_THREADS) void gradient_l2_sum_parts(const GradientL2SumArgs args)
{
    const i64 at = (i64)blockIdx.x * GL2_THREADS + threadIdx.x;
    if (at >= args.count) return;
    float total = args.partial[at];
    for (int part = 1; part < args.parts; ++part) total += args.partial[part * args.stride + at];
    args.sum[at] = total;
}

// c_transposed[k][o] = c[o][k]
__global__ __launch_bounds__(GL2_THREADS) void gradient_l2_transpose_c(const GradientL2PrepareArgs args)
{
    const int k = blockIdx.x * GL2_THREADS + threadIdx.x, batch = blockIdx.y;
    if (k >= args.k) return;
    const float *c = args.c + batch * args.c_bs;
    float *row = args.c_transposed + batch * args.c_transposed_bs + (i64)k * args.c_transposed_ld;
    for (int o = 0; o < args.o; ++o) row[o] = c[(i64)o * args.c_ld + k];
}

}  // namespace kmc
