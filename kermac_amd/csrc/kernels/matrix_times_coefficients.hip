// kmc_matrix_times_coefficients: a stored panel of the kernel matrix times coefficients,
//   out[m, o] (+)= sum_n matrix[n, m] * coef[n, o],
// the second half of the kernel-matrix x coefficients product when the matrix is built in
// panels of centres by kmc_build_kernel (the matrix-core routes for squared differences build
// a panel several times faster than the fused kernel walks it, so large products go: panel,
// contraction, next panel).  The panel is read once, near the rate memory delivers it.
//
// Both kernels multiply with v_mfma_f32_32x32x2_f32 (fp32 operands, fp32 sums): the instruction
// wants, per lane, matrix[n + lane / 32][m + lane % 32] and coef[n + lane / 32][o + lane % 32],
// which is what a plain vector load of each delivers, so nothing is staged in LDS.  One
// instruction covers 256 bytes of the panel in 64 cycles of a SIMD's matrix pipeline (the vector
// ALU would need 128 cycles for the same 32 multiply-adds per value, and was measured at
// 2.3 TB/s).  The waves of a workgroup share its n, and their partial sums are added in wave
// order, so the result does not depend on timing; the caller may cut the n further, into ranges
// with partial products of their own, when the rows m alone do not make a workgroup per CU.
//
// matrix_times_coefficients: any alignment.  A workgroup owns 32 rows m and 32 coefficient
// columns, a half wave reads 128 contiguous bytes of a row; sums in two levels (128 n in the
// accumulator of the instruction, then fp32 totals).
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../host/host_common.hpp"
#include "launch.hpp"

namespace kmc {

using i64 = long long;
using mc_floatx16 = __attribute__((__vector_size__(16 * sizeof(float)))) float;

constexpr int MC_WAVES = 4;
constexpr int MC_THREADS = 64 * MC_WAVES;
constexpr int MC_ROWS = 32;          // rows m per workgroup
constexpr int MC_COLUMNS = 32;       // coefficient columns per workgroup
constexpr int MC_GROUP = 8;          // matrix instructions per group of loads: 16 n
constexpr int MC_LEVEL = 8;          // groups per first-level sum: 128 n

struct MatrixCoefArgs {
    const float *matrix; i64 matrix_ld, matrix_bs;
    const float *coef; i64 coef_ld, coef_bs;
    float *out; i64 out_ld, out_bs;
    int m, n, o;
    int accumulate;
    int splits; i64 out_split_stride;      // the n in `splits` ranges, each with a partial product of its own
};

// The rows n of split `split`, in whole groups of `group` except at the end of the panel.
__device__ __forceinline__ void rows_of_split(const MatrixCoefArgs &args, int split, int group, int *begin, int *end)
{
    const int per_split = (args.n + args.splits * group - 1) / (args.splits * group) * group;
    *begin = split * per_split < args.n ? split * per_split : args.n;
    *end = *begin + per_split < args.n ? *begin + per_split : args.n;
}

__global__ __launch_bounds__(MC_THREADS) void matrix_times_coefficients(const MatrixCoefArgs args)
{
    __shared__ float partial[MC_WAVES - 1][16][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = lane >> 5, column = lane & 31;
    const int batch = blockIdx.z / args.splits, split = blockIdx.z % args.splits;
    const int o0 = blockIdx.y * MC_COLUMNS, m0 = blockIdx.x * MC_ROWS;
    // lanes beyond the last row or column read the last one (a valid address); a column that
    // does not exist contributes zeros, a row that does not exist is not stored
    const int m = m0 + column, o = o0 + column;
    const float column_exists = o < args.o ? 1.0f : 0.0f;
    const float *matrix = args.matrix + batch * args.matrix_bs + (m < args.m ? m : args.m - 1);
    const float *coef = args.coef + batch * args.coef_bs + (o < args.o ? o : args.o - 1);

    constexpr int GROUP_N = 2 * MC_GROUP;
    int first, last;
    rows_of_split(args, split, GROUP_N, &first, &last);
    const int per_wave = (last - first + MC_WAVES * GROUP_N - 1) / (MC_WAVES * GROUP_N) * GROUP_N;
    const int begin = first + wave * per_wave < last ? first + wave * per_wave : last;
    const int end = begin + per_wave < last ? begin + per_wave : last;

    mc_floatx16 total = {0}, sum = {0};
    int n = begin;
    int level = 0;
    for (; n + GROUP_N <= end; n += GROUP_N) {
        float from_matrix[MC_GROUP], from_coef[MC_GROUP];
#pragma unroll
        for (int u = 0; u < MC_GROUP; ++u) {
            const i64 row = n + 2 * u + half;
            from_matrix[u] = matrix[row * args.matrix_ld];
            from_coef[u] = coef[row * args.coef_ld] * column_exists;
        }
#pragma unroll
        for (int u = 0; u < MC_GROUP; ++u)
            sum = __builtin_amdgcn_mfma_f32_32x32x2f32(from_coef[u], from_matrix[u], sum, 0, 0, 0);
        if (++level == MC_LEVEL) {
            total += sum;
            sum = mc_floatx16{0};
            level = 0;
        }
    }
    if (n < end) {
        // the last rows of the range: rows beyond its end read the last row and count as zeros
#pragma unroll
        for (int u = 0; u < MC_GROUP; ++u) {
            const int row = n + 2 * u + half;
            const i64 read = row < end ? row : end - 1;
            const float of_coef = row < end ? coef[read * args.coef_ld] * column_exists : 0.0f;
            const float of_matrix = row < end ? matrix[read * args.matrix_ld] : 0.0f;
            sum = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, of_matrix, sum, 0, 0, 0);
        }
    }
    total += sum;

    // register r of lane (half, column) holds column o0 + 8 * (r / 4) + 4 * half + r % 4 of row m
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) partial[wave - 1][r][lane] = total[r];
    }
    __syncthreads();
    if (wave > 0 || m >= args.m) return;
    float *out = args.out + split * args.out_split_stride + batch * args.out_bs + m * args.out_ld + o0;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        float value = total[r];
#pragma unroll
        for (int w = 0; w < MC_WAVES - 1; ++w) value += partial[w][r][lane];
        const int at = 8 * (r / 4) + 4 * half + r % 4;
        if (o0 + at < args.o) out[at] = args.accumulate ? out[at] + value : value;
    }
}

// The same product for panels whose rows can be read 16 bytes per lane (matrix, matrix_ld and
// matrix_bs multiples of 4 floats): a lane reads matrix[n + lane / 32][m + 4 * (lane % 32) .. + 3], a
// half wave 512 contiguous bytes, and the four components feed four matrix instructions that
// share the coefficient operand, so a wave owns 128 rows m (instruction c holds rows m + 4 j + c in
// its columns j).  WAVES_M waves sit side by side in m and walk the same n together; WAVES_N such
// teams share the n of the workgroup and pass their partial sums to the first through LDS, in
// order.  A wave issues the loads of a group of rows before the matrix instructions of the group
// before it, so that it always has loads under way: 1 GB panels are read at 4.8 - 5.3 TB/s (3.5 - 4.0
// without that; reads of 128 bytes per row, as the kernel above issues them, reach 1.8).
constexpr int MC4_WAVE_ROWS = 128;
constexpr int MC4_GROUP = 4;         // loads of 16 bytes per group: 8 n, 16 matrix instructions

template <int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void matrix_times_coefficients_rows4(const MatrixCoefArgs args)
{
    __shared__ float passed[WAVES_M][64][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_m = wave % WAVES_M, wave_n = wave / WAVES_M;
    const int half = lane >> 5, column = lane & 31;
    const int batch = blockIdx.z / args.splits, split = blockIdx.z % args.splits;
    const int o0 = blockIdx.y * MC_COLUMNS, m0 = (blockIdx.x * WAVES_M + wave_m) * MC4_WAVE_ROWS;
    const int o = o0 + column;
    const float column_exists = o < args.o ? 1.0f : 0.0f;
    // a lane whose four rows lie beyond the last reads the last four of the padded row
    const int m_last = (args.m + 3) / 4 * 4 - 4;
    const int m = m0 + 4 * column;
    const float *matrix = args.matrix + batch * args.matrix_bs + (m < m_last ? m : m_last);
    const float *coef = args.coef + batch * args.coef_bs + (o < args.o ? o : args.o - 1);

    constexpr int GROUP_N = 2 * MC4_GROUP;
    int first, last;
    rows_of_split(args, split, GROUP_N, &first, &last);
    const int per_wave = (last - first + WAVES_N * GROUP_N - 1) / (WAVES_N * GROUP_N) * GROUP_N;
    const int begin = first + wave_n * per_wave < last ? first + wave_n * per_wave : last;
    const int end = begin + per_wave < last ? begin + per_wave : last;

    mc_floatx16 sum[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) sum[c] = mc_floatx16{0};
    float4 from_matrix[2][MC4_GROUP];
    float from_coef[2][MC4_GROUP];
    auto load = [&](auto buffer, int at) {
#pragma unroll
        for (int u = 0; u < MC4_GROUP; ++u) {
            const i64 row = at + 2 * u + half;
            from_matrix[buffer][u] = *reinterpret_cast<const float4 *>(matrix + row * args.matrix_ld);
            from_coef[buffer][u] = coef[row * args.coef_ld];
        }
    };
    auto multiply = [&](auto buffer) {
#pragma unroll
        for (int u = 0; u < MC4_GROUP; ++u) {
            const float of_coef = from_coef[buffer][u] * column_exists;
            sum[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, from_matrix[buffer][u].x, sum[0], 0, 0, 0);
            sum[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, from_matrix[buffer][u].y, sum[1], 0, 0, 0);
            sum[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, from_matrix[buffer][u].z, sum[2], 0, 0, 0);
            sum[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, from_matrix[buffer][u].w, sum[3], 0, 0, 0);
        }
    };
    // the loads of a group are issued before the matrix instructions of the group before it
    using Zero = std::integral_constant<int, 0>;
    using One = std::integral_constant<int, 1>;
    int n = begin;
    const int groups = (end - begin) / GROUP_N;
    if (groups > 0) load(Zero{}, n);
    int g = 0;
    for (; g + 2 <= groups; g += 2) {
        load(One{}, n + GROUP_N);
        multiply(Zero{});
        if (g + 2 < groups) load(Zero{}, n + 2 * GROUP_N);
        multiply(One{});
        n += 2 * GROUP_N;
    }
    if (g < groups) {
        multiply(Zero{});
        n += GROUP_N;
    }
    if (n < end) {
#pragma unroll
        for (int u = 0; u < MC4_GROUP; ++u) {
            const int row = n + 2 * u + half;
            const i64 read = row < end ? row : end - 1;
            const float of_coef = row < end ? coef[read * args.coef_ld] * column_exists : 0.0f;
            float4 of_matrix = *reinterpret_cast<const float4 *>(matrix + read * args.matrix_ld);
            if (row >= end) of_matrix = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            sum[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, of_matrix.x, sum[0], 0, 0, 0);
            sum[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, of_matrix.y, sum[1], 0, 0, 0);
            sum[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, of_matrix.z, sum[2], 0, 0, 0);
            sum[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(of_coef, of_matrix.w, sum[3], 0, 0, 0);
        }
    }

    // the partial sums of teams 1 .. WAVES_N - 1 reach team 0 one after the other
    for (int team = 1; team < WAVES_N; ++team) {
        if (wave_n == team) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int r = 0; r < 16; ++r) passed[wave_m][c * 16 + r][lane] = sum[c][r];
        }
        __syncthreads();
        if (wave_n == 0) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int r = 0; r < 16; ++r) sum[c][r] += passed[wave_m][c * 16 + r][lane];
        }
        __syncthreads();
    }
    if (wave_n > 0) return;
    // register r of instruction c holds column o0 + 8 * (r / 4) + 4 * half + r % 4 of row m + c
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        if (m + c >= args.m) continue;
        float *out = args.out + split * args.out_split_stride + batch * args.out_bs + (m + c) * args.out_ld + o0;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int at = 8 * (r / 4) + 4 * half + r % 4;
            if (o0 + at < args.o) out[at] = args.accumulate ? out[at] + sum[c][r] : sum[c][r];
        }
    }
}

}  // namespace kmc

extern "C" int kmc_matrix_times_coefficients(const kmc_matrix_coefficients_params *p, void *stream_handle)
{
    using kmc_host::fail;
    kmc_host::clear_error();
    if (!p) return fail(KMC_ERR_INVALID_ARGUMENT, "null parameter block");
    if (p->m < 0 || p->n < 0 || p->o < 0 || p->l < 0) return fail(KMC_ERR_INVALID_ARGUMENT, "negative extent");
    if (p->matrix_ld < 0 || p->matrix_bs < 0 || p->coef_ld < 0 || p->coef_bs < 0 || p->out_ld < 0 || p->out_bs < 0)
        return fail(KMC_ERR_INVALID_ARGUMENT, "negative stride");
    if (p->l > 65535) return fail(KMC_ERR_INVALID_ARGUMENT, "batch count %d exceeds 65535", p->l);
    if (p->n_splits < 0 || p->out_split_stride < 0 || static_cast<int64_t>(p->l) * (p->n_splits > 1 ? p->n_splits : 1) > 65535)
        return fail(KMC_ERR_INVALID_ARGUMENT, "n_splits = %d, l = %d: negative, or l * n_splits exceeds 65535", p->n_splits, p->l);
    if (p->o > 65535 * kmc::MC_COLUMNS) return fail(KMC_ERR_INVALID_ARGUMENT, "o = %d exceeds %d", p->o, 65535 * kmc::MC_COLUMNS);
    if (p->m == 0 || p->o == 0 || p->l == 0) return KMC_OK;
    if (!p->out || (p->n > 0 && (!p->matrix || !p->coef))) return fail(KMC_ERR_INVALID_ARGUMENT, "null pointer");
    if (p->n > 0 && (p->matrix_ld < p->m || p->coef_ld < p->o)) return fail(KMC_ERR_INVALID_ARGUMENT, "leading dimension below the row length");
    if (p->out_ld < p->o) return fail(KMC_ERR_INVALID_ARGUMENT, "out_ld = %lld is below o = %d", static_cast<long long>(p->out_ld), p->o);
    const int status = kmc_host::require_gfx950();
    if (status != KMC_OK) return status;

    kmc::MatrixCoefArgs args;
    args.matrix = p->matrix; args.matrix_ld = p->matrix_ld; args.matrix_bs = p->matrix_bs;
    args.coef = p->coef; args.coef_ld = p->coef_ld; args.coef_bs = p->coef_bs;
    args.out = p->out; args.out_ld = p->out_ld; args.out_bs = p->out_bs;
    args.m = p->m; args.n = p->n; args.o = p->o;
    args.accumulate = p->accumulate != 0;
    args.splits = p->n_splits > 1 ? p->n_splits : 1;
    args.out_split_stride = p->out_split_stride;
    hipStream_t stream = static_cast<hipStream_t>(stream_handle);

    const int column_tiles = (p->o + kmc::MC_COLUMNS - 1) / kmc::MC_COLUMNS;
    const bool rows4 = p->n > 0 && kmc_host::aligned16(p->matrix) && p->matrix_ld % 4 == 0 && p->matrix_bs % 4 == 0;
    const unsigned z = static_cast<unsigned>(p->l) * args.splits;
    hipError_t e;
    if (rows4) {
        // Measured on a 1 GB panel: 5.2 TB/s with one or two workgroups per CU, 4.0 with four and
        // more, so teams of 256 rows where those still make a workgroup per CU, of 128 otherwise.
        auto grid = [&](int waves_m) { return dim3((p->m + waves_m * kmc::MC4_WAVE_ROWS - 1) / (waves_m * kmc::MC4_WAVE_ROWS), column_tiles, z); };
        const dim3 wide = grid(2);
        if (static_cast<int64_t>(wide.x) * wide.y * wide.z >= 256)
            e = kmc_host::launch(kmc::matrix_times_coefficients_rows4<2, 4>, wide, dim3(512), stream, args);
        else
            e = kmc_host::launch(kmc::matrix_times_coefficients_rows4<1, 8>, grid(1), dim3(512), stream, args);
    } else
        e = kmc_host::launch(kmc::matrix_times_coefficients, dim3((p->m + kmc::MC_ROWS - 1) / kmc::MC_ROWS, column_tiles, z),
                             dim3(kmc::MC_THREADS), stream, args);
    if (e != hipSuccess) return kmc_host::fail_hip(e, "matrix_times_coefficients launch");
    return KMC_OK;
}
