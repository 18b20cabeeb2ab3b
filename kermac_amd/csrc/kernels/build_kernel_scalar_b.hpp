// The direct kernel for large problems whose panels have their rows contiguous: the b operand in scalar registers.
//
// build_kernel (build_kernel.hpp) stages both operands in LDS and every lane reads 16 floats of fragments per k
// for its 8 x 8 results -- a quarter of a float per term, 1 TB per launch at M = N = 30000, K = 1024, and with the
// copies that feed them the reason why the kernel runs at 2.1 GHz where its arithmetic alone runs at 2.37.  Here
// a wave owns 16 columns n and ALL its lanes share them, so b[n, k] is the same for every lane: it is loaded by
// scalar loads into scalar registers and enters the vector instructions as their scalar operand, which costs no
// LDS traffic at all.  A lane owns 4 consecutive rows m x those 16 columns: one 16-byte LDS read per k for 128
// vector instructions (a sixteenth of a float per term), and only a passes through LDS (copied straight from
// memory by global_load_lds_dwordx4, 1 KB per k-row of the 256 x 64 tile).  Workgroup 4 waves = 256 (m) x 64 (n),
// 92 registers, 33 KB of LDS, four workgroups per CU.  Measured on the walk alone, same box, M = N = 30000,
// K = 1024: 27.4 ms against 28.3 ms for build_kernel_four_waves (8 waves per workgroup on 256 x 128: 28.7; the
// 8 x 8 lane tile with b in scalar registers, 512 x 64: 28.4; five waves per SIMD: 27.6).
//
// What the host guarantees before it launches this kernel (build_kernel_inst.hip): both operands with rows
// contiguous and 16-byte aligned (the LOAD_COL_VEC loaders), K a multiple of 16, N a multiple of 16 or b a copy
// whose rows are padded to one (a wave's 16 columns can be loaded or do not exist; panel_copy.hip makes such copies
// of operands in any other storage), no ranges of one contraction (k_total = 0), not a repair launch.  A panel
// against itself (args.symmetric) runs the tiles that reach the diagonal or lie below it and stores each twice.
// The last tile row may be ragged in m: lanes beyond M copy nothing and store nothing.
// Results are those of build_kernel bit for bit: every element sums its terms over k in the same order.
// The reference has one kernel for all shapes (include/build_a_kernel.cuh:339-462).
#pragma once

#include "build_kernel.hpp"

namespace kmc {

constexpr int SB_TILE_M = 256;      // 64 lanes x 4 rows
constexpr int SB_WAVE_N = 16;       // columns of a wave: 16 scalars per k
constexpr int SB_TILE_N = 4 * SB_WAVE_N;
constexpr int SB_CHUNK = 4;         // k per group of scalar loads (64 scalar registers)
constexpr int SB_XCD_ROWS = 2;      // row blocks of a that one XCD works on at a time

// Two columns at a time: 8 independent subtractions (scalar minus vector), then 8 independent accumulations, as
// in row_abs_diff / row_square_diff of build_kernel.hpp.
#define KMC_SB_SUB8 \
    "v_sub_f32 %8, %20, %16\n\tv_sub_f32 %9, %20, %17\n\tv_sub_f32 %10, %20, %18\n\tv_sub_f32 %11, %20, %19\n\t" \
    "v_sub_f32 %12, %21, %16\n\tv_sub_f32 %13, %21, %17\n\tv_sub_f32 %14, %21, %18\n\tv_sub_f32 %15, %21, %19\n\t"
#define KMC_SB_OPERANDS \
    : "+v"(acc0[0]), "+v"(acc0[1]), "+v"(acc0[2]), "+v"(acc0[3]), "+v"(acc1[0]), "+v"(acc1[1]), "+v"(acc1[2]), "+v"(acc1[3]), \
      "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7) \
    : "v"(fa[0]), "v"(fa[1]), "v"(fa[2]), "v"(fa[3]), "s"(b0), "s"(b1)

template <int INNER_POW>
__device__ __forceinline__ void scalar_b_pair(float (&acc0)[4], float (&acc1)[4], const float (&fa)[4], float b0, float b1)
{
    static_assert(INNER_POW == POW_ABS || INNER_POW == POW_SQUARE || INNER_POW == POW_ABS_CUBE || INNER_POW == POW_ABS_FOURTH,
                  "absolute differences, their squares, cubes and fourth powers");
    float t0, t1, t2, t3, t4, t5, t6, t7;
    if (INNER_POW == POW_ABS) {
        asm volatile(KMC_SB_SUB8
                     "v_add_f32 %0, |%8|, %0\n\tv_add_f32 %1, |%9|, %1\n\tv_add_f32 %2, |%10|, %2\n\tv_add_f32 %3, |%11|, %3\n\t"
                     "v_add_f32 %4, |%12|, %4\n\tv_add_f32 %5, |%13|, %5\n\tv_add_f32 %6, |%14|, %6\n\tv_add_f32 %7, |%15|, %7"
                     KMC_SB_OPERANDS);
    } else if (INNER_POW == POW_SQUARE) {
        asm volatile(KMC_SB_SUB8
                     "v_fmac_f32 %0, %8, %8\n\tv_fmac_f32 %1, %9, %9\n\tv_fmac_f32 %2, %10, %10\n\tv_fmac_f32 %3, %11, %11\n\t"
                     "v_fmac_f32 %4, %12, %12\n\tv_fmac_f32 %5, %13, %13\n\tv_fmac_f32 %6, %14, %14\n\tv_fmac_f32 %7, %15, %15"
                     KMC_SB_OPERANDS);
    } else if (INNER_POW == POW_ABS_FOURTH) {
        // (t t) (t t), as inner_term of device_common.hpp compiles: the square in place of t, then one multiply-add
        asm volatile(KMC_SB_SUB8
                     "v_mul_f32 %8, %8, %8\n\tv_mul_f32 %9, %9, %9\n\tv_mul_f32 %10, %10, %10\n\tv_mul_f32 %11, %11, %11\n\t"
                     "v_mul_f32 %12, %12, %12\n\tv_mul_f32 %13, %13, %13\n\tv_mul_f32 %14, %14, %14\n\tv_mul_f32 %15, %15, %15\n\t"
                     "v_fmac_f32 %0, %8, %8\n\tv_fmac_f32 %1, %9, %9\n\tv_fmac_f32 %2, %10, %10\n\tv_fmac_f32 %3, %11, %11\n\t"
                     "v_fmac_f32 %4, %12, %12\n\tv_fmac_f32 %5, %13, %13\n\tv_fmac_f32 %6, %14, %14\n\tv_fmac_f32 %7, %15, %15"
                     KMC_SB_OPERANDS);
    } else {
        // |t| (t t): the squares into a second set of registers, then |t| times them added to the sums in one instruction each
        float u0, u1, u2, u3, u4, u5, u6, u7;
        asm volatile("v_sub_f32 %8, %28, %24\n\tv_sub_f32 %9, %28, %25\n\tv_sub_f32 %10, %28, %26\n\tv_sub_f32 %11, %28, %27\n\t"
                     "v_sub_f32 %12, %29, %24\n\tv_sub_f32 %13, %29, %25\n\tv_sub_f32 %14, %29, %26\n\tv_sub_f32 %15, %29, %27\n\t"
                     "v_mul_f32 %16, %8, %8\n\tv_mul_f32 %17, %9, %9\n\tv_mul_f32 %18, %10, %10\n\tv_mul_f32 %19, %11, %11\n\t"
                     "v_mul_f32 %20, %12, %12\n\tv_mul_f32 %21, %13, %13\n\tv_mul_f32 %22, %14, %14\n\tv_mul_f32 %23, %15, %15\n\t"
                     "v_fma_f32 %0, |%8|, %16, %0\n\tv_fma_f32 %1, |%9|, %17, %1\n\tv_fma_f32 %2, |%10|, %18, %2\n\tv_fma_f32 %3, |%11|, %19, %3\n\t"
                     "v_fma_f32 %4, |%12|, %20, %4\n\tv_fma_f32 %5, |%13|, %21, %5\n\tv_fma_f32 %6, |%14|, %22, %6\n\tv_fma_f32 %7, |%15|, %23, %7"
                     : "+v"(acc0[0]), "+v"(acc0[1]), "+v"(acc0[2]), "+v"(acc0[3]), "+v"(acc1[0]), "+v"(acc1[1]), "+v"(acc1[2]), "+v"(acc1[3]),
                       "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7),
                       "=&v"(u0), "=&v"(u1), "=&v"(u2), "=&v"(u3), "=&v"(u4), "=&v"(u5), "=&v"(u6), "=&v"(u7)
                     : "v"(fa[0]), "v"(fa[1]), "v"(fa[2]), "v"(fa[3]), "s"(b0), "s"(b1));
    }
}

__device__ __forceinline__ void scalar_b_fragment(float (&f)[4], const float *p)
{
    const float4 v = *reinterpret_cast<const float4 *>(p);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}

// The K walk of one 256 x 64 tile: acc[j][i] += inner(b[n0 + j, k] - a[m0 + 4 lane + i, k]) over k_slices slices of 16 k.
// `a_lane` points at this lane's 16 bytes of k-row 0 of the tile's rows (a + m0 + 4 lane), `b_columns` at the wave's 16
// columns of k-row 0 (uniform over the wave: the loads are scalar loads, provided the kernel's operand pointers are
// restrict-qualified parameters of their own).  `lds_a`: two slices of 16 k-rows of 256 floats and one row more, which
// the fragment read ahead of the last k of the second slice touches.  Every wave of the workgroup calls it (copies and
// barriers are the workgroup's); a wave without columns computes nothing.  Ends with a barrier: lds_a is free afterwards.
template <int INNER_POW>
__device__ __forceinline__ void scalar_b_walk(float (&acc)[SB_WAVE_N][4], const float *a_lane, i64 a_ld, const float *b_columns, i64 b_ld,
                                              int k_slices, bool lane_copies, bool wave_has_columns, float *lds_a, int lane, int wave)
{
    typedef const __attribute__((address_space(1))) void *global_address;
    typedef __attribute__((address_space(3))) void *lds_address;
    // copy j of 4 per slice and wave: k-row 4 * wave + j, 256 floats = 64 lanes x 16 bytes
    const float *src[4];
#pragma unroll
    for (int j = 0; j < 4; j++) src[j] = a_lane + (i64)(4 * wave + j) * a_ld;
    const i64 step_a = (i64)BK_TILE_K * a_ld;
    auto copy_slice = [&](int buffer) {
        if (lane_copies) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const unsigned to = (unsigned)(unsigned long)(lds_address)(lds_a + (buffer * BK_TILE_K + 4 * wave + j) * SB_TILE_M);
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"((global_address)src[j]), "s"(to) : "memory", "m0");
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) src[j] += step_a;
    };
    copy_slice(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
    __syncthreads();
    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        if (slice + 1 < k_slices) copy_slice(cur ^ 1);
        if (wave_has_columns) {
            const float *sa = lds_a + cur * BK_TILE_K * SB_TILE_M + 4 * lane;
            const float *bk = b_columns + (i64)slice * BK_TILE_K * b_ld;
            float fa0[4], fa1[4];
            scalar_b_fragment(fa0, sa);
#pragma unroll 1
            for (int kk = 0; kk < BK_TILE_K; kk += SB_CHUNK) {
                float sb[SB_CHUNK][SB_WAVE_N];
#pragma unroll
                for (int q = 0; q < SB_CHUNK; q++) {
                    const float4 *row = reinterpret_cast<const float4 *>(bk + (i64)(kk + q) * b_ld);
#pragma unroll
                    for (int v = 0; v < SB_WAVE_N / 4; v++) {
                        const float4 x = row[v];
                        sb[q][4 * v] = x.x; sb[q][4 * v + 1] = x.y; sb[q][4 * v + 2] = x.z; sb[q][4 * v + 3] = x.w;
                    }
                }
#pragma unroll
                for (int q = 0; q < SB_CHUNK; q += 2) {
                    scalar_b_fragment(fa1, sa + (kk + q + 1) * SB_TILE_M);
#pragma unroll
                    for (int j = 0; j < SB_WAVE_N; j += 2) scalar_b_pair<INNER_POW>(acc[j], acc[j + 1], fa0, sb[q][j], sb[q][j + 1]);
                    scalar_b_fragment(fa0, sa + (kk + q + 2) * SB_TILE_M);       // past the slice on its last k: read, never used
#pragma unroll
                    for (int j = 0; j < SB_WAVE_N; j += 2) scalar_b_pair<INNER_POW>(acc[j], acc[j + 1], fa1, sb[q + 1][j], sb[q + 1][j + 1]);
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);      // this wave's copies of the next slice have landed
        __syncthreads();
    }
}

// Outer power, epsilon mask, kernel function, regularised diagonal -- finish_tile of build_kernel.hpp on this kernel's
// 16 x 4 results per lane: columns n0 .. n0 + 15, rows m_first .. m_first + 3.
__device__ __forceinline__ void scalar_b_finish(float (&acc)[SB_WAVE_N][4], const BuildKernelArgs &args, int batch, int m_first, int n0)
{
    const int outer_power = args.outer_power;
    const int kernel_type = args.kernel_type;
    float p_outer = 0.0f, neg_gamma = 0.0f, regularization = 0.0f;
    if (outer_power == POW_POW) p_outer = args.p_outer ? args.p_outer[batch * args.p_outer_bs] : args.p_outer_value;
    if (kernel_type != KERNEL_NONE) {
        const float bw = args.bandwidth ? args.bandwidth[batch * args.bandwidth_bs] : args.bandwidth_value;
        neg_gamma = kernel_neg_gamma(kernel_type, bw);
        regularization = args.regularization ? args.regularization[batch * args.regularization_bs] : args.regularization_value;
    }
    const float epsilon = args.epsilon;
    auto for_each = [&](auto &&f) {
#pragma unroll
        for (int j = 0; j < SB_WAVE_N; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc[j][i] = f(acc[j][i]);
    };
    switch (outer_power) {
    case POW_ABS: for_each([](float v) { return __builtin_fabsf(v); }); break;
    case POW_SQUARE: for_each([](float v) { return v * v; }); break;
    case POW_SQRT: for_each([](float v) { return __builtin_amdgcn_sqrtf(v); }); break;
    case POW_POW: for_each([p_outer](float v) { return exp2f(p_outer * log2f(v)); }); break;
    default: break;
    }
    if (kernel_type != KERNEL_NONE)
        for_each([epsilon, neg_gamma](float v) { return expf((v < epsilon ? 0.0f : v) * neg_gamma); });
    if (kernel_type != KERNEL_NONE && regularization != 0.0f) {
        const float diagonal_value = 1.0f + regularization;
#pragma unroll
        for (int j = 0; j < SB_WAVE_N; j++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (args.reg_off_x + m_first + i == args.reg_off_y + n0 + j) acc[j][i] = diagonal_value;
    }
}

// The operands come in twice: inside `args`, and as restrict-qualified parameters, which is what lets the compiler
// prove that nothing the kernel writes (the copies into LDS, the result) can change b, and so load it with scalar
// loads (through args.b it takes vector loads of one address for all lanes, and the kernel spills).
template <int INNER_OP, int INNER_POW>
__global__ __launch_bounds__(BK_THREADS, 4) void build_kernel_scalar_b(const BuildKernelArgs args, const float *__restrict__ operand_a,
                                                                      const float *__restrict__ operand_b, float *__restrict__ result)
{
    static_assert(INNER_OP == OP_DIFF, "differences only");
    // Launched between a matrix-core kernel for squared differences and its repair launch: the whole result when the
    // sample taken in front of them left the call to the direct kernel (the matrix-core kernel has then only stamped
    // its tiles, and the repair launch behind finds none of the stamps), nothing otherwise.
    if (args.sample != nullptr && !sample_leaves_it_to_the_direct_kernel(args.sample)) return;
    __shared__ __attribute__((aligned(16))) float lds_a[(2 * BK_TILE_K + 1) * SB_TILE_M];
    const int tid = threadIdx.x;
    const int batch = blockIdx.y;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Tile order.  The hardware deals workgroups to the 8 XCDs round-robin by their launch-wide id.  Bands of 16 row
    // blocks of a: inside a band XCD x owns row blocks 2x and 2x + 1 and walks n with the row block fastest, so the ~128
    // workgroups resident on an XCD share 2 MB of a through its L2, and the two workgroups that stream the same b panel
    // (by scalar loads, which nothing but the L2 can share) run side by side: the second finds it there.  Measured at
    // M = N = 30000, K = 1024: 19 GB fetched from memory per launch against 31 GB with n fastest over the whole launch
    // or one row block per XCD, and 19.7 GB with three (3 MB of a no longer stay in a 4 MB L2 beside the stream).
    // The row blocks that do not fill a band are walked n fastest across all XCDs: a band of fewer than 16 would
    // leave XCDs idle for its whole length.
    const int tiles_n = (args.n + SB_TILE_N - 1) / SB_TILE_N;
    int tile_m, tile_n;
    if (args.symmetric) {
        // A panel against itself: the tiles that reach the diagonal or lie below it, tile row r holding columns
        // 0 .. 4 r + 3 (a tile is 256 x 64) and starting at id 2 r (r + 1); every tile is also stored mirrored.
        const int id = blockIdx.x;
        int row = (int)((sqrtf(2.0f * (float)id + 1.0f) - 1.0f) * 0.5f);
        while (2 * row * (row + 1) > id) row--;
        while (2 * (row + 1) * (row + 2) <= id) row++;
        tile_m = row;
        tile_n = id - 2 * row * (row + 1);
    } else {
        constexpr int band_rows = 8 * SB_XCD_ROWS;
        const int banded_rows = ((args.m + SB_TILE_M - 1) / SB_TILE_M) / band_rows * band_rows;
        const int banded = banded_rows * tiles_n;                    // a multiple of 8
        const int id = blockIdx.x;
        if (id < banded) {
            // the XCD of this workgroup: gridDim.x * blockIdx.y + id mod 8 -- a permutation of every 8 consecutive ids
            const int xcd = (id + (int)((gridDim.x % 8u) * (blockIdx.y % 8u))) & 7;
            const int sequence = id >> 3;                            // position in that XCD's queue
            const int band = sequence / (SB_XCD_ROWS * tiles_n);
            const int in_band = sequence - band * (SB_XCD_ROWS * tiles_n);
            tile_n = in_band / SB_XCD_ROWS;
            tile_m = band * band_rows + xcd * SB_XCD_ROWS + (in_band - tile_n * SB_XCD_ROWS);
        } else {
            const int rest = id - banded;
            const int row = rest / tiles_n;
            tile_n = rest - row * tiles_n;
            tile_m = banded_rows + row;
        }
    }
    const int m0 = tile_m * SB_TILE_M;
    const int n0 = tile_n * SB_TILE_N + SB_WAVE_N * wave;        // uniform over the wave
    const int m_valid = args.m - m0;
    const bool wave_has_columns = n0 < args.n;                   // all 16 can be loaded: n is a multiple of 16, or b a padded copy
    const int columns = args.n - n0 < SB_WAVE_N ? args.n - n0 : SB_WAVE_N;     // ... and these are stored
    const bool lane_copies = 4 * lane < m_valid;                 // the 16 bytes lie inside the row: its length is a multiple of 4 floats

    float acc[SB_WAVE_N][4];
#pragma unroll
    for (int j = 0; j < SB_WAVE_N; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[j][i] = 0.0f;
    scalar_b_walk<INNER_POW>(acc, operand_a + batch * args.a_bs + m0 + 4 * lane, args.a_ld,
                             operand_b + batch * args.b_bs + n0, args.b_ld, args.k / BK_TILE_K, lane_copies, wave_has_columns, lds_a, lane, wave);
    if (!wave_has_columns && !args.symmetric) return;

    // Epilogue and stores.  What depends on the lane's position is derived from a copy of the lane id that the compiler
    // cannot see through, so that it is not computed before the walk and kept through it.
    if (wave_has_columns) {
        int lane_after = lane;
        asm volatile("" : "+v"(lane_after));
        const int m_first = m0 + 4 * lane_after;
        scalar_b_finish(acc, args, batch, m_first, n0);
        // a wave writes 1 KB of consecutive m for each of its 16 columns
        float *c_rows = result + batch * args.c_bs + (i64)n0 * args.c_ld + m_first;
        if (args.c_vec && m_first + 3 < args.m) {
#pragma unroll
            for (int j = 0; j < SB_WAVE_N; j++)
                if (j < columns) *reinterpret_cast<float4 *>(c_rows + (i64)j * args.c_ld) = make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
        } else {
#pragma unroll
            for (int j = 0; j < SB_WAVE_N; j++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (j < columns && m_first + i < args.m) c_rows[(i64)j * args.c_ld + i] = acc[j][i];
        }
    }
    if (!args.symmetric) return;

    // The same values at C(n, m).  Through LDS (idle after the walk, which ends with a barrier), 64 rows m at a time: the
    // lanes that hold them write their 4 x 16 results as [m][n], and the workgroup stores 16 rows of 256 bytes per
    // instruction.  Elements on the far side of the diagonal that this writes are the ones another tile computes for
    // itself, from the same terms in the same order: the same bits.
    constexpr int MIRROR_PITCH = SB_TILE_N + 4;
    static_assert(64 * MIRROR_PITCH <= (2 * BK_TILE_K + 1) * SB_TILE_M, "a quarter of the tile fits the staging array");
    float *c_batch = result + batch * args.c_bs;
    const int n_tile = tile_n * SB_TILE_N;
#pragma unroll 1
    for (int quarter = 0; quarter < 4; quarter++) {
        if ((lane >> 4) == quarter) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int v = 0; v < SB_WAVE_N / 4; v++)
                    *reinterpret_cast<float4 *>(lds_a + (4 * (lane & 15) + i) * MIRROR_PITCH + SB_WAVE_N * wave + 4 * v) =
                        make_float4(acc[4 * v][i], acc[4 * v + 1][i], acc[4 * v + 2][i], acc[4 * v + 3][i]);
        }
        __syncthreads();
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const int row = 16 * pass + (tid >> 4), column = 4 * (tid & 15);
            const int m = m0 + 64 * quarter + row, n = n_tile + column;
            if (m < args.m && n < args.n) {
                const float4 v = *reinterpret_cast<const float4 *>(lds_a + row * MIRROR_PITCH + column);
                float *to = c_batch + (i64)m * args.c_ld + n;
                if (args.c_vec && n + 3 < args.n) {
                    *reinterpret_cast<float4 *>(to) = v;
                } else {
                    to[0] = v.x;
                    if (n + 1 < args.n) to[1] = v.y;
                    if (n + 2 < args.n) to[2] = v.z;
                    if (n + 3 < args.n) to[3] = v.w;
                }
            }
        }
        __syncthreads();
    }
}

}  // namespace kmc
