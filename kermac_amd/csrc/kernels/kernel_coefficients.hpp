// Fused kernel matrix x coefficients for gfx950:
//
//   out[m, o, l] = sum_n Kmat(m, n, l) * coef[n, o, l]
//
// where Kmat is the value the pairwise-reduction kernel (build_kernel.hpp) would
// store; the m x n matrix never leaves the chip.  The reference has no such
// kernel: its run_kernel always writes out[L,M,N]
// (src/kermac/build_a_kernel.py:259,378-392) and leaves the contraction to the
// caller.
//
// One workgroup owns 128 rows m (and one batch, and one chunk of up to 32
// coefficient columns) and walks over all n in tiles of 128:
//   1. the tile's 128 x 32 block of coefficients is staged in LDS;
//   2. the tile's kernel values are produced in registers exactly as in
//      build_kernel (same K walk on the vector ALU, same epilogue);
//   3. they are written to LDS 32 n at a time (into the staging buffers of step
//      2, which are idle by then) and contracted on the matrix cores:
//      out[128 m x 32 o] += Kv[128 m x 32 n] * coef[32 n x 32 o] as 16 x 16 x 4
//      fp32 MFMAs, each wave owning 32 m x 32 o.
// Step 3 runs on the matrix pipe, so it overlaps with step 2 of the other
// workgroups resident on the same CU instead of competing for VALU issue slots.
#pragma once

#include "build_kernel.hpp"

namespace kmc {

typedef float kc_float4 __attribute__((ext_vector_type(4)));

struct KernelCoefficientsArgs {
    BuildKernelArgs kernel;        // c / c_ld / c_bs unused
    int o;                         // coefficient columns in total
    int o_chunks;                  // ceil(o / columns); blockIdx.y = batch * o_chunks + chunk
    const float *coef; i64 coef_ld, coef_bs;   // [n, o], o contiguous
    float *out; i64 out_ld, out_bs;            // [m, o], o contiguous
    int coef_vec;                  // coef, coef_ld, coef_bs multiples of 16 bytes
    int columns;                   // coefficient columns per workgroup: the COLUMNS the launched kernel was built with
    // The centres can be cut into consecutive ranges of whole n tiles, one per blockIdx.z: range z
    // walks `split_tiles` tiles from tile z * split_tiles on and writes its partial product to
    // out + z * out_split_stride; the caller adds the ranges.  One range: the whole product.
    int split_tiles;
    i64 out_split_stride;
};

// First centre and one past the last centre of the range this workgroup walks.
__device__ __forceinline__ void centre_range(const KernelCoefficientsArgs &kc, int &n_begin, int &n_end)
{
    const i64 first = (i64)blockIdx.z * kc.split_tiles * BK_TILE_N;
    const i64 last = first + (i64)kc.split_tiles * BK_TILE_N;
    n_begin = (int)(first < kc.kernel.n ? first : kc.kernel.n);
    n_end = (int)(last < kc.kernel.n ? last : kc.kernel.n);
}

constexpr int KC_COLUMNS = 32;      // coefficient columns per workgroup (64 in the wide instantiations)
constexpr int KC_PASS_N = 32;       // n per contraction pass
// [n][m] pitch of the kernel values in LDS: the 4 n-rows an MFMA operand read
// touches land in 4 disjoint groups of 16 banks.
constexpr int KC_KV_PITCH = BK_TILE_M + 16;
constexpr int KC_STAGE_FLOATS = 2 * (2 * BK_LDS_SLICE + BK_LDS_PITCH);

// COLUMNS: 32, or 64 for more than 32 coefficient columns (every chunk of columns
// rebuilds the whole kernel matrix, so O = 64 in two chunks of 32 costs twice O = 32;
// 64 columns per workgroup still leave LDS for two workgroups per CU).
// Waves per SIMD the 32-column kernel is compiled for.  Three (168 registers; the compiler spills
// about 20, none of them inside the K walk) let a CU hold three workgroups, which is what the K
// walk needs to reach its rate; measured with the centres cut into ranges (so that there are
// workgroups for every place) 9.6 against 10.4 ms at L = 4, M = N = 16384, K = 256, O = 32.
#ifndef KC_MIN_WAVES
#define KC_MIN_WAVES 3
#endif
template <int INNER_OP, int INNER_POW, int LOAD_A, int LOAD_B, int COLUMNS = KC_COLUMNS>
__global__ __launch_bounds__(BK_THREADS, COLUMNS == KC_COLUMNS ? KC_MIN_WAVES : 2) void kernel_times_coefficients(const KernelCoefficientsArgs kc)
{
    static_assert(COLUMNS % 32 == 0, "whole pairs of 16-column blocks");
    constexpr int COLUMN_BLOCKS = COLUMNS / 16;
    static_assert(KC_PASS_N * KC_KV_PITCH <= KC_STAGE_FLOATS, "kernel values must fit in the staging buffers");
    // Staging buffers of the K walk; between two K walks the same memory holds
    // one pass of kernel values.
    __shared__ __attribute__((aligned(16))) float lds_stage[KC_STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float lds_coef[BK_TILE_N * COLUMNS];   // [n][o]
    float *lds_a = lds_stage;
    float *lds_b = lds_stage + KC_STAGE_FLOATS / 2;
    float *lds_kv = lds_stage;

    const BuildKernelArgs &args = kc.kernel;
    const int tid = threadIdx.x;
    const int tx = tid & 15;
    const int ty = tid >> 4;
    const int batch = blockIdx.y / kc.o_chunks;
    const int o_base = (blockIdx.y % kc.o_chunks) * COLUMNS;
    const int m0 = blockIdx.x * BK_TILE_M;
    const int m_valid = args.m - m0;

    float p_inner = 0.0f;
    if (INNER_POW == POW_POW) {
        p_inner = args.p_inner ? args.p_inner[batch * args.p_inner_bs] : args.p_inner_value;
    }

    // Contraction role (v_mfma_f32_16x16x4_f32, lane = 16 q + r): wave w owns rows
    // 32 w .. 32 w + 31 as two row blocks of 16, times COLUMNS / 16 column blocks of 16.
    // Operand A: lane supplies Kv[m = r][n = q]; operand B: coef[n = q][o = r];
    // result: lane holds rows 4 q .. 4 q + 3 of column r.
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int q = lane >> 4;
    const int r = lane & 15;
    const float *coef_batch = kc.coef + batch * kc.coef_bs;
    const bool coef_vec = kc.coef_vec;
    kc_float4 out_acc[2][COLUMN_BLOCKS];   // [row block][column block]
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int ob = 0; ob < COLUMN_BLOCKS; ob++) out_acc[mb][ob] = kc_float4{0.0f, 0.0f, 0.0f, 0.0f};

    int n_begin, n_end;
    centre_range(kc, n_begin, n_end);
    for (int n0 = n_begin; n0 < n_end; n0 += BK_TILE_N) {
        const int n_valid = args.n - n0;

        // 1. coefficients of this n tile -> LDS, zero filled past N and past O.
        //    Lane t stages row t/2, half t&1 of the columns.  The barrier that ends
        //    the previous tile's last pass protects lds_coef; the barriers inside
        //    the K walk below publish it.
        {
            const int n_local = tid >> 1;
            const int c0 = (tid & 1) * (COLUMNS / 2);
            const bool row_live = n_local < n_valid;
            const float *src = coef_batch + (i64)(n0 + n_local) * kc.coef_ld + o_base + c0;
#pragma unroll
            for (int v4 = 0; v4 < COLUMNS / 8; v4++) {
                const int cols_left = kc.o - (o_base + c0 + 4 * v4);
                float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (row_live) v = load4_guarded(src + 4 * v4, cols_left, coef_vec);
                *reinterpret_cast<float4 *>(lds_coef + n_local * COLUMNS + c0 + 4 * v4) = v;
            }
        }

        // 2. kernel values of the tile, in registers.
        TileLoader<LOAD_A> load_a;
        TileLoader<LOAD_B> load_b;
        load_a.init(args.a + batch * args.a_bs, args.a_ld, m0, tid);
        load_b.init(args.b + batch * args.b_bs, args.b_ld, n0, tid);
        float acc[8][8];
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int i = 0; i < 8; i++) acc[j][i] = 0.0f;
        if (m_valid >= BK_TILE_M && n_valid >= BK_TILE_N && args.k % BK_TILE_K == 0) {
            accumulate_tile<INNER_OP, INNER_POW, LOAD_A, LOAD_B, true>(
                acc, load_a, load_b, lds_a, lds_b, args.k, m_valid, n_valid, p_inner, args.diff_sign, tx, ty);
        } else {
            accumulate_tile<INNER_OP, INNER_POW, LOAD_A, LOAD_B, false>(
                acc, load_a, load_b, lds_a, lds_b, args.k, m_valid, n_valid, p_inner, args.diff_sign, tx, ty);
        }
        if (args.k == 0) __syncthreads();   // no K walk, no barrier: publish lds_coef here
        finish_tile(acc, args, batch, m0, n0, tx, ty);

        // 3. four passes of 32 n.  Pass p holds n_local in [32 p, 32 p + 32): rows j
        //    with (j >> 2) == (p >> 1) of the lanes with (ty >> 3) == (p & 1).  The K
        //    walk ended with a barrier, so its staging memory is free.
#pragma unroll
        for (int pass = 0; pass < BK_TILE_N / KC_PASS_N; pass++) {
            if ((ty >> 3) == (pass & 1)) {
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int j = (pass >> 1) * 4 + jj;
                    const int n_pass = (ty & 7) * 4 + jj;                    // 0..31 inside the pass
                    const bool live = pass * KC_PASS_N + n_pass < n_valid;   // columns past N contribute 0
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        float4 v = make_float4(acc[j][4 * h], acc[j][4 * h + 1], acc[j][4 * h + 2], acc[j][4 * h + 3]);
                        if (!live) v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                        *reinterpret_cast<float4 *>(lds_kv + n_pass * KC_KV_PITCH + tx * 4 + h * 64) = v;
                    }
                }
            }
            __syncthreads();
            const float *kv_src = lds_kv + q * KC_KV_PITCH + wave * 32 + r;
            const float *coef_src = lds_coef + (pass * KC_PASS_N + q) * COLUMNS + r;
            // Operand double buffer: reads of chunk c+1 go out before the MFMAs of chunk c.
            float fa[2][2], fb[2][COLUMN_BLOCKS];
#pragma unroll
            for (int t = 0; t < 2; t++) fa[0][t] = kv_src[t * 16];
#pragma unroll
            for (int t = 0; t < COLUMN_BLOCKS; t++) fb[0][t] = coef_src[t * 16];
#pragma unroll
            for (int chunk = 0; chunk < KC_PASS_N / 4; chunk++) {
                const int use = chunk & 1;
                if (chunk + 1 < KC_PASS_N / 4) {
#pragma unroll
                    for (int t = 0; t < 2; t++) fa[use ^ 1][t] = kv_src[(chunk + 1) * 4 * KC_KV_PITCH + t * 16];
#pragma unroll
                    for (int t = 0; t < COLUMN_BLOCKS; t++) fb[use ^ 1][t] = coef_src[(chunk + 1) * 4 * COLUMNS + t * 16];
                }
                __builtin_amdgcn_sched_barrier(0);   // keep those reads above the MFMAs
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
#pragma unroll
                    for (int ob = 0; ob < COLUMN_BLOCKS; ob++)
                        out_acc[mb][ob] =
                            __builtin_amdgcn_mfma_f32_16x16x4f32(fa[use][mb], fb[use][ob], out_acc[mb][ob], 0, 0, 0);
            }
            __syncthreads();
        }
    }

    // Store: this lane holds rows 32 wave + 16 mb + 4 q + i, column 16 ob + r.
    float *out_batch = kc.out + batch * kc.out_bs + blockIdx.z * kc.out_split_stride;
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int ob = 0; ob < COLUMN_BLOCKS; ob++) {
            const int o = o_base + ob * 16 + r;
            if (o >= kc.o) continue;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int m_local = wave * 32 + mb * 16 + q * 4 + i;
                if (m_local < m_valid) out_batch[(i64)(m0 + m_local) * kc.out_ld + o] = out_acc[mb][ob][i];
            }
        }
}

}  // namespace kmc
