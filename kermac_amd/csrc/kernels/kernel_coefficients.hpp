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
//      build_kernel (same K walk, same epilogue);
//   3. they are written to LDS 32 n at a time and contracted: every lane owns
//      4 rows m x 8 columns o and half of the 32 n, so one pass is 16 steps of
//      three 128-bit LDS reads and 32 multiply-adds.
// Step 3 costs 2 x 32 VALU operations per (m, n) against 2 x K for step 2.  The
// two n-halves are summed through LDS once, at the very end.
#pragma once

#include "build_kernel.hpp"

namespace kmc {

struct KernelCoefficientsArgs {
    BuildKernelArgs kernel;        // c / c_ld / c_bs unused
    int o;                         // coefficient columns in total
    int o_chunks;                  // ceil(o / 32); blockIdx.y = batch * o_chunks + chunk
    const float *coef; i64 coef_ld, coef_bs;   // [n, o], o contiguous
    float *out; i64 out_ld, out_bs;            // [m, o], o contiguous
    int coef_vec;                  // coef, coef_ld, coef_bs multiples of 16 bytes
};

constexpr int KC_COLUMNS = 32;      // coefficient columns per workgroup
constexpr int KC_PASS_N = 32;       // n per contraction pass

template <int INNER_OP, int INNER_POW, int LOAD_A, int LOAD_B>
__global__ __launch_bounds__(BK_THREADS) void kernel_times_coefficients(const KernelCoefficientsArgs kc)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * BK_LDS_SLICE + BK_LDS_PITCH];
    __shared__ __attribute__((aligned(16))) float lds_kv[KC_PASS_N * BK_LDS_PITCH];   // [n][m]
    __shared__ __attribute__((aligned(16))) float lds_coef[BK_TILE_N * KC_COLUMNS];   // [n][o]

    const BuildKernelArgs &args = kc.kernel;
    const int tid = threadIdx.x;
    const int tx = tid & 15;
    const int ty = tid >> 4;
    const int batch = blockIdx.y / kc.o_chunks;
    const int o_base = (blockIdx.y % kc.o_chunks) * KC_COLUMNS;
    const int m0 = blockIdx.x * BK_TILE_M;
    const int m_valid = args.m - m0;

    float p_inner = 0.0f;
    if (INNER_POW == POW_POW) {
        p_inner = args.p_inner ? args.p_inner[batch * args.p_inner_bs] : args.p_inner_value;
    }

    // Contraction role of this lane: rows 4*row_group .. +3, columns 8*col_group .. +7
    // (relative to o_base), and the n of parity-half n_half of every pass.
    const int row_group = tid & 31;
    const int col_group = (tid >> 5) & 3;
    const int n_half = tid >> 7;
    const float *coef_batch = kc.coef + batch * kc.coef_bs;
    const bool coef_vec = kc.coef_vec;
    float out_acc[4][8];
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
        for (int o = 0; o < 8; o++) out_acc[r][o] = 0.0f;

    for (int n0 = 0; n0 < args.n; n0 += BK_TILE_N) {
        const int n_valid = args.n - n0;

        // 1. coefficients of this n tile -> LDS, zero filled past N and past O.
        //    Lane t stages row t/2, columns 16*(t&1) .. +15.  The barrier that ends
        //    the previous tile's last pass protects lds_coef; the barriers inside
        //    the K walk below publish it.
        {
            const int n_local = tid >> 1;
            const int c0 = (tid & 1) * 16;
            const bool row_live = n_local < n_valid;
            const float *src = coef_batch + (i64)(n0 + n_local) * kc.coef_ld + o_base + c0;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int cols_left = kc.o - (o_base + c0 + 4 * q);
                float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (row_live) v = load4_guarded(src + 4 * q, cols_left, coef_vec);
                *reinterpret_cast<float4 *>(lds_coef + n_local * KC_COLUMNS + c0 + 4 * q) = v;
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

        // 3. four passes of 32 n.  Pass q holds n_local in [32 q, 32 q + 32); those
        //    are rows j with (j >> 2) == (q >> 1) of the lanes with (ty >> 3) == (q & 1).
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
                        *reinterpret_cast<float4 *>(lds_kv + n_pass * BK_LDS_PITCH + tx * 4 + h * 64) = v;
                    }
                }
            }
            __syncthreads();
            const float *kv_src = lds_kv + row_group * 4;
            const float *coef_src = lds_coef + pass * KC_PASS_N * KC_COLUMNS + col_group * 8;
#pragma unroll 4
            for (int step = 0; step < KC_PASS_N / 2; step++) {
                const int n_pass = 2 * step + n_half;
                const float4 kv = *reinterpret_cast<const float4 *>(kv_src + n_pass * BK_LDS_PITCH);
                const float4 w0 = *reinterpret_cast<const float4 *>(coef_src + n_pass * KC_COLUMNS);
                const float4 w1 = *reinterpret_cast<const float4 *>(coef_src + n_pass * KC_COLUMNS + 4);
                const float kvv[4] = {kv.x, kv.y, kv.z, kv.w};
                const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int o = 0; o < 8; o++) out_acc[r][o] += kvv[r] * wv[o];
            }
            __syncthreads();
        }
    }

    // Sum the two n-halves through LDS (lds_kv is free after the last barrier) and store.
    float *exchange = lds_kv;   // 128 lanes x 32 floats = 4096 <= 32 * 132
    if (n_half == 1) {
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int o = 0; o < 8; o++) exchange[(r * 8 + o) * 128 + (tid & 127)] = out_acc[r][o];
    }
    __syncthreads();
    if (n_half == 0) {
        float *out_batch = kc.out + batch * kc.out_bs;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int m_local = row_group * 4 + r;
            if (m_local >= m_valid) continue;
            float *dst = out_batch + (i64)(m0 + m_local) * kc.out_ld + o_base + col_group * 8;
#pragma unroll
            for (int o = 0; o < 8; o++) {
                const float total = out_acc[r][o] + exchange[(r * 8 + o) * 128 + (tid & 127)];
                if (o_base + col_group * 8 + o < kc.o) dst[o] = total;
            }
        }
    }
}

}  // namespace kmc
