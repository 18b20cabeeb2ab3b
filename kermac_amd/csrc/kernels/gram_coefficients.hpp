// Fused kernel matrix x coefficients for the squared-difference descriptors (L2
// norm, Laplace-L2, Gaussian) with the kernel matrix produced on the matrix cores:
//
//   out[m, o, l] = sum_n Kmat(m, n, l) * coef[n, o, l]
//   Kmat from  sum_k (b[n,k] - a[m,k])^2 = |a_m|^2 + |b_n|^2 - 2 a_m . b_n
//
// The opt-in counterpart of kernel_times_coefficients (kernel_coefficients.hpp) in
// the way gram_l2_kernel (gram_kernel.hpp) is the counterpart of build_kernel: same
// workgroup ownership (128 rows m, up to 32 coefficient columns, all n in tiles of
// 128), same staging of the coefficients, same contraction on the matrix cores;
// only the tile's kernel values come from gram_walk instead of the vector K walk.
// The expansion cancels for near-duplicate points, so every tile is checked with
// the rule of gram_l2_kernel (an element with d^2 < gram_trust * (|a|^2 + |b|^2)
// makes the tile distrusted); a distrusted tile is recomputed on the spot with the
// subtract-square-accumulate walk, so its values are those of the direct kernel.
// The reference has neither kernel (src/kermac/build_a_kernel.py:259,378-392).
#pragma once

#include "gram_kernel.hpp"
#include "kernel_coefficients.hpp"

namespace kmc {

template <int LOAD_A, int LOAD_B, bool CENTRED = false>
__global__ __launch_bounds__(BK_THREADS, 2) void gram_times_coefficients(const KernelCoefficientsArgs kc)
{
    static_assert(GRAM_DEPTH == 1, "the staging buffers below hold one slice per stage");
    __shared__ __attribute__((aligned(16))) float lds_stage[KC_STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float lds_coef[BK_TILE_N * KC_COLUMNS];   // [n][o]
    __shared__ float lds_norm_a[BK_TILE_M];
    __shared__ float lds_norm_b[BK_TILE_N];
    float *lds_a = lds_stage;
    float *lds_b = lds_stage + KC_STAGE_FLOATS / 2;
    float *lds_kv = lds_stage;

    const BuildKernelArgs &args = kc.kernel;
    const int tid = threadIdx.x;
    const int tx = tid & 15;
    const int ty = tid >> 4;
    const int batch = blockIdx.y / kc.o_chunks;
    const int o_base = (blockIdx.y % kc.o_chunks) * KC_COLUMNS;
    const int m0 = blockIdx.x * BK_TILE_M;
    const int m_valid = args.m - m0;

    // Roles in the matrix-core K walk (see gram_kernel.hpp): wave (wave_m, wave_n) owns
    // 64 x 64 of the tile, lane = 32 h + i.
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = (wave & 1) * 64;
    const int wave_n = (wave >> 1) * 64;
    const int h = lane >> 5;
    const int i = lane & 31;
    // Roles in the contraction (see kernel_coefficients.hpp): wave owns rows 32 wave ..
    // 32 wave + 31, lane = 16 q + r.
    const int q = lane >> 4;
    const int r = lane & 15;

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
    const bool regularize = kernel_type != KERNEL_NONE && regularization != 0.0f;
    const float diagonal_value = 1.0f + regularization;

    const float *coef_batch = kc.coef + batch * kc.coef_bs;
    const bool coef_vec = kc.coef_vec;
    kc_float4 out_acc[2][2];   // [row block][column block]
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int ob = 0; ob < 2; ob++) out_acc[mb][ob] = kc_float4{0.0f, 0.0f, 0.0f, 0.0f};

    int n_begin, n_end;
    centre_range(kc, n_begin, n_end);
    for (int n0 = n_begin; n0 < n_end; n0 += BK_TILE_N) {
        const int n_valid = args.n - n0;

        // 1. coefficients of this n tile -> LDS, zero filled past N and past O (as in
        //    kernel_times_coefficients; the barriers of the K walk publish them).
        {
            const int n_local = tid >> 1;
            const int c0 = (tid & 1) * 16;
            const bool row_live = n_local < n_valid;
            const float *src = coef_batch + (i64)(n0 + n_local) * kc.coef_ld + o_base + c0;
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                const int cols_left = kc.o - (o_base + c0 + 4 * v4);
                float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (row_live) v = load4_guarded(src + 4 * v4, cols_left, coef_vec);
                *reinterpret_cast<float4 *>(lds_coef + n_local * KC_COLUMNS + c0 + 4 * v4) = v;
            }
        }

        // 2. kernel values of the tile.  kv[] holds them in one of two register layouts:
        //    the matrix-core one (kv[32 mt + 16 nt + v] = tile element at
        //    m = wave_m + 32 mt + 8 (v / 4) + 4 h + v % 4, n = wave_n + 32 nt + i) or,
        //    for a distrusted tile, the one of the vector walk (kv[8 j + i2] at
        //    n = 4 ty + j % 4 + 64 (j / 4), m = 4 tx + i2 % 4 + 64 (i2 / 4)).
        float kv[64];
        bool distrusted;
        {
            TileLoader<LOAD_A> load_a;
            TileLoader<LOAD_B> load_b;
            load_a.init(args.a + batch * args.a_bs, args.a_ld, m0, tid);
            load_b.init(args.b + batch * args.b_bs, args.b_ld, n0, tid);
            float square_a[8], square_b[8];
#pragma unroll
            for (int s = 0; s < 8; s++) square_a[s] = square_b[s] = 0.0f;
            gram_float16 acc[2][2];
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[mt][nt][v] = 0.0f;
            const float *frag_a = lds_a + h * BK_LDS_PITCH + wave_m + i;
            const float *frag_b = lds_b + h * BK_LDS_PITCH + wave_n + i;
            const float *centre = CENTRED ? centre_to_subtract(args, batch) : nullptr;
            auto walk = [&](auto centred) {
                constexpr bool C = decltype(centred)::value;
                if (m_valid >= BK_TILE_M && n_valid >= BK_TILE_N && args.k % GRAM_STAGE_K == 0) {
                    gram_walk<LOAD_A, LOAD_B, true, C>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, frag_a, frag_b,
                                                       args.k, m_valid, n_valid, centre);
                } else {
                    gram_walk<LOAD_A, LOAD_B, false, C>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, frag_a, frag_b,
                                                        args.k, m_valid, n_valid, centre);
                }
            };
            if (CENTRED && centre) walk(GramSwitch<CENTRED>{});
            else walk(GramSwitch<false>{});
            row_norms<LOAD_A>(load_a, square_a, lds_a, lds_norm_a, tid);
            row_norms<LOAD_B>(load_b, square_b, lds_b, lds_norm_b, tid);
            __syncthreads();

            int distrust = 0;
            float norm_b[2];
            int n_local[2];
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                n_local[nt] = wave_n + nt * 32 + i;
                norm_b[nt] = lds_norm_b[n_local[nt]];
            }
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m_local = wave_m + mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                    const float norm_a = lds_norm_a[m_local];
#pragma unroll
                    for (int nt = 0; nt < 2; nt++) {
                        const float norms = norm_a + norm_b[nt];
                        float d2 = norms - 2.0f * acc[mt][nt][v];
                        // a result that is not a number (inf - inf of huge operands) is not trusted either
                        if (m_local < m_valid && n_local[nt] < n_valid && !(d2 >= args.gram_trust * norms)) distrust = 1;
                        d2 = fmaxf(d2, 0.0f);
                        float value = epilogue_value(d2, outer_power, kernel_type, p_outer, neg_gamma, args.epsilon);
                        if (regularize && args.reg_off_x + m0 + m_local == args.reg_off_y + n0 + n_local[nt])
                            value = diagonal_value;
                        kv[32 * mt + 16 * nt + v] = value;
                    }
                }
            // The barrier inside also ends every read of the norms and of the staging memory.
            distrusted = __syncthreads_or(distrust) != 0;
        }
        if (distrusted) {
            TileLoader<LOAD_A> load_a;
            TileLoader<LOAD_B> load_b;
            load_a.init(args.a + batch * args.a_bs, args.a_ld, m0, tid);
            load_b.init(args.b + batch * args.b_bs, args.b_ld, n0, tid);
            float acc[8][8];
#pragma unroll
            for (int j = 0; j < 8; j++)
#pragma unroll
                for (int i2 = 0; i2 < 8; i2++) acc[j][i2] = 0.0f;
            if (m_valid >= BK_TILE_M && n_valid >= BK_TILE_N && args.k % BK_TILE_K == 0) {
                accumulate_tile<OP_DIFF, POW_SQUARE, LOAD_A, LOAD_B, true>(
                    acc, load_a, load_b, lds_a, lds_b, args.k, m_valid, n_valid, 0.0f, args.diff_sign, tx, ty);
            } else {
                accumulate_tile<OP_DIFF, POW_SQUARE, LOAD_A, LOAD_B, false>(
                    acc, load_a, load_b, lds_a, lds_b, args.k, m_valid, n_valid, 0.0f, args.diff_sign, tx, ty);
            }
            finish_tile(acc, args, batch, m0, n0, tx, ty);
#pragma unroll
            for (int j = 0; j < 8; j++)
#pragma unroll
                for (int i2 = 0; i2 < 8; i2++) kv[8 * j + i2] = acc[j][i2];
        }

        // 3. four passes of 32 n: kernel values -> LDS ([n][m], into the idle staging
        //    memory), then out[128 m x 32 o] += Kv[128 m x 32 n] * coef[32 n x 32 o].
#pragma unroll
        for (int pass = 0; pass < BK_TILE_N / KC_PASS_N; pass++) {
            if (distrusted) {
                if ((ty >> 3) == (pass & 1)) {
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) {
                        const int j = (pass >> 1) * 4 + jj;
                        const int n_pass = (ty & 7) * 4 + jj;
                        const bool live = pass * KC_PASS_N + n_pass < n_valid;
#pragma unroll
                        for (int hh = 0; hh < 2; hh++) {
                            float4 v = make_float4(kv[8 * j + 4 * hh], kv[8 * j + 4 * hh + 1], kv[8 * j + 4 * hh + 2],
                                                   kv[8 * j + 4 * hh + 3]);
                            if (!live) v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                            *reinterpret_cast<float4 *>(lds_kv + n_pass * KC_KV_PITCH + tx * 4 + hh * 64) = v;
                        }
                    }
                }
            } else if (wave_n == 64 * (pass >> 1)) {
                // the two waves that own these 32 columns: row i of the pass, 8 pieces of 4 m
                const int nt = pass & 1;
                const bool live = pass * KC_PASS_N + i < n_valid;
#pragma unroll
                for (int mt = 0; mt < 2; mt++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const int base = 32 * mt + 16 * nt + 4 * g;
                        float4 v = make_float4(kv[base], kv[base + 1], kv[base + 2], kv[base + 3]);
                        if (!live) v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                        *reinterpret_cast<float4 *>(lds_kv + i * KC_KV_PITCH + wave_m + mt * 32 + 8 * g + 4 * h) = v;
                    }
            }
            __syncthreads();
            const float *kv_src = lds_kv + q * KC_KV_PITCH + wave * 32 + r;
            const float *coef_src = lds_coef + (pass * KC_PASS_N + q) * KC_COLUMNS + r;
            float fa[2][2], fb[2][2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                fa[0][t] = kv_src[t * 16];
                fb[0][t] = coef_src[t * 16];
            }
#pragma unroll
            for (int chunk = 0; chunk < KC_PASS_N / 4; chunk++) {
                const int use = chunk & 1;
                if (chunk + 1 < KC_PASS_N / 4) {
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        fa[use ^ 1][t] = kv_src[(chunk + 1) * 4 * KC_KV_PITCH + t * 16];
                        fb[use ^ 1][t] = coef_src[(chunk + 1) * 4 * KC_COLUMNS + t * 16];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);   // keep those reads above the MFMAs
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
#pragma unroll
                    for (int ob = 0; ob < 2; ob++)
                        out_acc[mb][ob] =
                            __builtin_amdgcn_mfma_f32_16x16x4f32(fa[use][mb], fb[use][ob], out_acc[mb][ob], 0, 0, 0);
            }
            __syncthreads();
        }
    }

    // Store: this lane holds rows 32 wave + 16 mb + 4 q + e, column 16 ob + r.
    float *out_batch = kc.out + batch * kc.out_bs + blockIdx.z * kc.out_split_stride;
#pragma unroll
    for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int ob = 0; ob < 2; ob++) {
            const int o = o_base + ob * 16 + r;
            if (o >= kc.o) continue;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int m_local = wave * 32 + mb * 16 + q * 4 + e;
                if (m_local < m_valid) out_batch[(i64)(m0 + m_local) * kc.out_ld + o] = out_acc[mb][ob][e];
            }
        }
}

}  // namespace kmc
