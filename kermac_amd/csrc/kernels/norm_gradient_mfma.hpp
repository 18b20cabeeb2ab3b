// Kernel-gradient contraction for more than 8 outputs per (m, n), on the matrix
// cores of gfx950:
//
//   E[m, n, o, l] = sum_k C[o,k,l] * T[(m,n), k]      T = A[m,k,l] * g( D[m,n,l] - B[n,k,l] )
//
// Same operator as norm_gradient.hpp (reference: include/p_norm_gradient.cuh:407-497);
// this formulation is used when O > 8.  For a fixed n the contraction is a small
// GEMM: rows = 16 consecutive m, columns = 16 outputs o, depth = k.  Its left
// operand T does not exist in memory: every lane computes the one element it has
// to supply (2 to 3 VALU instructions, see gradient_term) right before the
// v_mfma_f32_16x16x4_f32 that consumes it, so the vector ALU generates operands
// while the matrix core does the 2*O flops per (m,n,k) that dominate the work.
//
// Operand layouts of v_mfma_f32_16x16x4_f32 (lane = 16*q + r, q = 0..3, r = 0..15):
//   A (16 x 4):  lane supplies A[row r][k q]
//   B (4 x 16):  lane supplies B[k q][column r]
//   D (16 x 16): lane holds D[rows 4q .. 4q+3][column r] in 4 registers
// so a lane ends up with 4 consecutive m of one output o: one 128-bit store.
//
// One workgroup (4 waves) owns 64 m x 16 n; wave w owns the 4 n  4w..4w+3  and all
// 64 m, i.e. 16 row blocks of 16 m, each with COLUMN_BLOCKS accumulator quads.
#pragma once

#include "norm_gradient.hpp"

namespace kmc {

typedef float mfma_float4 __attribute__((ext_vector_type(4)));

constexpr int NGM_TILE_M = 64;
constexpr int NGM_TILE_N = 16;
constexpr int NGM_TILE_K = 16;
constexpr int NGM_THREADS = 256;
// [k][m] with a pitch of 80 floats: the 4 k-rows a wave reads at once land in 4
// disjoint groups of 16 banks.
constexpr int NGM_PITCH_A = 80;
constexpr int NGM_PITCH_B = 16;

// K_TAIL = false: K is a multiple of the slice depth, no term needs a select.
template <int NORM, int COLUMN_BLOCKS, bool K_TAIL>
__global__ __launch_bounds__(NGM_THREADS) void norm_kernel_gradient_mfma(const NormGradientArgs args)
{
    constexpr int O_TILE = 16 * COLUMN_BLOCKS;
    __shared__ __attribute__((aligned(16))) float lds_a[2 * NGM_TILE_K * NGM_PITCH_A];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * NGM_TILE_K * NGM_PITCH_B];
    __shared__ __attribute__((aligned(16))) float lds_c[2 * NGM_TILE_K * O_TILE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int q = lane >> 4;     // k inside a chunk of 4 (operands), row quad (result)
    const int r = lane & 15;     // row m (operand A) / column o (operand B, result)
    const int batch = blockIdx.z / args.o_chunks;
    const int o0 = (blockIdx.z % args.o_chunks) * O_TILE;
    const int m0 = blockIdx.x * NGM_TILE_M;
    const int n0 = blockIdx.y * NGM_TILE_N;

    const float *a_base = args.a + batch * args.a_bs;
    const float *b_base = args.b + batch * args.b_bs;
    const float *c_base = args.c + batch * args.c_bs;
    const float *d_base = args.d + batch * args.d_bs;
    float *e_base = args.e + batch * args.e_bs;

    float p_minus_1 = 0.0f;
    if (NORM == NORM_P) p_minus_1 = (args.p ? args.p[batch * args.p_bs] : args.p_value) - 1.0f;

    // Staging roles: every lane one float4 of A (k = tid/16, m = 4*(tid%16)); lanes
    // 0..63 one float4 of B (n = tid/4, k = 4*(tid%4)); lanes 64..64+4*O_TILE-1 one
    // float4 of C (o = (tid-64)/4, k = 4*(tid%4)).
    const int a_k = tid >> 4, a_m = (tid & 15) * 4;
    const bool stages_b = tid < 64;
    const bool stages_c = tid >= 64 && tid < 64 + 4 * O_TILE;
    const int bc_row = (stages_b ? tid : tid - 64) >> 2, bc_k = (tid & 3) * 4;
    const float *a_ptr = a_base + (i64)a_k * args.a_ld + m0 + a_m;
    const float *b_ptr = b_base + (i64)(n0 + bc_row) * args.b_ld + bc_k;
    const float *c_ptr = c_base + (i64)(o0 + bc_row) * args.c_ld + bc_k;
    const int a_m_valid = args.m - (m0 + a_m);
    const bool b_row_valid = stages_b && n0 + bc_row < args.n;
    const bool c_row_valid = stages_c && o0 + bc_row < args.o;

    // Interior workgroup with 16-byte aligned operands and K a multiple of the
    // slice depth: plain 128-bit loads, nothing to predicate, so the loads of the
    // next slice stay in flight while the current one is consumed.
    const bool fast = args.a_vec && args.b_vec && args.c_vec && args.k % 16 == 0 && m0 + NGM_TILE_M <= args.m &&
                      n0 + NGM_TILE_N <= args.n && o0 + O_TILE <= args.o;
    const float *bc_ptr = stages_b ? b_ptr : c_ptr;
    const bool stages_bc = stages_b || stages_c;
    float4 stage_a, stage_bc;
    auto fetch = [&](int k0) {
        if (fast) {
            stage_a = *reinterpret_cast<const float4 *>(a_ptr + (i64)k0 * args.a_ld);
            if (stages_bc) stage_bc = *reinterpret_cast<const float4 *>(bc_ptr + k0);
            return;
        }
        const int k_left = args.k - k0;
        stage_a = a_k < k_left ? load4_guarded(a_ptr + (i64)k0 * args.a_ld, a_m_valid, args.a_vec)
                               : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        stage_bc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (b_row_valid) stage_bc = load4_guarded(b_ptr + k0, k_left - bc_k, args.b_vec);
        if (c_row_valid) stage_bc = load4_guarded(c_ptr + k0, k_left - bc_k, args.c_vec);
    };
    auto commit = [&](int buffer) {
        *reinterpret_cast<float4 *>(lds_a + (buffer * NGM_TILE_K + a_k) * NGM_PITCH_A + a_m) = stage_a;
        if (stages_b) {
            float *dst = lds_b + (buffer * NGM_TILE_K + bc_k) * NGM_PITCH_B + bc_row;
            dst[0] = gradient_operand<NORM>(stage_bc.x);
            dst[NGM_PITCH_B] = gradient_operand<NORM>(stage_bc.y);
            dst[2 * NGM_PITCH_B] = gradient_operand<NORM>(stage_bc.z);
            dst[3 * NGM_PITCH_B] = gradient_operand<NORM>(stage_bc.w);
        } else if (stages_c) {
            float *dst = lds_c + (buffer * NGM_TILE_K + bc_k) * O_TILE + bc_row;
            dst[0] = stage_bc.x; dst[O_TILE] = stage_bc.y; dst[2 * O_TILE] = stage_bc.z; dst[3 * O_TILE] = stage_bc.w;
        }
    };

    // D[n, m] of the 16 row blocks: row block (mb, nb) covers m0 + 16 mb + r, n0 + 4 wave + nb.
    float dval[4][4];   // [nb][mb]
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int n = n0 + wave * 4 + nb;
#pragma unroll
        for (int mb = 0; mb < 4; mb++) {
            const int m = m0 + mb * 16 + r;
            dval[nb][mb] = gradient_operand<NORM>((n < args.n && m < args.m) ? d_base[(i64)n * args.d_ld + m] : 0.0f);
        }
    }

    mfma_float4 acc[4][4][COLUMN_BLOCKS];   // [nb][mb][column block]
#pragma unroll
    for (int nb = 0; nb < 4; nb++)
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int cb = 0; cb < COLUMN_BLOCKS; cb++) acc[nb][mb][cb] = mfma_float4{0.0f, 0.0f, 0.0f, 0.0f};

    const int k_slices = (args.k + NGM_TILE_K - 1) / NGM_TILE_K;
    if (k_slices > 0) {
        fetch(0);
        commit(0);
        __syncthreads();
    }

    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        const bool has_next = slice + 1 < k_slices;
        if (has_next) fetch((slice + 1) * NGM_TILE_K);

        const float *sa = lds_a + cur * NGM_TILE_K * NGM_PITCH_A + q * NGM_PITCH_A + r;
        const float *sb = lds_b + cur * NGM_TILE_K * NGM_PITCH_B + q * NGM_PITCH_B + wave * 4;
        const float *sc = lds_c + cur * NGM_TILE_K * O_TILE + q * O_TILE + r;
        // k that exist in this slice, relative to this lane's k inside each chunk:
        // chunk c supplies k = 4 c + q, which is real when 4 c + q < k_here.
        const int k_here = min(NGM_TILE_K, args.k - slice * NGM_TILE_K);
#pragma unroll
        for (int chunk = 0; chunk < NGM_TILE_K / 4; chunk++) {
            float fa[4], fb[4], fc[COLUMN_BLOCKS];
#pragma unroll
            for (int mb = 0; mb < 4; mb++) fa[mb] = sa[chunk * 4 * NGM_PITCH_A + mb * 16];
#pragma unroll
            for (int nb = 0; nb < 4; nb++) fb[nb] = sb[chunk * 4 * NGM_PITCH_B + nb];
#pragma unroll
            for (int cb = 0; cb < COLUMN_BLOCKS; cb++) fc[cb] = sc[chunk * 4 * O_TILE + cb * 16];
            // A padded k must contribute exactly 0: g(d - 0) can be inf for p < 1.
            const bool k_real = chunk * 4 + q < k_here;
#pragma unroll
            for (int nb = 0; nb < 4; nb++)
#pragma unroll
                for (int mb = 0; mb < 4; mb++) {
                    float t = gradient_term<NORM>(fa[mb], dval[nb][mb], fb[nb], p_minus_1);
                    if (K_TAIL) t = k_real ? t : 0.0f;
#pragma unroll
                    for (int cb = 0; cb < COLUMN_BLOCKS; cb++)
                        acc[nb][mb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(t, fc[cb], acc[nb][mb][cb], 0, 0, 0);
                }
            // Keeps the scheduler from hoisting the operand reads of later chunks above
            // this one: with them hoisted the kernel needs 136 registers, without 128,
            // which is the step from 3 to 4 waves per SIMD (10.2 -> 9.95 ms at the
            // benchmark shape, same board).
            __builtin_amdgcn_sched_barrier(0);
        }

        if (has_next) commit(cur ^ 1);
        __syncthreads();
    }

    // Store E[o, n, m .. m+3]: this lane holds column o0 + 16 cb + r, rows 4 q .. 4 q + 3.
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int n = n0 + wave * 4 + nb;
        if (n >= args.n) continue;
#pragma unroll
        for (int cb = 0; cb < COLUMN_BLOCKS; cb++) {
            const int o = o0 + cb * 16 + r;
            if (o >= args.o) continue;
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
                const int m = m0 + mb * 16 + q * 4;
                const int m_valid = args.m - m;
                float *dst = e_base + (i64)o * args.e_ld_o + (i64)n * args.e_ld_n + m;
                const mfma_float4 v = acc[nb][mb][cb];
                if (args.e_vec && m_valid >= 4) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (i < m_valid) dst[i] = v[i];
                }
            }
        }
    }
}

}  // namespace kmc
