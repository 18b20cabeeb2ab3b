// Fused kernel-gradient contraction for gfx950:
//
//   E[m, n, o, l] = sum_k C[o,k,l] * A[m,k,l] * g( D[m,n,l] - B[n,k,l] )
//   g(x) = copysign(1, x)              (L1)
//          x                           (L2, no factor 2)
//          copysign(1, x) |x|^(p-1)    (P)
//
// Replaces the reference's cute_norm_kernel_gradient
// (include/p_norm_gradient.cuh:407-497).  Layouts are the reference's: A[k,m]
// and D[n,m] and E[o,n,m] have m contiguous, B[n,k] and C[o,k] have k
// contiguous.
//
// One workgroup of 256 lanes owns 64 (m) x 32 (n) x O_TILE outputs and walks K
// in slices of 16.  Each lane owns 4 (m) x 2 (n) x O_TILE accumulators, so the
// expensive part of the inner loop, g(d - b) * a, is computed once per (m,n,k)
// and reused for all O_TILE outputs -- the trick the reference documents at
// include/p_norm_gradient.cuh:368-372 -- while O_TILE is chosen to fit the
// caller's O (4, 8 or 16) instead of a fixed 32, so O = 16 wastes nothing.
#pragma once

#include "device_common.hpp"

namespace kmc {

struct NormGradientArgs {
    int m, n, o, k, l;
    const float *a; i64 a_ld, a_bs;
    const float *b; i64 b_ld, b_bs;
    const float *c; i64 c_ld, c_bs;
    const float *d; i64 d_ld, d_bs;
    float *e; i64 e_ld_n, e_ld_o, e_bs;
    const float *p; i64 p_bs; float p_value;
    int o_chunks;                  // ceil(o / O_TILE): blockIdx.z = l * o_chunks + chunk
    int a_vec, b_vec, c_vec, e_vec;  // 128-bit access allowed for that operand
};

constexpr int NG_TILE_M = 64;
constexpr int NG_TILE_N = 32;
constexpr int NG_TILE_K = 16;
constexpr int NG_THREADS = 256;
constexpr int NG_PITCH_A = NG_TILE_M + 4;
constexpr int NG_PITCH_B = NG_TILE_N + 4;

template <int NORM>
__device__ __forceinline__ float gradient_weight(float diff, float p_minus_1)
{
    // include/p_norm_gradient.cuh:377-387
    if (NORM == NORM_L2) return diff;
    if (NORM == NORM_L1) return signum(diff);
    // |diff|^(p-1) is never negative, so multiplying by copysign(1, diff) is a sign transfer:
    // one instruction instead of two
    return __builtin_copysignf(fast_pow_abs(__builtin_fabsf(diff), p_minus_1), diff);
}

// For the L1 norm only the sign of d - b is needed, and copysign(1, d - b) is
// negative exactly when d < b or (d, b) = (-0, +0).  Mapping a float to the
// integer  bits ^ ((bits >> 31) & 0x7fffffff)  turns that rule into one signed
// integer comparison (-0 maps to -1, +0 to 0, everything else keeps its order),
// so D and B are held as such keys and a term costs two instructions, compare
// and select, instead of subtract, sign transfer and multiply.
__device__ __forceinline__ float sign_order_key(float x)
{
    const int bits = __float_as_int(x);
    return __int_as_float(bits ^ ((bits >> 31) & 0x7fffffff));
}

// What D and B are replaced by when they enter registers / LDS.
template <int NORM>
__device__ __forceinline__ float gradient_operand(float x)
{
    return NORM == NORM_L1 ? sign_order_key(x) : x;
}

// a * g(d - b) with d and b prepared by gradient_operand.
template <int NORM>
__device__ __forceinline__ float gradient_term(float a, float d, float b, float p_minus_1)
{
    if (NORM == NORM_L1) return __float_as_int(d) < __float_as_int(b) ? -a : a;
    return a * gradient_weight<NORM>(d - b, p_minus_1);
}

template <int NORM, int O_TILE>
__global__ __launch_bounds__(NG_THREADS) void norm_kernel_gradient(const NormGradientArgs args)
{
    // [buffer][k][row]; the extra row per array is the target of the last,
    // unused fragment prefetch of a slice.
    __shared__ __attribute__((aligned(16))) float lds_a[2 * NG_TILE_K * NG_PITCH_A + NG_PITCH_A];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * NG_TILE_K * NG_PITCH_B + NG_PITCH_B];
    __shared__ __attribute__((aligned(16))) float lds_c[2 * NG_TILE_K * O_TILE + O_TILE];

    const int tid = threadIdx.x;
    const int tx = tid & 15;   // m direction: 4 consecutive m per lane
    const int ty = tid >> 4;   // n direction: 2 consecutive n per lane
    const int batch = blockIdx.z / args.o_chunks;
    const int o0 = (blockIdx.z % args.o_chunks) * O_TILE;
    const int m0 = blockIdx.x * NG_TILE_M;
    const int n0 = blockIdx.y * NG_TILE_N;

    const float *a_base = args.a + batch * args.a_bs;
    const float *b_base = args.b + batch * args.b_bs;
    const float *c_base = args.c + batch * args.c_bs;
    const float *d_base = args.d + batch * args.d_bs;
    float *e_base = args.e + batch * args.e_bs;

    float p_minus_1 = 0.0f;
    if (NORM == NORM_P) p_minus_1 = (args.p ? args.p[batch * args.p_bs] : args.p_value) - 1.0f;

    // Who stages what: all lanes one float4 of A (k = tid/16, m = 4*(tid%16));
    // lanes 0..127 one float4 of B (n = tid/4, k = 4*(tid%4)); lanes 128.. one
    // float4 of C (o = (tid-128)/4, k = 4*(tid%4)).
    const int a_k = tid >> 4, a_m = (tid & 15) * 4;
    const bool stages_b = tid < 128;
    const int bc_row = (stages_b ? tid : tid - 128) >> 2, bc_k = (tid & 3) * 4;
    const bool stages_c = !stages_b && bc_row < O_TILE;

    const float *a_ptr = a_base + (i64)a_k * args.a_ld + m0 + a_m;
    const float *b_ptr = b_base + (i64)(n0 + bc_row) * args.b_ld + bc_k;
    const float *c_ptr = c_base + (i64)(o0 + bc_row) * args.c_ld + bc_k;
    const int a_m_valid = args.m - (m0 + a_m);
    const bool b_row_valid = stages_b && n0 + bc_row < args.n;
    const bool c_row_valid = stages_c && o0 + bc_row < args.o;

    // Interior workgroup with 16-byte aligned operands and K a multiple of the
    // slice depth: plain 128-bit loads, nothing to predicate, so the loads of the
    // next slice stay in flight while the current one is consumed.
    const bool fast = args.a_vec && args.b_vec && args.c_vec && args.k % 16 == 0 && m0 + NG_TILE_M <= args.m &&
                      n0 + NG_TILE_N <= args.n && o0 + O_TILE <= args.o;
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
        *reinterpret_cast<float4 *>(lds_a + (buffer * NG_TILE_K + a_k) * NG_PITCH_A + a_m) = stage_a;
        if (stages_b) {
            float *dst = lds_b + (buffer * NG_TILE_K + bc_k) * NG_PITCH_B + bc_row;
            dst[0] = gradient_operand<NORM>(stage_bc.x);
            dst[NG_PITCH_B] = gradient_operand<NORM>(stage_bc.y);
            dst[2 * NG_PITCH_B] = gradient_operand<NORM>(stage_bc.z);
            dst[3 * NG_PITCH_B] = gradient_operand<NORM>(stage_bc.w);
        } else if (stages_c) {
            float *dst = lds_c + (buffer * NG_TILE_K + bc_k) * O_TILE + bc_row;
            dst[0] = stage_bc.x; dst[O_TILE] = stage_bc.y; dst[2 * O_TILE] = stage_bc.z; dst[3 * O_TILE] = stage_bc.w;
        }
    };

    // D values of this lane's 4 x 2 outputs stay in registers for the whole walk.
    float dval[2][4];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int n = n0 + ty * 2 + j;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = m0 + tx * 4 + i;
            dval[j][i] = gradient_operand<NORM>((n < args.n && m < args.m) ? d_base[(i64)n * args.d_ld + m] : 0.0f);
        }
    }

    float acc[2][4][O_TILE];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int o = 0; o < O_TILE; o++) acc[j][i][o] = 0.0f;

    const int k_slices = (args.k + NG_TILE_K - 1) / NG_TILE_K;
    if (k_slices > 0) {
        fetch(0);
        commit(0);
        __syncthreads();
    }

    auto step = [&](const float4 &fa, const float2 &fb, const float (&fc)[O_TILE]) {
        const float av[4] = {fa.x, fa.y, fa.z, fa.w};
        const float bv[2] = {fb.x, fb.y};
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float t = gradient_term<NORM>(av[i], dval[j][i], bv[j], p_minus_1);
#pragma unroll
                for (int o = 0; o < O_TILE; o++) acc[j][i][o] += fc[o] * t;
            }
    };
    auto read_c = [&](float (&fc)[O_TILE], const float *src) {
        if (O_TILE % 4 != 0) {     // rows of O_TILE floats are not 16-byte aligned: scalar (broadcast) reads
#pragma unroll
            for (int o = 0; o < O_TILE; o++) fc[o] = src[o];
            return;
        }
#pragma unroll
        for (int q = 0; q < O_TILE / 4; q++) {
            const float4 v = *reinterpret_cast<const float4 *>(src + 4 * q);
            fc[4 * q] = v.x; fc[4 * q + 1] = v.y; fc[4 * q + 2] = v.z; fc[4 * q + 3] = v.w;
        }
    };

    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        const bool has_next = slice + 1 < k_slices;
        if (has_next) fetch((slice + 1) * NG_TILE_K);

        const float *sa = lds_a + cur * NG_TILE_K * NG_PITCH_A + tx * 4;
        const float *sb = lds_b + cur * NG_TILE_K * NG_PITCH_B + ty * 2;
        const float *sc = lds_c + cur * NG_TILE_K * O_TILE;
        const int k_here = min(NG_TILE_K, args.k - slice * NG_TILE_K);
        if (k_here == NG_TILE_K) {
            // Full slice: two k-steps per trip with the next fragments requested
            // before the current ones are consumed.  Kept rolled, and for the L1 and
            // L2 norms fenced so that the scheduler leaves each group of reads one
            // step ahead of its use instead of gathering all reads of a trip at the
            // top, which exposes the LDS latency once per trip (O = 8, same board:
            // 7.68 -> 7.38 ms; the fractional norm is 3 % faster without fences).
            float4 fa0 = *reinterpret_cast<const float4 *>(sa);
            float2 fb0 = *reinterpret_cast<const float2 *>(sb);
            float fc0[O_TILE], fc1[O_TILE];
            read_c(fc0, sc);
#pragma unroll 1
            for (int kk = 0; kk < NG_TILE_K; kk += 2) {
                const float4 fa1 = *reinterpret_cast<const float4 *>(sa + (kk + 1) * NG_PITCH_A);
                const float2 fb1 = *reinterpret_cast<const float2 *>(sb + (kk + 1) * NG_PITCH_B);
                read_c(fc1, sc + (kk + 1) * O_TILE);
                if (NORM != NORM_P) __builtin_amdgcn_sched_barrier(0);
                step(fa0, fb0, fc0);
                if (NORM != NORM_P) __builtin_amdgcn_sched_barrier(0);
                // kk + 2 == 16 reads the first row of the other buffer / the pad
                // row; those values are never used.
                fa0 = *reinterpret_cast<const float4 *>(sa + (kk + 2) * NG_PITCH_A);
                fb0 = *reinterpret_cast<const float2 *>(sb + (kk + 2) * NG_PITCH_B);
                read_c(fc0, sc + (kk + 2) * O_TILE);
                if (NORM != NORM_P) __builtin_amdgcn_sched_barrier(0);
                step(fa1, fb1, fc1);
                if (NORM != NORM_P) __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            // K tail: only the k that exist, so that g(d - 0) * 0 of a padded k
            // can never produce inf * 0.
#pragma unroll 1
            for (int kk = 0; kk < k_here; kk++) {
                const float4 fa = *reinterpret_cast<const float4 *>(sa + kk * NG_PITCH_A);
                const float2 fb = *reinterpret_cast<const float2 *>(sb + kk * NG_PITCH_B);
                float fc[O_TILE];
                read_c(fc, sc + kk * O_TILE);
                step(fa, fb, fc);
            }
        }

        if (has_next) commit(cur ^ 1);
        __syncthreads();
    }

    // Store E[o, n, m..m+3] (include/p_norm_gradient.cuh:398-404).
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int n = n0 + ty * 2 + j;
        if (n >= args.n) continue;
        const int m = m0 + tx * 4;
        const int m_valid = args.m - m;
#pragma unroll
        for (int o = 0; o < O_TILE; o++) {
            if (o0 + o >= args.o) break;
            float *dst = e_base + (i64)(o0 + o) * args.e_ld_o + (i64)n * args.e_ld_n + m;
            if (args.e_vec && m_valid >= 4) {
                *reinterpret_cast<float4 *>(dst) = make_float4(acc[j][0][o], acc[j][1][o], acc[j][2][o], acc[j][3][o]);
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (i < m_valid) dst[i] = acc[j][i][o];
            }
        }
    }
}

}  // namespace kmc
