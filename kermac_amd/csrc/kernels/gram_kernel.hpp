// Optional matrix-core path for the squared-difference descriptors (L2 norm,
// Laplace-L2, Gaussian):
//
//   sum_k (b[n,k] - a[m,k])^2  =  |a_m|^2 + |b_n|^2 - 2 * sum_k a[m,k] * b[n,k]
//
// The cross term is a plain GEMM and runs as v_mfma_f32_32x32x2_f32 on the matrix
// cores; the row norms are accumulated on the side from the values each lane
// stages into LDS anyway.  The reference has no such path (its kernels are SIMT
// only, include/build_a_kernel.cuh:339-370); it is offered as an opt-in because
// the expansion cancels: the absolute error of the result is about
// sqrt(K) * 2^-24 * (|a|^2 + |b|^2), which is harmless when the distance is
// comparable to the norms and ruinous for near-duplicate points.
//
// Therefore every workgroup checks its own tile: if any element has
//   d^2 < gram_trust * (|a_m|^2 + |b_n|^2)
// the tile is not trusted; the workgroup stamps BK_REPAIR_MARKER into the tile's
// first element and the host launches the direct kernel (build_kernel.hpp) in
// repair mode right after, which recomputes exactly the stamped tiles with the
// subtract-square-accumulate arithmetic.  Trusted tiles keep a relative error of
// at most about sqrt(K) * 2^-24 / gram_trust on d^2.
//
// Tiling: workgroup 256 lanes = 2 x 2 waves, tile 128 x 128, K slices of 16 staged
// exactly like the direct kernel (same loaders, same LDS layout).  A wave owns
// 64 x 64 as 2 x 2 MFMA tiles of 32 x 32.  Operand layouts (lane = 32 h + i):
//   A (32 x 2): lane supplies A[row i][k h];  B (2 x 32): lane supplies B[k h][column i]
//   D (32 x 32): register v of the lane is D[row 8 (v/4) + 4 h + v%4][column i]
// With a on the row side a lane holds 4 x 4 consecutive m of one n: 128-bit stores.
#pragma once

#include "build_kernel.hpp"

namespace kmc {

typedef float gram_float16 __attribute__((ext_vector_type(16)));

// norm[row] = sum over everything the workgroup staged for that row of `square`.
// `partial` is scratch for lanes_per_row() x 128 floats.  Contains one barrier;
// the caller adds another before reading `norm`.
template <int MODE>
__device__ __forceinline__ void row_norms(
    const TileLoader<MODE> &loader, const float (&square)[8], float *partial, float *norm, int tid)
{
    const int share = TileLoader<MODE>::share_index(tid);
#pragma unroll
    for (int s = 0; s < 8; s++) {
        // the first register of each distinct row collects the others of that row
        bool first = true;
#pragma unroll
        for (int e = 0; e < s; e++)
            if (TileLoader<MODE>::row_offset_of(e) == TileLoader<MODE>::row_offset_of(s)) first = false;
        if (!first) continue;
        float sum = square[s];
#pragma unroll
        for (int e = s + 1; e < 8; e++)
            if (TileLoader<MODE>::row_offset_of(e) == TileLoader<MODE>::row_offset_of(s)) sum += square[e];
        partial[share * BK_TILE_M + loader.lane_row + TileLoader<MODE>::row_offset_of(s)] = sum;
    }
    __syncthreads();
    if (tid < BK_TILE_M) {
        float total = 0.0f;
#pragma unroll
        for (int part = 0; part < TileLoader<MODE>::lanes_per_row(); part++) total += partial[part * BK_TILE_M + tid];
        norm[tid] = total;
    }
}

// The K walk of one tile: stage slices through LDS (double buffered, loads of
// slice t+1 in flight while slice t is consumed), feed the matrix cores, and keep
// per-register sums of squares of everything staged.  FULL = no load needs a
// predicate.  Ends with a barrier.
template <int LOAD_A, int LOAD_B, bool FULL>
__device__ __forceinline__ void gram_walk(
    gram_float16 (&acc)[2][2], float (&square_a)[8], float (&square_b)[8],
    TileLoader<LOAD_A> &load_a, TileLoader<LOAD_B> &load_b, float *lds_a, float *lds_b,
    const float *frag_a, const float *frag_b, int k_total, int m_valid, int n_valid)
{
    const int k_slices = (k_total + BK_TILE_K - 1) / BK_TILE_K;
    const int k_tail = k_total - (k_slices - 1) * BK_TILE_K;
    float stage_a[8], stage_b[8];

    auto fetch = [&](int slice) {
        if (FULL) {
            load_a.load_full(stage_a);
            load_b.load_full(stage_b);
        } else {
            const int kv = slice + 1 == k_slices ? k_tail : BK_TILE_K;
            load_a.load_edge(stage_a, m_valid, kv);    // zero fill: adds 0 to norms and dot products
            load_b.load_edge(stage_b, n_valid, kv);
        }
    };
    auto commit = [&](int buffer) {
#pragma unroll
        for (int s = 0; s < 8; s++) {
            square_a[s] += stage_a[s] * stage_a[s];
            square_b[s] += stage_b[s] * stage_b[s];
        }
        load_a.store(lds_a + buffer * BK_LDS_SLICE, stage_a);
        load_b.store(lds_b + buffer * BK_LDS_SLICE, stage_b);
    };

    if (k_slices > 0) {
        fetch(0);
        commit(0);
    }
    __syncthreads();

    for (int slice = 0; slice < k_slices; slice++) {
        const int cur = slice & 1;
        const bool has_next = slice + 1 < k_slices;
        if (has_next) {
            load_a.advance();
            load_b.advance();
            fetch(slice + 1);
        }
        const float *sa = frag_a + cur * BK_LDS_SLICE;
        const float *sb = frag_b + cur * BK_LDS_SLICE;
        // Operand double buffer: the LDS reads of pair p+1 are issued before the
        // four MFMAs of pair p, so the matrix pipe never waits for LDS latency.
        float fa[2][2], fb[2][2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            fa[0][t] = sa[t * 32];
            fb[0][t] = sb[t * 32];
        }
#pragma unroll
        for (int pair = 0; pair < BK_TILE_K / 2; pair++) {
            const int use = pair & 1;
            if (pair + 1 < BK_TILE_K / 2) {
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    fa[use ^ 1][t] = sa[(pair + 1) * 2 * BK_LDS_PITCH + t * 32];
                    fb[use ^ 1][t] = sb[(pair + 1) * 2 * BK_LDS_PITCH + t * 32];
                }
            }
            // Keep the instruction scheduler from sinking those reads below the
            // MFMAs (it would, to save four registers).
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[use][mt], fb[use][nt], acc[mt][nt], 0, 0, 0);
        }
        if (has_next) commit(cur ^ 1);
        __syncthreads();
    }
}

template <int LOAD_A, int LOAD_B>
__global__ __launch_bounds__(BK_THREADS, 2) void gram_l2_kernel(const BuildKernelArgs args)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * BK_LDS_SLICE];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * BK_LDS_SLICE];
    __shared__ float lds_norm_a[BK_TILE_M];
    __shared__ float lds_norm_b[BK_TILE_N];

    const int tid = threadIdx.x;
    const int batch = blockIdx.y;
    int tile_m, tile_n;
    if (!tile_of_workgroup(args, tile_m, tile_n)) return;
    const int m0 = tile_m * BK_TILE_M;
    const int n0 = tile_n * BK_TILE_N;
    const int m_valid = args.m - m0;
    const int n_valid = args.n - n0;

    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = (wave & 1) * 64;
    const int wave_n = (wave >> 1) * 64;
    const int h = lane >> 5;     // k inside a pair (operands) / row half (result)
    const int i = lane & 31;     // row (operand A) / column (operand B, result)

    TileLoader<LOAD_A> load_a;
    TileLoader<LOAD_B> load_b;
    load_a.init(args.a + batch * args.a_bs, args.a_ld, m0, tid);
    load_b.init(args.b + batch * args.b_bs, args.b_ld, n0, tid);

    float square_a[8], square_b[8];   // running sum of squares of what this lane staged, per register slot
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
    if (m_valid >= BK_TILE_M && n_valid >= BK_TILE_N && args.k % BK_TILE_K == 0) {
        gram_walk<LOAD_A, LOAD_B, true>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, frag_a, frag_b,
                                        args.k, m_valid, n_valid);
    } else {
        gram_walk<LOAD_A, LOAD_B, false>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, frag_a, frag_b,
                                         args.k, m_valid, n_valid);
    }

    // Row norms, summed in a fixed order so that the same point gets the same norm
    // in every workgroup (results are reproducible and x-vs-x matrices symmetric):
    // first the registers of one row inside a lane, then the lanes sharing a row,
    // through the staging memory, which is idle after the last barrier.
    row_norms<LOAD_A>(load_a, square_a, lds_a, lds_norm_a, tid);
    row_norms<LOAD_B>(load_b, square_b, lds_b, lds_norm_b, tid);
    __syncthreads();

    // d^2, trust check, epilogue.
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

    int distrust = 0;
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
        const int n_local = wave_n + nt * 32 + i;
        const float norm_b = lds_norm_b[n_local];
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m_local = wave_m + mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                const float norms = lds_norm_a[m_local] + norm_b;
                float d2 = norms - 2.0f * acc[mt][nt][v];
                // NaN compares false: a NaN result is stored as is, not repaired.
                if (m_local < m_valid && n_local < n_valid && d2 < args.gram_trust * norms) distrust = 1;
                d2 = fmaxf(d2, 0.0f);
                float value = epilogue_value(d2, outer_power, kernel_type, p_outer, neg_gamma, args.epsilon);
                if (regularize && args.reg_off_x + m0 + m_local == args.reg_off_y + n0 + n_local) value = diagonal_value;
                acc[mt][nt][v] = value;
            }
    }
    const bool repair = __syncthreads_or(distrust) != 0;

    float *c_tile = args.c + batch * args.c_bs;
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
        const int n_local = wave_n + nt * 32 + i;
        if (n_local >= n_valid) continue;
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int m_local = wave_m + mt * 32 + 8 * g + 4 * h;
                float v4[4] = {acc[mt][nt][4 * g], acc[mt][nt][4 * g + 1], acc[mt][nt][4 * g + 2], acc[mt][nt][4 * g + 3]};
                if (repair && m_local == 0 && n_local == 0) v4[0] = __uint_as_float(BK_REPAIR_MARKER);
                float *dst = c_tile + (i64)(n0 + n_local) * args.c_ld + m0 + m_local;
                if (args.c_vec && m_local + 3 < m_valid) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(v4[0], v4[1], v4[2], v4[3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (m_local + e < m_valid) dst[e] = v4[e];
                }
            }
    }
}

}  // namespace kmc
