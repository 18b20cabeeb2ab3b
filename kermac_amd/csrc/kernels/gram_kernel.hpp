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
// Tiling: workgroup 256 lanes = 2 x 2 waves, tile 128 x 128, K staged through LDS
// with the loaders and the layout of the direct kernel, two of its slices at a time.  A wave owns
// 64 x 64 as 2 x 2 MFMA tiles of 32 x 32.  Operand layouts (lane = 32 h + i):
//   A (32 x 2): lane supplies A[row i][k h];  B (2 x 32): lane supplies B[k h][column i]
//   D (32 x 32): register v of the lane is D[row 8 (v/4) + 4 h + v%4][column i]
// With a on the row side a lane holds 4 x 4 consecutive m of one n: 128-bit stores.
#pragma once

#include "build_kernel.hpp"

namespace kmc {

typedef float gram_float16 __attribute__((ext_vector_type(16)));

template <bool B>
struct GramSwitch {
    static constexpr bool value = B;
};

// The centre of batch entry `batch` if it is to be subtracted, else null.  The vector (k floats,
// padded with zeros to a multiple of GRAM_CENTRE_PAD) is followed by a flag: 0 says that the
// centre is too close to the origin to matter (kmc_sample_mean decides), and the walk then leaves
// the subtraction out.  Uniform over the workgroup.
__device__ __forceinline__ const float *centre_to_subtract(const BuildKernelArgs &args, int batch)
{
    if (!args.centre) return nullptr;
    const float *centre = args.centre + batch * args.centre_bs;
    const int padded = (args.k + GRAM_CENTRE_PAD - 1) / GRAM_CENTRE_PAD * GRAM_CENTRE_PAD;
    return centre[padded] != 0.0f ? centre : nullptr;
}

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

// Loader slices (of BK_TILE_K = 16 k) per pipeline stage.  One stage is what sits
// between two barriers and what the global loads run ahead by: at 32 k a stage
// keeps the matrix pipe busy for about 1.8 us, longer than a global load that
// misses the L2 takes, and there are half as many barriers as with 16.
#ifndef GRAM_DEPTH
#define GRAM_DEPTH 1
#endif
#ifndef GRAM_WAVES
#define GRAM_WAVES 4
#endif
constexpr int GRAM_STAGE_K = GRAM_DEPTH * BK_TILE_K;
constexpr int GRAM_STAGE_FLOATS = GRAM_DEPTH * BK_LDS_SLICE;   // per operand and buffer

// The K walk of one tile: stage slices through LDS (double buffered, loads of
// stage t+1 in flight while stage t is consumed), feed the matrix cores, and keep
// per-register sums of squares of everything staged.  FULL = no load needs a
// predicate.  Ends with a barrier.
template <int LOAD_A, int LOAD_B, bool FULL, bool CENTRED>
__device__ __forceinline__ void gram_walk(
    gram_float16 (&acc)[2][2], float (&square_a)[8], float (&square_b)[8],
    TileLoader<LOAD_A> &load_a, TileLoader<LOAD_B> &load_b, float *lds_a, float *lds_b,
    const float *frag_a, const float *frag_b, int k_total, int m_valid, int n_valid, const float *centre)
{
    const int k_slices = (k_total + BK_TILE_K - 1) / BK_TILE_K;
    const int k_tail = k_total - (k_slices - 1) * BK_TILE_K;
    const int stages = (k_slices + GRAM_DEPTH - 1) / GRAM_DEPTH;
    float stage_a[GRAM_DEPTH][8], stage_b[GRAM_DEPTH][8];
    // CENTRED: `centre` is subtracted from everything that is staged: distances do not
    // change, but norms and dot products shrink to the spread of the data around that point, and
    // with them the error of |a|^2 + |b|^2 - 2 a.b.  Rows past M / N become -centre; they are
    // never stored.  Both loaders of one mode hold the same k per register.
    float centre_a[GRAM_DEPTH][8], centre_b[GRAM_DEPTH][8];
    const float *next_centre = centre;

    // The loaders point at the next slice to fetch and move on after every fetch.
    auto fetch = [&](int stage) {
#pragma unroll
        for (int d = 0; d < GRAM_DEPTH; d++) {
            if (FULL) {
                load_a.load_full(stage_a[d]);
                load_b.load_full(stage_b[d]);
            } else {
                const int slice = stage * GRAM_DEPTH + d;
                // slices past the end: k_valid 0, nothing is dereferenced, zeros are staged
                const int kv = slice + 1 < k_slices ? BK_TILE_K : (slice + 1 == k_slices ? k_tail : 0);
                load_a.load_edge(stage_a[d], m_valid, kv);    // zero fill: adds 0 to norms and dot products
                load_b.load_edge(stage_b[d], n_valid, kv);
            }
            if (CENTRED) {
                load_a.load_centre(centre_a[d], next_centre);
                if (LOAD_A != LOAD_B) load_b.load_centre(centre_b[d], next_centre);
                next_centre += BK_TILE_K;
            }
            load_a.advance();
            load_b.advance();
        }
    };
    auto commit = [&](int buffer) {
#pragma unroll
        for (int d = 0; d < GRAM_DEPTH; d++) {
#pragma unroll
            for (int s = 0; s < 8; s++) {
                if (CENTRED) {
                    stage_a[d][s] -= centre_a[d][s];
                    stage_b[d][s] -= LOAD_A != LOAD_B ? centre_b[d][s] : centre_a[d][s];
                }
                square_a[s] += stage_a[d][s] * stage_a[d][s];
                square_b[s] += stage_b[d][s] * stage_b[d][s];
            }
            load_a.store(lds_a + buffer * GRAM_STAGE_FLOATS + d * BK_LDS_SLICE, stage_a[d]);
            load_b.store(lds_b + buffer * GRAM_STAGE_FLOATS + d * BK_LDS_SLICE, stage_b[d]);
        }
    };

    if (stages > 0) {
        fetch(0);
        commit(0);
    }
    __syncthreads();

    for (int stage = 0; stage < stages; stage++) {
        const int cur = stage & 1;
        const bool has_next = stage + 1 < stages;
        if (has_next) fetch(stage + 1);
        const float *sa = frag_a + cur * GRAM_STAGE_FLOATS;
        const float *sb = frag_b + cur * GRAM_STAGE_FLOATS;
        // Operand double buffer: the LDS reads of pair p+1 are issued before the
        // four MFMAs of pair p, so the matrix pipe never waits for LDS latency.
        float fa[2][2], fb[2][2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            fa[0][t] = sa[t * 32];
            fb[0][t] = sb[t * 32];
        }
#pragma unroll
        for (int pair = 0; pair < GRAM_STAGE_K / 2; pair++) {
            const int use = pair & 1;
            if (pair + 1 < GRAM_STAGE_K / 2) {
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

// CENTRED: args.centre is subtracted from both operands while they are staged.
template <int LOAD_A, int LOAD_B, bool CENTRED = false>
__global__ __launch_bounds__(BK_THREADS, GRAM_WAVES) void gram_l2_kernel(const BuildKernelArgs args)
{
    __shared__ __attribute__((aligned(16))) float lds_a[2 * GRAM_STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * GRAM_STAGE_FLOATS];
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

    // The sample of the result says that the repair launch would redo (nearly) every tile: stamp this one
    // and leave (uniform over the launch: every workgroup reads the same words).
    if (args.sample && sample_leaves_it_to_the_direct_kernel(args.sample)) {
        if (tid == 0) args.c[batch * args.c_bs + (i64)n0 * args.c_ld + m0] = __uint_as_float(BK_REPAIR_MARKER);
        return;
    }

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
    const float *centre = CENTRED ? centre_to_subtract(args, batch) : nullptr;
    auto walk = [&](auto centred) {
        constexpr bool C = decltype(centred)::value;
        if (m_valid >= BK_TILE_M && n_valid >= BK_TILE_N && args.k % GRAM_STAGE_K == 0) {
            gram_walk<LOAD_A, LOAD_B, true, C>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, frag_a, frag_b, args.k,
                                               m_valid, n_valid, centre);
        } else {
            gram_walk<LOAD_A, LOAD_B, false, C>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, frag_a, frag_b, args.k,
                                                m_valid, n_valid, centre);
        }
    };
    if (CENTRED && centre) walk(GramSwitch<CENTRED>{});
    else walk(GramSwitch<false>{});

    // Row norms, summed in a fixed order so that the same point gets the same norm
    // in every workgroup (results are reproducible and x-vs-x matrices symmetric):
    // first the registers of one row inside a lane, then the lanes sharing a row,
    // through the staging memory, which is idle after the last barrier.
    row_norms<LOAD_A>(load_a, square_a, lds_a, lds_norm_a, tid);
    row_norms<LOAD_B>(load_b, square_b, lds_b, lds_norm_b, tid);
    __syncthreads();

#include "gram_epilogue.inc"
}

}  // namespace kmc
