// Matrix-core path for the squared-difference descriptors with the cross term on
// the bf16 matrix instruction, at fp32 accuracy:
//
//   sum_k (b[n,k] - a[m,k])^2  =  |a_m|^2 + |b_n|^2 - 2 * sum_k a[m,k] * b[n,k]
//
// gfx950 multiplies bf16 matrices 13 times faster than fp32 ones
// (v_mfma_f32_32x32x16_bf16: measured 2.1 PFLOP/s against 155 TFLOP/s for
// v_mfma_f32_32x32x2_f32).  Every fp32 operand is therefore split, once, when it is
// staged, into three bf16 pieces  x = x1 + x2 + x3  (x1 = bf16(x), x2 = bf16(x - x1),
// x3 = bf16(x - x1 - x2); together they carry the 24 bits of x), and the cross term
// is accumulated in fp32 from the six largest of the nine piece products:
//   a1 b1 + (a1 b2 + a2 b1) + (a1 b3 + a3 b1 + a2 b2)
// The three dropped products are below 2^-24 |a| |b|.  Measured error of the dot
// product: 9e-8 |a| |b| for K = 1024, the same as a sequential fp32 sum (with two
// pieces and three products it is 5e-7 and grows as K shrinks, which the trust rule
// below could not absorb).  Six bf16 instructions per 16 k replace eight fp32
// instructions of twice their duration.
//
// Everything around the cross term is that of gram_kernel.hpp: norms accumulated from
// the fp32 values while staging, the per-tile trust check with the repair marker, the
// shared epilogue and stores (gram_epilogue.inc), the tile order of build_kernel.
// The reference has no such path (include/build_a_kernel.cuh:339-370 is SIMT only).
//
// Staging: every lane owns one row of the 128-row panel and one half of a 16-deep K
// slice (k = 8 half .. 8 half + 7).  From a K-major panel (m contiguous) lane t takes
// row t % 128, half t / 128: 8 scalar loads per slice, each one 256 contiguous bytes
// per wave.  From a row-major operand lane t takes row t / 2, half t % 2: two 128-bit
// loads (or 8 scalar ones), 64 contiguous bytes per row.  The lane splits its 8 values and
// writes one 16-byte chunk per piece: LDS holds piece[3][half][row 0..127][8 k] in
// bf16, so both these writes (a wave covers 64 consecutive rows of one half) and the
// operand reads of the matrix instruction (lane 32 h + i reads row i of half h) are
// contiguous across lanes and free of bank conflicts.
//
// Pipeline of one slice s: the raw values of slice s + 2 are requested at its start
// (scalar base addresses, so this costs no vector work), and the values of slice
// s + 1, requested one slice earlier, are split and written to the other LDS buffer
// in the shadow of the 24 matrix instructions of slice s, one part of the split after
// each of them.  One barrier per slice.  Left alone the compiler gathers the matrix
// instructions and the split into two blocks, which serialises them; scheduling
// fences keep them interleaved.
#pragma once

#include "gram_kernel.hpp"

namespace kmc {

typedef __bf16 gram_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 gram_bf16x2 __attribute__((ext_vector_type(2)));
typedef float gram_float2 __attribute__((ext_vector_type(2)));
typedef float gram_float4 __attribute__((ext_vector_type(4)));
typedef unsigned int gram_chunk __attribute__((ext_vector_type(4)));   // 8 bf16 = one 16-byte LDS chunk

#ifndef GB_WAVES
#define GB_WAVES 3      // waves per SIMD the register budget is cut for
#endif

constexpr int GB_PIECES = 3;
constexpr int GB_PANEL_CHUNKS = GB_PIECES * BK_TILE_M * 2;   // 16-byte chunks per operand and buffer

// Addresses are a wave-uniform base (scalar registers, advanced by scalar arithmetic)
// plus a small per-lane offset, so that stepping through K costs no vector work.
template <int MODE>
struct RowOwnerLoader {
    typedef const float __attribute__((address_space(1))) *global_pointer;
    typedef const gram_float4 __attribute__((address_space(1))) *global_quad_pointer;
    static constexpr bool COL = MODE == LOAD_COL_VEC || MODE == LOAD_COL_SCALAR;
    // loads a lane issues per slice: 8 scalars, or two 128-bit loads
    static constexpr int LOADS = MODE == LOAD_ROW_VEC ? 2 : 8;

    const float *base;      // COL: wave-uniform, row 0 of the tile at this wave's K half; ROW: this lane's row
    i64 ld, step;
    int row, half;

    __device__ __forceinline__ void init(const float *origin, i64 ld_, int row0, int tid)
    {
        ld = ld_;
        if (COL) {
            // a wave takes 64 consecutive rows of one K half: each load is 256 contiguous bytes
            row = tid & (BK_TILE_M - 1);
            half = __builtin_amdgcn_readfirstlane(tid >> 7);
            base = origin + (i64)(8 * half) * ld + row0;
            step = (i64)BK_TILE_K * ld;
        } else {
            // neighbouring lanes take the two halves of a row: 64 contiguous bytes per row
            row = tid >> 1;
            half = tid & 1;
            base = origin + (i64)(row0 + row) * ld + 8 * half;
            step = BK_TILE_K;
        }
    }
    __device__ __forceinline__ global_pointer element(int e) const
    {
        if (COL) {
            const float *slice_row = base + (i64)e * ld;
            asm("" : "+s"(slice_row));      // stays a scalar base: the lane's row goes into the load itself
            return (global_pointer)slice_row + (unsigned)row;
        }
        return (global_pointer)(base + e);
    }
    // Load number `which` (0 .. LOADS - 1) of the current slice into r.  With EDGE, rows
    // >= rows_valid and k >= k_valid read as 0 (adds 0 to norms and dot products).
    // QUADS (row-major operands with 128-bit loads, kernels built for a ragged K, where every
    // tile comes through here): a predicated 128-bit load wherever all four k exist.
    template <bool EDGE, bool QUADS = false>
    __device__ __forceinline__ void load_part(float (&r)[8], int which, int rows_valid, int k_valid) const
    {
        if (MODE == LOAD_ROW_VEC && !EDGE) {
            const gram_float4 v = *(global_quad_pointer)element(4 * which);
            r[4 * which] = v.x; r[4 * which + 1] = v.y; r[4 * which + 2] = v.z; r[4 * which + 3] = v.w;
        } else if (MODE == LOAD_ROW_VEC) {
            if (QUADS && k_valid == BK_TILE_K) {      // uniform: every slice but the last of a ragged K
                gram_float4 v = {0.0f, 0.0f, 0.0f, 0.0f};
                if (row < rows_valid) v = *(global_quad_pointer)element(4 * which);
                r[4 * which] = v.x; r[4 * which + 1] = v.y; r[4 * which + 2] = v.z; r[4 * which + 3] = v.w;
            } else {
#pragma unroll
                for (int e = 4 * which; e < 4 * which + 4; e++)
                    r[e] = (row < rows_valid && 8 * half + e < k_valid) ? *element(e) : 0.0f;
            }
        } else if (EDGE) {
            r[which] = (row < rows_valid && 8 * half + which < k_valid) ? *element(which) : 0.0f;
        } else {
            r[which] = *element(which);
        }
    }
    __device__ __forceinline__ void advance() { base += step; }
};

// Two floats rounded to bf16 (nearest even) in one dword: x0 in the low half.
__device__ __forceinline__ unsigned int pack_bf16_pair(float x0, float x1)
{
    const gram_bf16x2 v = __builtin_convertvector(gram_float2{x0, x1}, gram_bf16x2);
    return __builtin_bit_cast(unsigned int, v);
}
__device__ __forceinline__ float bf16_low_as_float(unsigned int pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_high_as_float(unsigned int pair) { return __uint_as_float(pair & 0xffff0000u); }

template <int N>
struct GramStep {
    static constexpr int value = N;
};

template <int LOAD_A, int LOAD_B, bool FULL, bool CENTRED, bool QUADS = false>
__device__ __forceinline__ void gram_bf16_walk(
    gram_float16 (&acc)[2][2], float &square_a, float &square_b, RowOwnerLoader<LOAD_A> &load_a,
    RowOwnerLoader<LOAD_B> &load_b, gram_chunk *lds_a, gram_chunk *lds_b, int k_total, int m_valid, int n_valid,
    int wave_m, int wave_n, int h, int i, const float *centre)
{
    typedef const float __attribute__((address_space(4))) *uniform_pointer;
    constexpr bool COL_A = RowOwnerLoader<LOAD_A>::COL, COL_B = RowOwnerLoader<LOAD_B>::COL;
    const int k_slices = (k_total + BK_TILE_K - 1) / BK_TILE_K;
    const int k_tail = k_total - (k_slices - 1) * BK_TILE_K;
    // Raw values of two slices in flight: [set][operand][element].  A set that has no
    // slice to take holds zeros, which split into zeros and add nothing to the norms.
    float stage[2][2][8];
    // The k of the centre (see gram_walk) that match a lane's 8 values, through scalar loads so
    // that they cost no vector registers: the K half of a K-major loader is uniform over the wave
    // (8 values: cen[set][half 0]); the lanes of a row-major loader alternate between the two
    // halves, so both are fetched (16 values) and every lane picks its own when it subtracts.
    // Loaders of one kind share them.
    float cen[2][2][8];

    auto fetch = [&](auto set, int slice) {
        constexpr int S = decltype(set)::value;
        if (slice < k_slices) {
            const int kv = slice + 1 == k_slices ? k_tail : BK_TILE_K;
#pragma unroll
            for (int which = 0; which < RowOwnerLoader<LOAD_A>::LOADS; which++)
                load_a.template load_part<!FULL, QUADS>(stage[S][0], which, m_valid, kv);
#pragma unroll
            for (int which = 0; which < RowOwnerLoader<LOAD_B>::LOADS; which++)
                load_b.template load_part<!FULL, QUADS>(stage[S][1], which, n_valid, kv);
            load_a.advance();
            load_b.advance();
            if (CENTRED) {
                const uniform_pointer of_slice = (uniform_pointer)(centre + slice * BK_TILE_K);
                // the half of a K-major loader, or both halves for a row-major one
                const int first = COL_A ? 8 * load_a.half : (COL_B ? 8 * load_b.half : 0);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    cen[S][0][e] = of_slice[first + e];
                    if (!COL_A || !COL_B) cen[S][1][e] = of_slice[(COL_A || COL_B ? 0 : 8) + e + (COL_A != COL_B ? 8 * (1 - (COL_A ? load_a.half : load_b.half)) : 0)];
                }
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) stage[S][0][e] = stage[S][1][e] = cen[S][0][e] = cen[S][1][e] = 0.0f;
        }
    };
    const int write_a = load_a.half * BK_TILE_M + load_a.row;
    const int write_b = load_b.half * BK_TILE_N + load_b.row;
    const int read_a = h * BK_TILE_M + wave_m + i;
    const int read_b = h * BK_TILE_N + wave_n + i;

    // Splitting set S and writing its pieces to LDS buffer `buffer`, cut into 24 parts
    // (8 pairs of values x 3 rounding steps).  x = p1 + p2 + p3 exactly, every piece a
    // bf16: p1 = bf16(x), p2 = bf16(x - p1), p3 = bf16(x - p1 - p2).
    unsigned int piece[GB_PIECES][4];
    float rest0 = 0.0f, rest1 = 0.0f;
    auto commit_part = [&](auto set, auto part, int buffer) {
        constexpr int S = decltype(set)::value;
        constexpr int PART = decltype(part)::value;
        constexpr int pair = PART / 3, phase = PART % 3;
        constexpr int operand = pair / 4, q = pair % 4;
        if (phase == 0 && CENTRED) {
            constexpr bool col = operand == 0 ? COL_A : COL_B;
            // cen[S][0] is the half of the K-major loader if there is one, else half 0; cen[S][1] the other half
            const int uniform_half = COL_A ? load_a.half : load_b.half;     // meaningful when one loader is K-major
            const int lane_half = operand == 0 ? load_a.half : load_b.half;
            const bool other = col ? false : ((COL_A || COL_B) ? lane_half != uniform_half : lane_half != 0);
            stage[S][operand][2 * q] -= other ? cen[S][1][2 * q] : cen[S][0][2 * q];
            stage[S][operand][2 * q + 1] -= other ? cen[S][1][2 * q + 1] : cen[S][0][2 * q + 1];
        }
        const float x0 = stage[S][operand][2 * q], x1 = stage[S][operand][2 * q + 1];
        if (phase == 0) {
            float &square = operand == 0 ? square_a : square_b;
            square += x0 * x0;
            square += x1 * x1;
            piece[0][q] = pack_bf16_pair(x0, x1);
            rest0 = bf16_low_as_float(piece[0][q]);
            rest1 = bf16_high_as_float(piece[0][q]);
        } else if (phase == 1) {
            rest0 = x0 - rest0;
            rest1 = x1 - rest1;
            piece[1][q] = pack_bf16_pair(rest0, rest1);
        } else {
            rest0 -= bf16_low_as_float(piece[1][q]);
            rest1 -= bf16_high_as_float(piece[1][q]);
            piece[2][q] = pack_bf16_pair(rest0, rest1);
            if (q == 3) {
                gram_chunk *lds = (operand == 0 ? lds_a : lds_b) + buffer * GB_PANEL_CHUNKS + (operand == 0 ? write_a : write_b);
#pragma unroll
                for (int p = 0; p < GB_PIECES; p++)
                    lds[p * 2 * BK_TILE_M] = gram_chunk{piece[p][0], piece[p][1], piece[p][2], piece[p][3]};
            }
        }
    };
    auto for_all_parts = [&](auto &&body) {
        body(GramStep<0>{});   body(GramStep<1>{});   body(GramStep<2>{});   body(GramStep<3>{});
        body(GramStep<4>{});   body(GramStep<5>{});   body(GramStep<6>{});   body(GramStep<7>{});
        body(GramStep<8>{});   body(GramStep<9>{});   body(GramStep<10>{});  body(GramStep<11>{});
        body(GramStep<12>{});  body(GramStep<13>{});  body(GramStep<14>{});  body(GramStep<15>{});
        body(GramStep<16>{});  body(GramStep<17>{});  body(GramStep<18>{});  body(GramStep<19>{});
        body(GramStep<20>{});  body(GramStep<21>{});  body(GramStep<22>{});  body(GramStep<23>{});
    };

    // One slice, held in LDS buffer S (= slice & 1): the registers of set S are free and
    // take slice + 2; set 1 - S holds slice + 1 and goes to buffer 1 - S.  Smallest
    // products first; the four accumulators take turns, so consecutive matrix
    // instructions never depend on each other.
    gram_bf16x8 fa[2][GB_PIECES], fb[2][GB_PIECES];
    constexpr int term_a[6] = {1, 0, 2, 0, 1, 0};
    constexpr int term_b[6] = {1, 2, 0, 1, 0, 0};
    auto step = [&](auto set, int slice) {
        constexpr int S = decltype(set)::value;
        fetch(set, slice + 2);
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int p = 0; p < GB_PIECES; p++) {
                fa[t][p] = __builtin_bit_cast(gram_bf16x8, lds_a[S * GB_PANEL_CHUNKS + p * 2 * BK_TILE_M + read_a + 32 * t]);
                fb[t][p] = __builtin_bit_cast(gram_bf16x8, lds_b[S * GB_PANEL_CHUNKS + p * 2 * BK_TILE_N + read_b + 32 * t]);
            }
        __builtin_amdgcn_sched_barrier(0);
        for_all_parts([&](auto part) {
            constexpr int PART = decltype(part)::value;
            constexpr int term = PART / 4, mt = (PART >> 1) & 1, nt = PART & 1;
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mt][term_a[term]], fb[nt][term_b[term]],
                                                                 acc[mt][nt], 0, 0, 0);
            commit_part(GramStep<1 - S>{}, part, 1 - S);
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
    };

    fetch(GramStep<0>{}, 0);
    fetch(GramStep<1>{}, 1);
    for_all_parts([&](auto part) { commit_part(GramStep<0>{}, part, 0); });
    __syncthreads();

    for (int slice = 0; slice < k_slices; slice += 2) {
        step(GramStep<0>{}, slice);
        if (slice + 1 < k_slices) step(GramStep<1>{}, slice + 1);
    }
}

// RAGGED_K: built for K that is not a multiple of 16, where no tile can take the unpredicated
// walk; instantiated for the loader pairs with 128-bit row-major loads, which otherwise fall
// back to eight predicated scalar loads per slice (M = N = 16384, K = 1000: 6.8 -> 3.4 ms).
// A kernel of its own because the two kinds of predicated loads side by side cost the
// unpredicated walk of the same kernel 20 % (register allocation), and with a register
// budget for two waves per SIMD: within the budget for three the compiler spills 180.
// CENTRED: args.centre is subtracted from both operands while they are staged (a kernel of its
// own: a run-time switch inside the walk breaks the interleaving of matrix instructions and split).
template <int LOAD_A, int LOAD_B, bool RAGGED_K = false, bool CENTRED = false>
__global__ __launch_bounds__(BK_THREADS, RAGGED_K ? 2 : GB_WAVES) void gram_bf16_l2_kernel(const BuildKernelArgs args)
{
    __shared__ gram_chunk lds_a[2 * GB_PANEL_CHUNKS];
    __shared__ gram_chunk lds_b[2 * GB_PANEL_CHUNKS];
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
    const int h = lane >> 5;     // K half (operands) / row half (result)
    const int i = lane & 31;     // row (operand A) / column (operand B, result)

    RowOwnerLoader<LOAD_A> load_a;
    RowOwnerLoader<LOAD_B> load_b;
    load_a.init(args.a + batch * args.a_bs, args.a_ld, m0, tid);
    load_b.init(args.b + batch * args.b_bs, args.b_ld, n0, tid);

    float square_a = 0.0f, square_b = 0.0f;   // sum of squares of what this lane staged: half a row each
    gram_float16 acc[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mt][nt][v] = 0.0f;

    const float *centre = CENTRED ? centre_to_subtract(args, batch) : nullptr;
    auto walk = [&](auto centred) {
        constexpr bool C = decltype(centred)::value;
        if (RAGGED_K) {
            gram_bf16_walk<LOAD_A, LOAD_B, false, C, true>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, args.k, m_valid,
                                                           n_valid, wave_m, wave_n, h, i, centre);
        } else if (m_valid >= BK_TILE_M && n_valid >= BK_TILE_N && args.k % BK_TILE_K == 0) {
            gram_bf16_walk<LOAD_A, LOAD_B, true, C>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, args.k, m_valid,
                                                    n_valid, wave_m, wave_n, h, i, centre);
        } else {
            gram_bf16_walk<LOAD_A, LOAD_B, false, C>(acc, square_a, square_b, load_a, load_b, lds_a, lds_b, args.k, m_valid,
                                                     n_valid, wave_m, wave_n, h, i, centre);
        }
    };
    if (CENTRED && centre) walk(GramSwitch<CENTRED>{});
    else walk(GramSwitch<false>{});

    // Row norms: low K half first, so that the same point gets the same norm in every
    // workgroup and on either side.  The buffers of the walk are free by now.
    {
        float *partial = reinterpret_cast<float *>(lds_a);     // [operand][half][row]
        partial[load_a.half * BK_TILE_M + load_a.row] = square_a;
        partial[2 * BK_TILE_M + load_b.half * BK_TILE_N + load_b.row] = square_b;
        __syncthreads();
        if (tid < BK_TILE_M)
            lds_norm_a[tid] = partial[tid] + partial[BK_TILE_M + tid];
        else
            lds_norm_b[tid - BK_TILE_M] = partial[2 * BK_TILE_M + tid - BK_TILE_M] + partial[3 * BK_TILE_M + tid - BK_TILE_M];
    }
    __syncthreads();

#include "gram_epilogue.inc"
}

}  // namespace kmc
