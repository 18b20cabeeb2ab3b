// Matrix-core path for squared differences, large problems: the cross term of
//
//   sum_k (b[n,k] - a[m,k])^2  =  |a_m|^2 + |b_n|^2 - 2 * sum_k a[m,k] * b[n,k]
//
// on the fp16 matrix instruction (v_mfma_f32_32x32x16_f16, the rate of the bf16 one), from two
// fp16 pieces per fp32 value and three piece products, in three launches with a workspace
// between them:
//
//   gram_row_stats   per row of an operand: sum of squares (the norms of the expansion) and
//                    largest magnitude, both after the centre has been subtracted.
//   gram_f16_split   scales every row by a power of two that puts its largest magnitude into
//                    [2^14, 2^15), splits every scaled value x into h1 = fp16(x), h2 = fp16(x - h1)
//                    and writes the pieces in the order the matrix instruction reads them.
//   gram_f16_wide    one workgroup of 8 waves per 256 x 256 tile of the result: copies pieces from
//                    the workspace into LDS and multiplies; a1 b1 + a1 b2 + a2 b1, fp32 accumulators.
//
// Accuracy.  x - h1 is exact in fp32 and h2 keeps 11 of its bits: |x - h1 - h2| <= 2^-22 |x|, or
// 2^-25 where h2 is subnormal, which is 2^-39 of the row's largest magnitude.  The dropped product
// a2 b2 is below 2^-22 |a_k b_k|.  The error of a dot product from the pieces is therefore below
// 3 * 2^-22 sum_k |a_k b_k| <= 3.6e-7 (|a|^2 + |b|^2), in practice far less since the roundings
// do not line up, beside the rounding of the fp32 accumulation that every matrix-core path has
// (products of fp16 pieces are exact in fp32).  The scale per row is what makes the bound relative
// to that row's norm, which is what the trust rule of gram_kernel.hpp needs: with one scale per
// operand a row of small values next to a row of large ones would sit in fp16's subnormals.
// Scales are powers of two, so scaling and unscaling round nothing.  Rows that hold an infinity or
// a NaN produce results that are not numbers, which are distrusted and recomputed like any other.
//
// Why two fp16 pieces and not the three bf16 pieces of gram_bf16_kernel.hpp: measured with this
// same kernel structure at M = N = 30000, K = 1024, the board is power-limited (shader clock
// 1.87 GHz with copies and matrix instructions running together, 2.37 GHz with either alone; the
// matrix pipeline is busy two thirds of the cycles in all three cases), so time follows energy:
// six products of three pieces 8.9 ms, three products of two pieces 5.4 ms.  Why a workspace: a
// value is split once instead of once per tile that needs it (in the one-step kernel the split
// takes as long as the matrix instructions it hides behind), a 256 x 256 tile asks the L2 for half
// the bytes per matrix instruction of a 128 x 128 one, and the layout of an operand in memory
// only matters to the split.
//
// Workspace of one operand and batch entry, in 16-byte chunks of 8 fp16 (one row, one half of a
// 16-deep K slice, one piece):  chunk[slice][piece][half][row 0 .. rows_pad),  rows_pad a multiple
// of 256; rows that do not exist and k beyond K hold zeros, so the product kernel has no edge
// handling in its walk.  Four slices more than K has are allocated and never multiplied.
// Two compile-time switches leave a part of the product kernel out, for the measurements of what
// bounds it (the results are then wrong): -DGW_ABLATE_NO_COPY issues no copies from the workspace,
// -DGW_ABLATE_NO_EPILOGUE returns behind the walk.
// Statistics: partial[range][row] for the sums of squares and for the magnitudes, one partial per
// range of K slices that a workgroup walks, combined in the order of the ranges.
// The reference has no such path (include/build_a_kernel.cuh:339-370 is SIMT only).
#pragma once

#include "gram_bf16_kernel.hpp"

namespace kmc {

typedef _Float16 gram_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 gram_half2 __attribute__((ext_vector_type(2)));

constexpr int GW_TILE = 256;                                  // rows of a and of b per workgroup
constexpr int GW_THREADS = 512;
constexpr int GW_PIECES = 2;
constexpr int GW_SEGMENTS = 2 * GW_PIECES;                    // (piece, half) pairs of one slice
constexpr int GW_OPERAND_CHUNKS = GW_SEGMENTS * GW_TILE;      // 16 KB
constexpr int GW_BUFFER_CHUNKS = 2 * GW_OPERAND_CHUNKS;       // one slice of both operands: 32 KB
constexpr int GW_EXTRA_SLICES = 4;                            // copied ahead of the walk, never multiplied
constexpr int GW_BAND_N = 32;                                 // tile order: n tiles per band
constexpr int GW_ROW_THREADS = 256;
constexpr int GW_SCALE_EXPONENT = 14;                         // a row's largest magnitude goes to [2^14, 2^15)

// One operand, for gram_row_stats and gram_f16_split.
struct GramRowsArgs {
    const float *x; i64 ld, bs;
    int rows, k, row_major, vec;          // vec: 128-bit loads along k are allowed (row-major only)
    const float *centre; i64 centre_bs;   // as BuildKernelArgs::centre, or null
    gram_chunk *pieces; i64 pieces_bs;    // per batch entry, in chunks
    float *squares; float *magnitudes;    // [batch][range][rows_pad]
    float *unscale;                       // [batch][rows_pad]: 1 / the row's scale
    i64 stats_bs, unscale_bs;
    int rows_pad, slices, slices_per_range, ranges;
    int zero_slices;                      // slices behind the last that gram_f16_split fills with zeros (for
                                          // walks in steps of more than one slice)
};

struct GramWideArgs {
    BuildKernelArgs kernel;               // extents, result, epilogue, trust; tiles_* are not used
    const gram_chunk *pieces_a, *pieces_b;
    i64 pieces_a_bs, pieces_b_bs;
    const float *squares_a, *squares_b;
    i64 stats_a_bs, stats_b_bs;
    const float *unscale_a, *unscale_b;
    i64 unscale_a_bs, unscale_b_bs;
    int rows_pad_a, rows_pad_b, slices, ranges;
    int wide_tiles_m, wide_tiles_n, wide_tiles_n_padded;
    // GW_EPILOGUE_GRADIENT_L2 only: row r of b stands for (o, n) = (r / gradient_n, r % gradient_n) and
    // the result is (d[n][m] - shift[n]) * g[m][o] - a[m] . b[r]
    const float *gradient_d; i64 gradient_d_ld, gradient_d_bs;
    const float *gradient_g; i64 gradient_g_ld, gradient_g_bs;
    const float *gradient_shift; i64 gradient_shift_bs;
    int gradient_n;
};

constexpr int GW_MAX_RANGES = 9;      // ranges of K per row: ceil(slices / 8) up to 71 slices, 8 beyond

constexpr int GW_EPILOGUE_DISTANCE = 0;
constexpr int GW_EPILOGUE_GRADIENT_L2 = 1;
constexpr int GW_EPILOGUE_DOT = 2;

// The 16 values of row `row` in slice `slice`, centre subtracted; zeros where the row or k does not exist.
__device__ __forceinline__ void gram_load_row_slice(const GramRowsArgs &args, const float *x, const float *centre, int row,
                                                    int slice, float (&v)[BK_TILE_K])
{
    const bool live = row < args.rows;
    const int k0 = slice * BK_TILE_K;
    if (args.row_major) {
        const float *src = x + (i64)row * args.ld + k0;
        if (live && args.vec && k0 + BK_TILE_K <= args.k) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 f = reinterpret_cast<const float4 *>(src)[q];
                v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < BK_TILE_K; e++) v[e] = (live && k0 + e < args.k) ? src[e] : 0.0f;
        }
    } else {
#pragma unroll
        for (int e = 0; e < BK_TILE_K; e++) v[e] = (live && k0 + e < args.k) ? x[(i64)(k0 + e) * args.ld + row] : 0.0f;
    }
    if (centre) {
        // beyond K the centre is padded with zeros, like the values
#pragma unroll
        for (int e = 0; e < BK_TILE_K; e++) v[e] = live ? v[e] - centre[k0 + e] : 0.0f;
    }
}

__device__ __forceinline__ const float *gram_rows_centre(const GramRowsArgs &args, int batch)
{
    if (!args.centre) return nullptr;
    const float *centre = args.centre + batch * args.centre_bs;
    const int padded = (args.k + GRAM_CENTRE_PAD - 1) / GRAM_CENTRE_PAD * GRAM_CENTRE_PAD;
    return centre[padded] != 0.0f ? centre : nullptr;      // the flag behind the vector: see centre_to_subtract
}

// One thread per row, one workgroup per 256 rows and range of slices.  (The row kernels are
// templates only so that every translation unit that includes this header may hold them.)
__device__ __forceinline__ void gram_row_stats_of(const GramRowsArgs &args, int block)
{
    const int row = block * GW_ROW_THREADS + threadIdx.x;
    const int range = blockIdx.y, batch = blockIdx.z;
    const float *x = args.x + batch * args.bs;
    const float *centre = gram_rows_centre(args, batch);
    const int first = range * args.slices_per_range;
    const int last = min(first + args.slices_per_range, args.slices);
    float square = 0.0f, magnitude = 0.0f;
    bool not_a_number = false;
    for (int slice = first; slice < last; slice++) {
        float v[BK_TILE_K];
        gram_load_row_slice(args, x, centre, row, slice, v);
#pragma unroll
        for (int e = 0; e < BK_TILE_K; e++) {
            square += v[e] * v[e];
            magnitude = fmaxf(magnitude, fabsf(v[e]));      // skips NaNs
            not_a_number |= v[e] != v[e];
        }
    }
    const i64 at = batch * args.stats_bs + (i64)range * args.rows_pad + row;
    args.squares[at] = square;
    args.magnitudes[at] = not_a_number ? __builtin_nanf("") : magnitude;
}

template <int UNUSED = 0>
__global__ __launch_bounds__(GW_ROW_THREADS) void gram_row_stats(const GramRowsArgs args)
{
    gram_row_stats_of(args, blockIdx.x);
}

__device__ __forceinline__ void gram_f16_split_of(const GramRowsArgs &args, int block)
{
    const int row = block * GW_ROW_THREADS + threadIdx.x;
    const int range = blockIdx.y, batch = blockIdx.z;
    const float *x = args.x + batch * args.bs;
    const float *centre = gram_rows_centre(args, batch);

    // scale = 2^(GW_SCALE_EXPONENT - floor(log2 magnitude)), from the exponent field.  Rows of
    // zeros or of values below 2^-111 take the largest scale used, 2^125 (the scale and its
    // inverse must both be normal numbers); a row with a NaN or an infinity takes the smallest:
    // its products are not numbers whatever the scale.
    float magnitude = 0.0f;
    for (int r = 0; r < args.ranges; r++) {
        const float part = args.magnitudes[batch * args.stats_bs + (i64)r * args.rows_pad + row];
        magnitude = part != part ? part : fmaxf(magnitude, part);
        if (part != part) break;
    }
    int exponent_field = (__float_as_uint(magnitude) >> 23) & 0xff;
    exponent_field = max(exponent_field, 16);
    const float scale = __uint_as_float((unsigned)(127 + GW_SCALE_EXPONENT + 127 - exponent_field) << 23);
    if (range == 0)
        args.unscale[batch * args.unscale_bs + row] = __uint_as_float((unsigned)(exponent_field - GW_SCALE_EXPONENT) << 23);

    gram_chunk *pieces = args.pieces + batch * args.pieces_bs;
    const int first = range * args.slices_per_range;
    const int last = min(first + args.slices_per_range, args.slices);
    for (int slice = first; slice < last; slice++) {
        float v[BK_TILE_K];
        gram_load_row_slice(args, x, centre, row, slice, v);
        unsigned int piece[GW_PIECES][8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const float x0 = v[2 * q] * scale, x1 = v[2 * q + 1] * scale;
            const gram_half2 h1 = __builtin_convertvector(gram_float2{x0, x1}, gram_half2);
            const gram_float2 back = __builtin_convertvector(h1, gram_float2);
            const gram_half2 h2 = __builtin_convertvector(gram_float2{x0 - back.x, x1 - back.y}, gram_half2);
            piece[0][q] = __builtin_bit_cast(unsigned int, h1);
            piece[1][q] = __builtin_bit_cast(unsigned int, h2);
        }
        gram_chunk *dst = pieces + (i64)slice * GW_SEGMENTS * args.rows_pad + row;
#pragma unroll
        for (int p = 0; p < GW_PIECES; p++)
#pragma unroll
            for (int half = 0; half < 2; half++)
                dst[(i64)(2 * p + half) * args.rows_pad] =
                    gram_chunk{piece[p][4 * half], piece[p][4 * half + 1], piece[p][4 * half + 2], piece[p][4 * half + 3]};
    }
    if (range == args.ranges - 1) {
        for (int slice = args.slices; slice < args.slices + args.zero_slices; slice++) {
            gram_chunk *dst = pieces + (i64)slice * GW_SEGMENTS * args.rows_pad + row;
#pragma unroll
            for (int segment = 0; segment < GW_SEGMENTS; segment++) dst[(i64)segment * args.rows_pad] = gram_chunk{0u, 0u, 0u, 0u};
        }
    }
}

template <int UNUSED = 0>
__global__ __launch_bounds__(GW_ROW_THREADS) void gram_f16_split(const GramRowsArgs args)
{
    gram_f16_split_of(args, blockIdx.x);
}

// Both operands of a call in one launch each (at a few thousand rows a launch of these kernels is its own latency, and
// two of them one after the other cost twice that): the first `first_blocks` workgroups along x take the first operand.
// Both have the same ranges of slices; an operand with fewer batch entries than the grid leaves the surplus idle.
struct GramRowsPair {
    GramRowsArgs first, second;
    int first_blocks, first_batches, second_batches;
};

template <int UNUSED = 0>
__global__ __launch_bounds__(GW_ROW_THREADS) void gram_row_stats_pair(const GramRowsPair pair)
{
    if ((int)blockIdx.x < pair.first_blocks) {
        if ((int)blockIdx.z < pair.first_batches) gram_row_stats_of(pair.first, blockIdx.x);
    } else if ((int)blockIdx.z < pair.second_batches) {
        gram_row_stats_of(pair.second, blockIdx.x - pair.first_blocks);
    }
}

template <int UNUSED = 0>
__global__ __launch_bounds__(GW_ROW_THREADS) void gram_f16_split_pair(const GramRowsPair pair)
{
    if ((int)blockIdx.x < pair.first_blocks) {
        if ((int)blockIdx.z < pair.first_batches) gram_f16_split_of(pair.first, blockIdx.x);
    } else if ((int)blockIdx.z < pair.second_batches) {
        gram_f16_split_of(pair.second, blockIdx.x - pair.first_blocks);
    }
}

// Workgroup -> tile, as tile_of_workgroup of build_kernel.hpp with bands of GW_BAND_N tiles: a
// CU holds one workgroup, so the 32 of an XCD cover 4 n tiles x 8 m tiles of a band at a time.
// SYMMETRIC (a panel against itself): the ids count through the tiles on and below the diagonal,
// row r of the triangle starting at id r (r + 1) / 2.
template <bool SYMMETRIC>
__device__ __forceinline__ bool wide_tile_of_workgroup(const GramWideArgs &args, int &tile_m, int &tile_n)
{
    const int rotated = blockIdx.x + blockIdx.y % gridDim.x;
    const int linear = rotated >= (int)gridDim.x ? rotated - (int)gridDim.x : rotated;
    if (SYMMETRIC) {
        int row = (int)((sqrtf(8.0f * (float)linear + 1.0f) - 1.0f) * 0.5f);
        while (row * (row + 1) / 2 > linear) row--;
        while ((row + 1) * (row + 2) / 2 <= linear) row++;
        tile_m = row;
        tile_n = linear - row * (row + 1) / 2;
        return true;
    }
    const int band_tiles = GW_BAND_N * args.wide_tiles_m;
    const int band = linear / band_tiles;
    const int band_height = min(GW_BAND_N, args.wide_tiles_n_padded - band * GW_BAND_N);
    const int in_band = linear - band * band_tiles;
    tile_m = in_band / band_height;
    tile_n = band * GW_BAND_N + in_band % band_height;
    return tile_n < args.wide_tiles_n;
}

// Wave w of 8 owns rows wave_m .. +128 of a and wave_n .. +64 of b: 4 x 2 matrix-instruction
// tiles of 32 x 32, 128 accumulator registers, 24 matrix instructions per slice.
//
// The pieces go from the workspace straight into LDS (global_load_lds_dwordx4: a wave copies 64
// consecutive chunks, no registers involved), four slices in four buffers.  One barrier per
// slice.  The operands of a slice are read into registers during the slice before it, so behind
// the barrier of slice s the buffer of slice s is free and takes slice s + 4, and slice s + 1,
// whose copies were issued three slices earlier, is complete and is read.
//
// The copies are written as instructions: through the compiler's builtin every later LDS read
// waits for every copy under way (the copies carry no information on which array they fill), which
// leaves nothing in flight.  The compiler therefore does not count these copies either; the walk
// waits for them itself, and no other vector load is issued between the first copy and the wait
// for all of them behind the walk.
//
// SYMMETRIC: b is a, the result is symmetric, and it is made so bit for bit: one workgroup per
// tile on or below the diagonal; what lies below the diagonal is stored a second time, mirrored;
// of a 128 x 128 part on the diagonal the lower triangle is stored and mirrored (the two halves of
// such a part are computed with the pieces in exchanged roles and differ in the last bit); the
// part above the diagonal inside a diagonal tile is not stored from its own values at all.  A
// distrusted part is left to the repair launch, which mirrors what it recomputes.
//
// EPILOGUE GW_EPILOGUE_GRADIENT_L2: the same walk as a plain product of the pieces, for the gradient
// of the L2 norm (norm_gradient_l2_wide.hpp): no norms, no trust check, the epilogue combines the
// product with d and g as GramWideArgs says.
//
// EPILOGUE GW_EPILOGUE_DOT: the inner operator DOT (sum_k a b): the product of the pieces is the
// value itself, nothing cancels, so there is no trust check and no repair; outer power, kernel
// function, regularised diagonal and the stores, mirrored ones included, are those of the distance.
template <bool SYMMETRIC, int EPILOGUE = GW_EPILOGUE_DISTANCE>
__global__ __launch_bounds__(GW_THREADS) void gram_f16_wide(const GramWideArgs args)
{
    __shared__ gram_chunk lds0[GW_BUFFER_CHUNKS];
    __shared__ gram_chunk lds1[GW_BUFFER_CHUNKS];
    __shared__ gram_chunk lds2[GW_BUFFER_CHUNKS];
    __shared__ gram_chunk lds3[GW_BUFFER_CHUNKS];
    __shared__ __attribute__((aligned(16))) float lds_norm_a[GW_TILE], lds_norm_b[GW_TILE];
    __shared__ __attribute__((aligned(16))) float lds_unscale_a[GW_TILE], lds_unscale_b[GW_TILE];
    __shared__ int lds_distrust[4];

    const int tid = threadIdx.x;
    const int batch = blockIdx.y;
    int tile_m, tile_n;
    if (!wide_tile_of_workgroup<SYMMETRIC>(args, tile_m, tile_n)) return;
    const int m0 = tile_m * GW_TILE;
    const int n0 = tile_n * GW_TILE;
    const int m_valid = args.kernel.m - m0;
    const int n_valid = args.kernel.n - n0;

    if constexpr (EPILOGUE == GW_EPILOGUE_DISTANCE) {
        // The sample of the result says that the repair launch would redo (nearly) every part: stamp them all
        // and leave (the branch is uniform over the launch: every workgroup reads the same words).  Parts above the diagonal of a symmetric result belong to nobody.
        if (args.kernel.sample && sample_leaves_it_to_the_direct_kernel(args.kernel.sample)) {
            if (tid < 4) {
                const int part_m = tid & 1, part_n = tid >> 1;
                const bool above = SYMMETRIC && tile_m == tile_n && part_m < part_n;
                if (!above && part_m * 128 < m_valid && part_n * 128 < n_valid)
                    args.kernel.c[batch * args.kernel.c_bs + (i64)(n0 + part_n * 128) * args.kernel.c_ld + m0 + part_m * 128] =
                        __uint_as_float(BK_REPAIR_MARKER);
            }
            return;
        }
    }

    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = (wave & 1) * 128;
    const int wave_n = (wave >> 1) * 64;
    const int h = lane >> 5;
    const int i = lane & 31;

    // Norms of this tile's rows (the partial sums in the order of their ranges) and their scales.
    {
        const bool of_a = tid < GW_TILE;
        const int r = of_a ? tid : tid - GW_TILE;
        const float *partial = of_a ? args.squares_a + batch * args.stats_a_bs + m0 + r : args.squares_b + batch * args.stats_b_bs + n0 + r;
        const int pitch = of_a ? args.rows_pad_a : args.rows_pad_b;
        // all loads first, then the sum in range order: a loop would wait for each load in turn,
        // eight memory latencies before the first copy of the walk is issued
        float parts[GW_MAX_RANGES];
#pragma unroll
        for (int range = 0; range < GW_MAX_RANGES; range++) parts[range] = range < args.ranges ? partial[(i64)range * pitch] : 0.0f;
        float norm = 0.0f;
#pragma unroll
        for (int range = 0; range < GW_MAX_RANGES; range++) norm += range < args.ranges ? parts[range] : 0.0f;
        (of_a ? lds_norm_a : lds_norm_b)[r] = norm;
        (of_a ? lds_unscale_a : lds_unscale_b)[r] =
            of_a ? args.unscale_a[batch * args.unscale_a_bs + m0 + r] : args.unscale_b[batch * args.unscale_b_bs + n0 + r];
        if (tid < 4) lds_distrust[tid] = 0;
    }

    auto buffer = [&](auto which) -> gram_chunk * {
        constexpr int B = decltype(which)::value;
        if constexpr (B == 0) return lds0;
        else if constexpr (B == 1) return lds1;
        else if constexpr (B == 2) return lds2;
        else return lds3;
    };

    // Copies: 32 runs of 64 chunks per slice (operand, segment, quarter of the rows), 4 per wave:
    // runs 0 .. 15 belong to a (q < 2 for every wave), 16 .. 31 to b.
    typedef const __attribute__((address_space(1))) void *global_address;
    typedef __attribute__((address_space(3))) void *lds_address;
    const gram_chunk *src[4];
    int dst[4];     // first chunk of the run in a buffer: uniform over the wave
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int run = wave + 8 * q;
        const int operand = q < 2 ? 0 : 1, segment = (run % 16) / 4, quarter = run % 4;
        const gram_chunk *base = operand == 0 ? args.pieces_a + batch * args.pieces_a_bs + (i64)segment * args.rows_pad_a + m0
                                              : args.pieces_b + batch * args.pieces_b_bs + (i64)segment * args.rows_pad_b + n0;
        src[q] = base + quarter * 64 + lane;
        dst[q] = operand * GW_OPERAND_CHUNKS + segment * GW_TILE + quarter * 64;
    }
    const i64 step_a = (i64)GW_SEGMENTS * args.rows_pad_a, step_b = (i64)GW_SEGMENTS * args.rows_pad_b;
    auto copy = [&](auto into, auto which_run) {
        constexpr int q = decltype(which_run)::value;
        const unsigned lds_byte = (unsigned)(unsigned long)(lds_address)(buffer(into) + dst[q]);
#ifndef GW_ABLATE_NO_COPY
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :
                     : "v"((global_address)src[q]), "s"(lds_byte)
                     : "memory", "m0");
#endif
        src[q] += q < 2 ? step_a : step_b;
    };

    gram_float16 acc[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mt][nt][v] = 0.0f;

    const int read_a = h * GW_TILE + wave_m + i;
    const int read_b = GW_OPERAND_CHUNKS + h * GW_TILE + wave_n + i;
    // fa[set][p], fb[set][p]: piece p (0 the larger) of this wave's rows, for slices of either parity
    gram_half8 fa[2][GW_PIECES][4], fb[2][GW_PIECES][2];
    auto read_operands = [&](auto set, auto from) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int p = GW_PIECES - 1; p >= 0; p--) {
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
                fa[S][p][mt] = __builtin_bit_cast(gram_half8, buffer(from)[2 * p * GW_TILE + read_a + 32 * mt]);
            if (p == GW_PIECES - 1) {
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
                    fb[S][0][nt] = __builtin_bit_cast(gram_half8, buffer(from)[read_b + 32 * nt]);
            }
        }
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
            fb[S][1][nt] = __builtin_bit_cast(gram_half8, buffer(from)[2 * GW_TILE + read_b + 32 * nt]);
    };
    auto multiply = [&](auto set, int pa, int pb) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[S][pa][mt], fb[S][pb][nt], acc[mt][nt], 0, 0, 0);
    };

    // The slice in buffer B, whose operands are in register set S.  The four copies of a slice
    // are issued one per group of eight matrix instructions where they can be: three behind the
    // barrier of the slice whose buffer they fill, the fourth in the first group of the next slice.
    auto step = [&](auto set, auto which) {
        constexpr int S = decltype(set)::value;
        constexpr int B = decltype(which)::value;
        const GramStep<(B + 1) % 4> next;
        const GramStep<(B + 3) % 4> previous;
        multiply(set, 1, 0);                                // a2 b1
        copy(previous, GramStep<3>{});
        __builtin_amdgcn_sched_barrier(0);
        // what may still be under way: the eight copies issued last, of the two slices after the next one
        __builtin_amdgcn_s_waitcnt(0x0F78);                 // vmcnt(8), nothing else
        __syncthreads();
        read_operands(GramStep<1 - S>{}, next);
        copy(which, GramStep<0>{});
        __builtin_amdgcn_sched_barrier(0);
        multiply(set, 0, 0);                                // a1 b1
        copy(which, GramStep<1>{});
        __builtin_amdgcn_sched_barrier(0);
        multiply(set, 0, 1);                                // a1 b2
        copy(which, GramStep<2>{});
        __builtin_amdgcn_sched_barrier(0);
    };

    // slices 0, 1 and 2, and three of the four copies of slice 3
    copy(GramStep<0>{}, GramStep<0>{}); copy(GramStep<0>{}, GramStep<1>{}); copy(GramStep<0>{}, GramStep<2>{}); copy(GramStep<0>{}, GramStep<3>{});
    copy(GramStep<1>{}, GramStep<0>{}); copy(GramStep<1>{}, GramStep<1>{}); copy(GramStep<1>{}, GramStep<2>{}); copy(GramStep<1>{}, GramStep<3>{});
    copy(GramStep<2>{}, GramStep<0>{}); copy(GramStep<2>{}, GramStep<1>{}); copy(GramStep<2>{}, GramStep<2>{}); copy(GramStep<2>{}, GramStep<3>{});
    copy(GramStep<3>{}, GramStep<0>{}); copy(GramStep<3>{}, GramStep<1>{}); copy(GramStep<3>{}, GramStep<2>{});
    __builtin_amdgcn_s_waitcnt(0x0F7B);                     // vmcnt(11): slice 0 has arrived
    __syncthreads();
    read_operands(GramStep<0>{}, GramStep<0>{});
    for (int slice = 0;;) {
        step(GramStep<0>{}, GramStep<0>{});
        if (++slice == args.slices) break;
        step(GramStep<1>{}, GramStep<1>{});
        if (++slice == args.slices) break;
        step(GramStep<0>{}, GramStep<2>{});
        if (++slice == args.slices) break;
        step(GramStep<1>{}, GramStep<3>{});
        if (++slice == args.slices) break;
    }
    // copies of slices that do not exist may still be under way: they must not land in what follows
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

#ifdef GW_ABLATE_NO_EPILOGUE
    if (args.slices > 0) {      // keeps the accumulators alive without storing them
        float sum = 0.0f;
        for (int mt = 0; mt < 4; mt++)
            for (int nt = 0; nt < 2; nt++)
                for (int v = 0; v < 16; v++) sum += acc[mt][nt][v];
        if (sum == 123.456f) args.kernel.c[tid] = sum;
        return;
    }
#endif
    const BuildKernelArgs &kernel = args.kernel;
    if constexpr (EPILOGUE == GW_EPILOGUE_GRADIENT_L2) {
        // A lane holds, of every 32 x 32 tile, one row r of b (its lane number modulo 32) and 16 m in 4 runs of 4.
        const bool full = m_valid >= GW_TILE && n_valid >= GW_TILE;
        float *c_tile = kernel.c + batch * kernel.c_bs + (i64)n0 * kernel.c_ld + m0;
#pragma unroll
        for (int nt = 0; nt < 2; nt++) {
            const int r_local = wave_n + nt * 32 + i;
            if (!full && r_local >= n_valid) continue;
            const int r = n0 + r_local;
            const int o = r / args.gradient_n, n = r - o * args.gradient_n;
            const float unscale_b = lds_unscale_b[r_local];
            const float shift = args.gradient_shift[batch * args.gradient_shift_bs + n];
            const float *d_row = args.gradient_d + batch * args.gradient_d_bs + (i64)n * args.gradient_d_ld + m0;
            const float *g_column = args.gradient_g + batch * args.gradient_g_bs + (i64)m0 * args.gradient_g_ld + o;
            float *row = c_tile + (i64)r_local * kernel.c_ld;
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int m_local = wave_m + mt * 32 + 8 * g + 4 * h;
                    const float4 unscale_a = *reinterpret_cast<const float4 *>(&lds_unscale_a[m_local]);
                    const float unscales_a[4] = {unscale_a.x, unscale_a.y, unscale_a.z, unscale_a.w};
                    float v4[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const bool exists = full || m_local + e < m_valid;
                        const float d = exists ? d_row[m_local + e] - shift : 0.0f;
                        const float weight = exists ? g_column[(i64)(m_local + e) * args.gradient_g_ld] : 0.0f;
                        v4[e] = d * weight - (acc[mt][nt][4 * g + e] * unscales_a[e]) * unscale_b;
                    }
                    if (kernel.c_vec && (full || m_local + 3 < m_valid)) {
                        *reinterpret_cast<float4 *>(row + m_local) = make_float4(v4[0], v4[1], v4[2], v4[3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (m_local + e < m_valid) row[m_local + e] = v4[e];
                    }
                }
        }
        return;
    }
    // d^2 = |a|^2 + |b|^2 - 2 a.b, trust check per 128 x 128 part (the unit the repair launch
    // works in; every wave lies inside one part), epilogue, stores.
    const int outer_power = kernel.outer_power;
    const int kernel_type = kernel.kernel_type;
    float p_outer = 0.0f, neg_gamma = 0.0f, regularization = 0.0f;
    if (outer_power == POW_POW) p_outer = kernel.p_outer ? kernel.p_outer[batch * kernel.p_outer_bs] : kernel.p_outer_value;
    if (kernel_type != KERNEL_NONE) {
        const float bw = kernel.bandwidth ? kernel.bandwidth[batch * kernel.bandwidth_bs] : kernel.bandwidth_value;
        neg_gamma = kernel_neg_gamma(kernel_type, bw);
        regularization = kernel.regularization ? kernel.regularization[batch * kernel.regularization_bs] : kernel.regularization_value;
    }
    const bool regularize = kernel_type != KERNEL_NONE && regularization != 0.0f;
    const float diagonal_value = 1.0f + regularization;

    // A lane holds, of every 32 x 32 tile, one n (its lane number modulo 32) and 16 m in 4 runs of 4:
    //   acc[mt][nt][v]:  m = wave_m + 32 mt + 8 (v / 4) + 4 h + v % 4,  n = wave_n + 32 nt + i
    // (With the rows of b as the first operand of the matrix instruction a lane holds one m and
    // every store writes whole 128-byte lines, 32-bit stores instead of 128-bit ones: measured
    // 2 % slower.)
    //
    // d^2 and the trust check first, without branches: norms and scales of a come as 128-bit
    // reads; what is not trusted is collected as a lane mask in scalar registers.  A tile that is
    // not a full one masks the rows and columns that do not exist.  The outer function follows
    // with its switch outside the loop over the values.
    const bool full = m_valid >= GW_TILE && n_valid >= GW_TILE;
    unsigned long long distrusted = 0;
    float norm_b[2], unscale_b[2];
    int n_local[2];
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
        n_local[nt] = wave_n + nt * 32 + i;
        norm_b[nt] = lds_norm_b[n_local[nt]];
        unscale_b[nt] = -2.0f * lds_unscale_b[n_local[nt]];
    }
    const float trust = kernel.gram_trust;
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int m_local = wave_m + mt * 32 + 8 * g + 4 * h;
            const float4 norm_a = *reinterpret_cast<const float4 *>(&lds_norm_a[m_local]);
            const float4 unscale_a = *reinterpret_cast<const float4 *>(&lds_unscale_a[m_local]);
            const float norms_a[4] = {norm_a.x, norm_a.y, norm_a.z, norm_a.w};
            const float unscales_a[4] = {unscale_a.x, unscale_a.y, unscale_a.z, unscale_a.w};
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) {
                    if constexpr (EPILOGUE == GW_EPILOGUE_DOT) {
                        // unscale_b carries the factor -2 of the distance
                        acc[mt][nt][4 * g + e] = (acc[mt][nt][4 * g + e] * unscales_a[e]) * (-0.5f * unscale_b[nt]);
                    } else {
                        const float norms = norms_a[e] + norm_b[nt];
                        const float d2 = norms + (acc[mt][nt][4 * g + e] * unscales_a[e]) * unscale_b[nt];
                        // not a number (overflowing squares, NaN data): not trusted either
                        bool bad = !(d2 >= trust * norms);
                        if (!full) bad = bad && m_local + e < m_valid && n_local[nt] < n_valid;
                        distrusted |= __builtin_amdgcn_ballot_w64(bad);
                        acc[mt][nt][4 * g + e] = fmaxf(d2, 0.0f);
                    }
                }
        }
    auto for_each = [&](auto &&f) {
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[mt][nt][v] = f(acc[mt][nt][v]);
    };
    // the outer function and the kernel function of epilogue_value (device_common.hpp)
    switch (outer_power) {
    case POW_ABS: for_each([](float v) { return fabsf(v); }); break;
    case POW_SQUARE: for_each([](float v) { return v * v; }); break;
    case POW_SQRT: for_each([](float v) { return __builtin_amdgcn_sqrtf(v); }); break;
    case POW_POW: for_each([=](float v) { return epilogue_value(v, POW_POW, KERNEL_NONE, p_outer, 0.0f, 0.0f); }); break;
    default: break;
    }
    if (kernel_type != KERNEL_NONE) {
        const float epsilon = kernel.epsilon;
        for_each([=](float v) { return epilogue_value(v, POW_NOOP, kernel_type, 0.0f, neg_gamma, epsilon); });
    }
    if (regularize) {
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m_local = wave_m + mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
                    if (kernel.reg_off_x + m0 + m_local == kernel.reg_off_y + n0 + n_local[nt]) acc[mt][nt][v] = diagonal_value;
            }
    }
    const int part_m = wave & 1, part_n = wave >> 2;
    const int part = part_m + 2 * part_n;
    // where this wave's part lies: below the diagonal of the result (stored and mirrored), on it
    // (lower triangle stored and mirrored), above it inside a diagonal tile (not stored)
    const bool on_diagonal = SYMMETRIC && tile_m == tile_n && part_m == part_n;
    const bool above = SYMMETRIC && tile_m == tile_n && part_m < part_n;
    if (distrusted != 0 && lane == 0 && !above) lds_distrust[part] = 1;
    __syncthreads();
    if (above) return;
    const bool repair = lds_distrust[part] != 0;
    // the first element of a part is held by lane 0 of the wave that starts the part
    if (repair && lane == 0 && (wave_n & 127) == 0) acc[0][0][0] = __uint_as_float(BK_REPAIR_MARKER);

    float *c_tile = kernel.c + batch * kernel.c_bs + (i64)n0 * kernel.c_ld + m0;
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
        if (!full && n_local[nt] >= n_valid) continue;
        float *row = c_tile + (i64)n_local[nt] * kernel.c_ld;
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int m_local = wave_m + mt * 32 + 8 * g + 4 * h;
                const float v4[4] = {acc[mt][nt][4 * g], acc[mt][nt][4 * g + 1], acc[mt][nt][4 * g + 2], acc[mt][nt][4 * g + 3]};
                const bool whole = !on_diagonal || m_local >= n_local[nt];
                if (kernel.c_vec && whole && (full || m_local + 3 < m_valid)) {
                    *reinterpret_cast<float4 *>(row + m_local) = make_float4(v4[0], v4[1], v4[2], v4[3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (m_local + e < m_valid && (!on_diagonal || m_local + e >= n_local[nt])) row[m_local + e] = v4[e];
                }
            }
    }

    // The same values at C(n, m), where the 32 consecutive n of a half wave are the contiguous ones.
    if (SYMMETRIC && !repair) {
        float *mirror = kernel.c + batch * kernel.c_bs + (i64)m0 * kernel.c_ld + n0;
#pragma unroll
        for (int nt = 0; nt < 2; nt++) {
            if (!full && n_local[nt] >= n_valid) continue;
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m_local = wave_m + mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
                    if ((full || m_local < m_valid) && (!on_diagonal || m_local > n_local[nt]))
                        mirror[(i64)m_local * kernel.c_ld + n_local[nt]] = acc[mt][nt][v];
                }
        }
    }
}

}  // namespace kmc
