// Kernel-gradient contraction for the L1 norm on the fp16 matrix instruction:
//
//   E[m, n, o, l] = sum_k C[o,k,l] * A[m,k,l] * s(m,n,k),     s = copysign(1, D[m,n,l] - B[n,k,l])
//
// (reference: include/p_norm_gradient.cuh:407-497 with NormType::L1, whose weight of a term is
// the sign of d - b, :373-394).  The factor that depends on all of m, n and k is a sign, and a
// sign can be put on a 16-bit piece exactly.  So A and C are split once, like the operands of
// gram_f16_wide.hpp and by the same two kernels (a power-of-two scale per row m of A and per row
// o of C, two fp16 pieces per scaled value, 16-byte chunks of 8 k in the order the matrix
// instruction reads them), and the contraction over k runs on v_mfma_f32_16x16x32_f16 with
//
//   T1 = +-a1, T2 = +-a2 (the sign bit of d - b flipped into both pieces),   T1 c1 + T1 c2 + T2 c1
//
// per 32 k: 3 matrix instructions of 16 cycles where the fp32 kernel (norm_gradient_mfma.hpp)
// issues 8 of 32 cycles.  What a lane computes per (m, n, k) is one subtraction, half a byte
// permute, half an AND and two halves of an XOR: 3 vector instructions, as many as the fp32
// kernel spends, which now bound the kernel instead of the matrix pipeline.
// Accuracy: as in gram_f16_wide.hpp, |x - h1 - h2| <= 2^-22 |x| per value and the dropped product
// a2 c2 below 2^-22 |a c|: the error of E from the pieces is below 3 * 2^-22 sum_k |c a|, the size
// of the rounding of an fp32 accumulation over a few terms, beside the fp32 accumulation itself.
//
// Workgroup: 4 waves, 64 m x 32 n x 16 o (for more than 16 outputs 64 m x 16 n x 32 o or 64 m x 8 n x 64 o,
// below); wave w owns the 8 (4, 2) n  8w .. 8w + 7  and all 64 m as 4 row blocks of 16.  Per 32 k it reads the pieces of C (2 x 16 bytes per lane) and of its A rows
// (8 x 16 bytes), and per n the 8 values of B that match its 8 k (2 x 16 bytes, the same for the
// 16 lanes of a row block).  B is copied once into a padded array in the workspace (rows to 32,
// k to 32 plus what the walk copies ahead), so that everything the walk touches exists and all of
// it arrives in LDS by global_load_lds_dwordx4, three steps in three buffers, as in
// gram_f16_wide.hpp (the copies are inline instructions for the reason given there).
//
// Measured at M = K = 8192, N = 512, O = 16: 3.86 ms (O = 32 on the second shape 5.4 ms, O = 64 on the third 9.2 ms) for this kernel and 0.33 ms for the row kernels
// against 9.85 ms on the fp32 kernels.  Counters: 2.5 vector instructions per (m, n, k) (the
// compiler fuses AND and XOR into v_bitop3_b32), the matrix pipeline busy 46 % and the vector
// pipeline about 44 % of the elapsed cycles, hardly ever together, shader clock 1.75 GHz.  Tried
// against that and not kept: matrix instructions alternating between two accumulators (3.99 ms,
// the same), a software pipeline that makes the pieces of the next (n, row block) between the three
// matrix instructions of this one, pinned with scheduling groups (co-issue rises to 47 % of the
// matrix cycles, but the kernel takes more cycles: 4.1 .. 4.3 ms), D parked in LDS to free registers.
// Two compile-time switches leave a part of the walk out, for the measurement of what bounds it (the results are
// then wrong): -DNGF_ABLATE_NO_SIGN multiplies the pieces of A as they are, -DNGF_ABLATE_NO_MFMA makes the signed
// pieces and issues no matrix instruction.  Measured with them at M = K = 8192, N = 512, O = 16: matrix instructions and
// copies alone 2.01 ms (3.46e6 cycles at 1.72 GHz, the matrix pipeline busy 91 % of them), sign work and copies alone
// 2.04 ms (4.17e6 cycles at 2.05 GHz), both 3.72 ms (6.83e6 cycles at 1.84 GHz): the two parts take nine tenths of
// the sum of their cycles, whichever wave they come from -- a source-level pipeline that puts the vector work of pair
// i + 1 between the three dependent matrix instructions of pair i (one matrix instruction, seven vector instructions,
// three times; 255 registers) took 4.28 ms against 4.12 ms on the same box.  This 16-bit matrix instruction and the
// vector ALU do not run side by side here; the kernel is at the sum of two floors, each already at its minimum of
// instructions (2.5 vector instructions per (m, n, k) without packed fp32; three piece products).
#pragma once

#include "gram_f16_wide.hpp"
#include "norm_gradient.hpp"

namespace kmc {

typedef float ngf_float4 __attribute__((ext_vector_type(4)));

constexpr int NGF_TILE_M = 64;
constexpr int NGF_STEP_K = 32;                 // two slices of the split
constexpr int NGF_THREADS = 256;
constexpr int NGF_AHEAD = 3;                   // steps copied ahead of the walk
constexpr int NGF_N_PAD = 32;                  // rows of the padded copy of B come in whole multiples of this

// Three shapes of the workgroup's tile, 64 m in all: 32 n x 16 o (O_BLOCKS = 1), 16 n x 32 o
// (O_BLOCKS = 2) and 8 n x 64 o (O_BLOCKS = 4).  The signed pieces of A are made once per (m, n, k)
// and meet every block of 16 outputs, so with more outputs the wider shapes divide the vector work
// per result, which is what bounds the first (17 to 32 outputs: one pass instead of two of 16).
template <int O_BLOCKS>
struct GradientF16Tile {
    static constexpr int TILE_N = 32 / O_BLOCKS;
    static constexpr int TILE_O = 16 * O_BLOCKS;
    static constexpr int WAVE_N = TILE_N / 4;
    static constexpr int A_CHUNKS = 8 * NGF_TILE_M;    // per step: 8 runs (slice, piece, half) of 64 rows
    static constexpr int C_CHUNKS = 8 * TILE_O;
    static constexpr int B_CHUNKS = TILE_N * NGF_STEP_K / 4;
    static constexpr int BUFFER_CHUNKS = A_CHUNKS + C_CHUNKS + B_CHUNKS;      // 14 KB (17 KB for 64 outputs)
    static constexpr int COPIES = O_BLOCKS == 4 ? 5 : 4;                       // per wave and step
};

struct NormGradientF16Args {
    NormGradientArgs g;                        // extents, d, e, strides, o_chunks (of the tile's outputs); a, b, c are not read
    int o_begin;                               // the launch covers the outputs from here on
    const gram_chunk *pieces_a, *pieces_c;     // gram_f16_split of A (rows m) and of C (rows o)
    i64 pieces_a_bs, pieces_c_bs;              // per batch entry, in chunks
    const float *unscale_a, *unscale_c;
    i64 unscale_a_bs, unscale_c_bs;
    const float *b_padded;                     // [batch][n_pad][k_pad]
    i64 b_padded_bs;
    int rows_pad_a, rows_pad_c, k_pad, steps;
};

struct GradientPadArgs {
    const float *b; i64 b_ld, b_bs;
    float *padded; i64 padded_bs;
    int n, k, n_pad, k_pad;
};

// padded[batch][n][k] = b[batch][n][k], zeros beyond n and k.  One thread per 4 k.
__global__ __launch_bounds__(256) void gradient_pad_b(const GradientPadArgs args)
{
    const int quad = blockIdx.x * 256 + threadIdx.x;
    const int n = blockIdx.y, batch = blockIdx.z;
    if (quad * 4 >= args.k_pad) return;
    const float *src = args.b + batch * args.b_bs + (i64)n * args.b_ld;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = (n < args.n && quad * 4 + e < args.k) ? src[quad * 4 + e] : 0.0f;
    *reinterpret_cast<float4 *>(args.padded + batch * args.padded_bs + (i64)n * args.k_pad + quad * 4) = make_float4(v[0], v[1], v[2], v[3]);
}

template <int O_BLOCKS>
__global__ __launch_bounds__(NGF_THREADS, 2) void norm_gradient_l1_f16(const NormGradientF16Args args)
{
    using Tile = GradientF16Tile<O_BLOCKS>;
    constexpr int WAVE_N = Tile::WAVE_N;
    __shared__ gram_chunk lds0[Tile::BUFFER_CHUNKS];
    __shared__ gram_chunk lds1[Tile::BUFFER_CHUNKS];
    __shared__ gram_chunk lds2[Tile::BUFFER_CHUNKS];

    const NormGradientArgs &g = args.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int q = lane >> 4;     // 8 k of a step (operands), row quad (result)
    const int r = lane & 15;     // row m (T) / column o (C, result)
    const int batch = blockIdx.z / g.o_chunks;
    const int o0 = args.o_begin + (blockIdx.z % g.o_chunks) * Tile::TILE_O;
    const int m0 = blockIdx.x * NGF_TILE_M;
    const int n0 = blockIdx.y * Tile::TILE_N;

    auto buffer = [&](auto which) -> gram_chunk * {
        constexpr int B = decltype(which)::value;
        if constexpr (B == 0) return lds0;
        else if constexpr (B == 1) return lds1;
        else return lds2;
    };

    // Copies per step, four per wave (five for 64 outputs), the same number in every wave so that
    // one count of copies under way serves all.  A: 8 runs of 64 chunks, two per wave.  C: 8 runs of
    // 16, 32 or 64 chunks: with 16, two copies of 4 runs (waves 0 and 2 issue the first, 1 and 3 the
    // second: the same bytes twice); with 32, one copy of 2 runs per wave; with 64, two copies of one
    // run per wave.  B: rows of 128 bytes, 8 per copy: with 32 rows one copy per wave, with 16 rows
    // waves 2 and 3 repeat the copies of waves 0 and 1, with 8 rows every wave issues the one copy.
    // A run (slice, piece, half) of a step starts at chunk ((2 step + slice) * 4 + 2 piece + half) *
    // rows_pad of an operand's pieces.
    typedef const __attribute__((address_space(1))) void *global_address;
    typedef __attribute__((address_space(3))) void *lds_address;
    constexpr int COPIES = Tile::COPIES;
    const gram_chunk *src[COPIES];
    i64 advance[COPIES];
    int dst[COPIES];
    {
        const gram_chunk *pieces_a = args.pieces_a + batch * args.pieces_a_bs + m0;
        const gram_chunk *pieces_c = args.pieces_c + batch * args.pieces_c_bs + o0;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int run = 2 * wave + j;
            src[j] = pieces_a + (i64)run * args.rows_pad_a + lane;
            advance[j] = (i64)8 * args.rows_pad_a;
            dst[j] = run * NGF_TILE_M;
        }
        if constexpr (O_BLOCKS == 4) {
#pragma unroll
            for (int j = 0; j < 2; j++) {                                       // 64 chunks of the step's C each: one run
                const int run = 2 * wave + j;
                src[2 + j] = pieces_c + (i64)run * args.rows_pad_c + lane;
                advance[2 + j] = (i64)8 * args.rows_pad_c;
                dst[2 + j] = Tile::A_CHUNKS + 64 * run;
            }
        } else {
            const int c_copy = O_BLOCKS == 1 ? (wave & 1) : wave;               // 64 chunks of the step's C each
            const int c_run = O_BLOCKS == 1 ? 4 * c_copy + q : 2 * c_copy + (lane >> 5);
            const int c_row = O_BLOCKS == 1 ? r : (lane & 31);
            src[2] = pieces_c + (i64)c_run * args.rows_pad_c + c_row;
            advance[2] = (i64)8 * args.rows_pad_c;
            dst[2] = Tile::A_CHUNKS + 64 * c_copy;
        }
        // 8 rows of B per copy: lane -> row lane / 8, 16 bytes number lane % 8 of the step's 128
        const int b_copy = O_BLOCKS == 1 ? wave : O_BLOCKS == 2 ? (wave & 1) : 0;
        const float *b_row = args.b_padded + batch * args.b_padded_bs + (i64)(n0 + 8 * b_copy + (lane >> 3)) * args.k_pad + 4 * (lane & 7);
        src[COPIES - 1] = reinterpret_cast<const gram_chunk *>(b_row);
        advance[COPIES - 1] = NGF_STEP_K / 4;
        dst[COPIES - 1] = Tile::A_CHUNKS + Tile::C_CHUNKS + 64 * b_copy;
    }
    auto copy_step = [&](auto into) {
#pragma unroll
        for (int j = 0; j < COPIES; j++) {
            const unsigned lds_byte = (unsigned)(unsigned long)(lds_address)(buffer(into) + dst[j]);
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         :
                         : "v"((global_address)src[j]), "s"(lds_byte)
                         : "memory", "m0");
            src[j] += advance[j];
        }
    };

    // D[m, n] of this lane's rows, for the n of the wave.
    float dval[WAVE_N][4];
    {
        const float *d_base = g.d + batch * g.d_bs;
#pragma unroll
        for (int nb = 0; nb < WAVE_N; nb++) {
            const int n = n0 + WAVE_N * wave + nb;
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
                const int m = m0 + 16 * mb + r;
                dval[nb][mb] = (n < g.n && m < g.m) ? d_base[(i64)n * g.d_ld + m] : 0.0f;
            }
        }
    }
    // the copies are not counted by the compiler: nothing it loads may be under way beside them
    __builtin_amdgcn_s_waitcnt(0x0F70);

    ngf_float4 acc[WAVE_N][4][O_BLOCKS];
#pragma unroll
    for (int nb = 0; nb < WAVE_N; nb++)
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int ob = 0; ob < O_BLOCKS; ob++) acc[nb][mb][ob] = ngf_float4{0.0f, 0.0f, 0.0f, 0.0f};

    // lane (q, r): its 8 k are slice q / 2, half q % 2 of the step
    const int run_of_lane = 4 * (q >> 1) + (q & 1);      // + 2 piece
    auto step = [&](auto which) {
        const gram_chunk *lds = buffer(which);
        gram_half8 fc[O_BLOCKS][GW_PIECES], fa[4][GW_PIECES];
#pragma unroll
        for (int ob = 0; ob < O_BLOCKS; ob++)
#pragma unroll
            for (int p = 0; p < GW_PIECES; p++)
                fc[ob][p] = __builtin_bit_cast(gram_half8, lds[Tile::A_CHUNKS + (run_of_lane + 2 * p) * Tile::TILE_O + 16 * ob + r]);
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int p = 0; p < GW_PIECES; p++)
                fa[mb][p] = __builtin_bit_cast(gram_half8, lds[(run_of_lane + 2 * p) * NGF_TILE_M + 16 * mb + r]);
        const float4 *b_rows = reinterpret_cast<const float4 *>(lds + Tile::A_CHUNKS + Tile::C_CHUNKS);
#pragma unroll
        for (int nb = 0; nb < WAVE_N; nb++) {
            const float4 b_low = b_rows[(WAVE_N * wave + nb) * (NGF_STEP_K / 4) + 2 * q];
            const float4 b_high = b_rows[(WAVE_N * wave + nb) * (NGF_STEP_K / 4) + 2 * q + 1];
            const float bk[8] = {b_low.x, b_low.y, b_low.z, b_low.w, b_high.x, b_high.y, b_high.z, b_high.w};
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
                gram_chunk t1 = __builtin_bit_cast(gram_chunk, fa[mb][0]);
                gram_chunk t2 = __builtin_bit_cast(gram_chunk, fa[mb][1]);
#ifndef NGF_ABLATE_NO_SIGN
#pragma unroll
                for (int pair = 0; pair < 4; pair++) {
                    const unsigned low = __float_as_uint(dval[nb][mb] - bk[2 * pair]);
                    const unsigned high = __float_as_uint(dval[nb][mb] - bk[2 * pair + 1]);
                    // the two sign bits, at the sign bits of the two halves of a dword
                    const unsigned flip = __builtin_amdgcn_perm(high, low, 0x070c030c) & 0x80008000u;
                    t1[pair] ^= flip;
                    t2[pair] ^= flip;
                }
                const gram_half8 h1 = __builtin_bit_cast(gram_half8, t1), h2 = __builtin_bit_cast(gram_half8, t2);
#ifdef NGF_ABLATE_NO_MFMA
                asm volatile("" : : "v"(h1), "v"(h2));      // the signed pieces are made and dropped
#else
#pragma unroll
                for (int ob = 0; ob < O_BLOCKS; ob++) acc[nb][mb][ob] = __builtin_amdgcn_mfma_f32_16x16x32_f16(h2, fc[ob][0], acc[nb][mb][ob], 0, 0, 0);
#pragma unroll
                for (int ob = 0; ob < O_BLOCKS; ob++) acc[nb][mb][ob] = __builtin_amdgcn_mfma_f32_16x16x32_f16(h1, fc[ob][1], acc[nb][mb][ob], 0, 0, 0);
#pragma unroll
                for (int ob = 0; ob < O_BLOCKS; ob++) acc[nb][mb][ob] = __builtin_amdgcn_mfma_f32_16x16x32_f16(h1, fc[ob][0], acc[nb][mb][ob], 0, 0, 0);
#endif
            }
        }
#endif
        // the wave's own copies of the next step have arrived (the four of the step after it may
        // still be under way); behind the barrier everybody's have, and this step's buffer is free
        __builtin_amdgcn_s_waitcnt(0x0F70 | COPIES);            // vmcnt(COPIES)
        __syncthreads();
        copy_step(which);
    };

    copy_step(GramStep<0>{});
    copy_step(GramStep<1>{});
    copy_step(GramStep<2>{});
    __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * COPIES));      // vmcnt(2 COPIES): step 0 has arrived
    __syncthreads();
    for (int done = 0;;) {
        step(GramStep<0>{});
        if (++done == args.steps) break;
        step(GramStep<1>{});
        if (++done == args.steps) break;
        step(GramStep<2>{});
        if (++done == args.steps) break;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);

    // acc[nb][mb][ob][j]: m = m0 + 16 mb + 4 q + j, o = o0 + 16 ob + r, n = n0 + WAVE_N wave + nb
#pragma unroll
    for (int ob = 0; ob < O_BLOCKS; ob++) {
        const int o = o0 + 16 * ob + r;
        const float unscale_c = args.unscale_c[batch * args.unscale_c_bs + o];
        float *e_base = g.e + batch * g.e_bs + (i64)o * g.e_ld_o;
#pragma unroll
        for (int mb = 0; mb < 4; mb++) {
            const int m = m0 + 16 * mb + 4 * q;
            const float4 unscale_a = *reinterpret_cast<const float4 *>(args.unscale_a + batch * args.unscale_a_bs + m);
#pragma unroll
            for (int nb = 0; nb < WAVE_N; nb++) {
                const int n = n0 + WAVE_N * wave + nb;
                if (n >= g.n || o >= g.o) continue;
                const ngf_float4 sum = acc[nb][mb][ob];
                const float v[4] = {sum[0] * unscale_a.x * unscale_c, sum[1] * unscale_a.y * unscale_c,
                                    sum[2] * unscale_a.z * unscale_c, sum[3] * unscale_a.w * unscale_c};
                float *dst = e_base + (i64)n * g.e_ld_n + m;
                if (g.e_vec && m + 3 < g.m) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (m + j < g.m) dst[j] = v[j];
                }
            }
        }
    }
}

}  // namespace kmc
