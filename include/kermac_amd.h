/*
 * kermac_amd.h -- C ABI of libkermac_amd.so, the MI355X (gfx950) implementation
 * of kermac's fused distance hot path.
 *
 * Everything here is plain C: device pointers travel as `const float *`, the
 * HIP stream as `void *` (a hipStream_t; NULL = the default stream).  All
 * tensors are fp32 and already resident in device memory.  Launches are
 * asynchronous on the given stream; no entry point synchronises or allocates.
 *
 * Every entry point returns 0 on success.  A non-zero return is one of the
 * KMC_ERR_* codes below or (values >= 1000) 1000 + a hipError_t /
 * 2000 + a hiprtcResult; kmc_last_error() then holds a readable message for
 * the calling thread.
 *
 * The citations name the interface in the reference checkout that each entry
 * point stands in for.
 */
#ifndef KERMAC_AMD_H
#define KERMAC_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KMC_ABI_VERSION 2

enum kmc_status {
    KMC_OK = 0,
    KMC_ERR_INVALID_ARGUMENT = 1,   /* bad shape, stride, enum or null pointer */
    KMC_ERR_UNSUPPORTED_VARIANT = 2,/* descriptor not compiled into the library: JIT it */
    KMC_ERR_WRONG_DEVICE = 3,       /* the current device is not a gfx950 */
    KMC_ERR_JIT = 4,                /* hiprtc compilation failed; log in kmc_last_error() */
    KMC_ERR_HIP_BASE = 1000,
    KMC_ERR_HIPRTC_BASE = 2000
};

/* Template-parameter enums of the reference kernels
 * (include/kermac_internal_common.cuh:41-74).  The numeric values are ABI. */
enum kmc_inner_operator { KMC_OP_DIFF = 0, KMC_OP_DOT = 1 };
enum kmc_power_type { KMC_POW_NOOP = 0, KMC_POW_ABS = 1, KMC_POW_SQUARE = 2, KMC_POW_SQRT = 3, KMC_POW_POW = 4 };
enum kmc_kernel_type { KMC_KERNEL_NONE = 0, KMC_KERNEL_LAPLACE = 1, KMC_KERNEL_GAUSSIAN = 2 };
enum kmc_norm_type { KMC_NORM_L1 = 0, KMC_NORM_L2 = 1, KMC_NORM_P = 2 };
/* COL_MAJOR: the row index (m / n) has stride 1, k has stride ld ("K-major
 * panel", storage a[K,M]).  ROW_MAJOR: k has stride 1, rows have stride ld. */
enum kmc_majorness { KMC_COL_MAJOR = 0, KMC_ROW_MAJOR = 1 };

enum kmc_flags {
    /* Use the 32-bit loaders/stores even when the operands are 16-byte aligned
     * (what the reference does without try_to_align). */
    KMC_FLAG_FORCE_SCALAR_ACCESS = 1,
    /* Compute A(m,k) - B(n,k) instead of B(n,k) - A(m,k); only matters for the
     * sign-sensitive inner powers (NOOP, SQRT).  The reference's run_kernel hands its
     * operands over exchanged whenever the result is row-major (its default,
     * src/kermac/build_a_kernel.py:259,323-336), so what its callers see there is
     * first operand minus second; a caller that launches without that exchange sets
     * this flag (and exchanges the regularisation offsets) to get the same values. */
    KMC_FLAG_NEGATE_DIFF = 2,
    /* Only for inner_operator DIFF + inner_power SQUARE: compute the sum of squared
     * differences as |a|^2 + |b|^2 - 2 a.b with the cross term on the matrix cores
     * (fp32 MFMA), then recompute with the direct subtract-square-accumulate kernel
     * every 128 x 128 tile that contains an element below
     * gram_trust * (|a|^2 + |b|^2) (cancellation).  Two launches on the stream.
     * Trusted elements carry a relative error of about sqrt(K) * 2^-24 / gram_trust
     * on the squared distance; repaired tiles are bit-identical to the direct path.
     * kmc_kernel_times_coefficients honours the flag too (in kernel.flags): the kernel
     * values of each tile then come from the matrix cores, and a distrusted tile is
     * recomputed inside the same kernel (one launch).
     * The reference has no such path (include/build_a_kernel.cuh:339-370 is SIMT only). */
    KMC_FLAG_L2_GRAM = 4,
    /* kmc_build_kernel evaluates inner_operator DIFF + inner_power POW with a scalar
     * exponent (p_inner == NULL) of exactly 0.5, 1.5, 3 or 4 as sqrt|x|, |x| sqrt|x|,
     * |x| x^2 and (x^2)^2: no logarithm / exponential per term, 2 to 3.6 times faster
     * and closer to the exact power than the reference's ex2(p * lg2|x|)
     * (include/kermac_internal_common.cuh:139-161).  This flag keeps the generic
     * exp2(p * log2|x|) evaluation for those exponents too. */
    KMC_FLAG_GENERIC_POWER = 8,
    /* kmc_build_kernel notices when both operands are the same panel (a == b, same
     * strides, majorness and extent, equal regularisation offsets) and the inner term
     * does not change when its operands are exchanged (DOT; ABS, SQUARE or POW of a
     * difference).  The result is then symmetric bit for bit, so only the 128 x 128
     * tiles on and below the diagonal are computed and each is stored twice: about
     * half the time for x-against-x matrices.  The reference computes every tile
     * (its Symmetry enum, src/kermac/build_a_kernel.py:35-37, is not used anywhere).
     * This flag switches the shortcut off. */
    KMC_FLAG_NO_SYMMETRY = 16,
    /* kmc_build_kernel only; implies KMC_FLAG_L2_GRAM (same trust rule, same repair
     * launch, same stated tolerance), with the cross term a.b on the bf16 matrix
     * instruction: every fp32 operand is split into three bf16 pieces (exactly: the
     * pieces sum to the operand) while it is staged, and the six largest of the nine
     * piece products are accumulated in fp32.  The error of the cross term stays that of
     * an fp32 dot product (measured 9e-8 |a||b| at K = 1024); the launch takes about two
     * thirds of the fp32 matrix-core time.  The six products are not summed in an order
     * that is symmetric in a and b, so C(m,n) and C(n,m) of an x-against-x matrix agree
     * to rounding only, unless the symmetric shortcut (see KMC_FLAG_NO_SYMMETRY) mirrors
     * them.  kmc_kernel_times_coefficients does not look at this flag. */
    KMC_FLAG_L2_GRAM_BF16 = 32,
    /* With gram_workspace only (ignored by every launch that does not go through it): the
     * workspace still holds the split of `a` that the previous kmc_build_kernel call through this
     * workspace made, for the same a, a_ld, a_bs, a_majorness, m, k, l and gram_centre and with
     * `a` unchanged since; it is not made again.  For callers that build the matrix panel by panel
     * of `b` (the split of `a` is a quarter of the cost of a panel of 2048 rows of b).  The library
     * keeps, per workspace address, what the last split of `a` there was made from, and makes the
     * split again when these fields differ, when the previous call through the workspace took another
     * route, or when it has not seen the workspace before; that the contents of `a` and of the
     * workspace itself are unchanged is the caller's word. */
    KMC_FLAG_GRAM_A_KEPT = 64,
    /* kmc_build_kernel, inner_operator DOT with inner_power NOOP (sum_k a b: linear and polynomial
     * kernels), with gram_workspace: large problems are multiplied on the fp16 matrix instruction
     * from two fp16 pieces per value and a scale per row, in the 256 x 256 tiles of the route that
     * KMC_FLAG_L2_GRAM_BF16 describes (kmc_gram_workspace_bytes says which, and how much memory it
     * wants).  Error below 3 * 2^-22 sum_k |a b| + k * 2^-38 max|a[m]| max|b[n]| (a value below
     * 2^-28 of the largest of its row is kept to 2^-40 of that largest one, not to 2^-22 of
     * itself): the size of the rounding of an fp32 sum of k >= 100 terms; nothing cancels, so
     * nothing is checked or repaired.  Without a workspace, or
     * for a problem the query reports 0 for, the direct kernel runs. */
    KMC_FLAG_DOT_PIECES = 128,
    /* With KMC_FLAG_L2_GRAM_BF16 or KMC_FLAG_DOT_PIECES: the route through gram_workspace for a
     * problem of any size (k >= 1), also where kmc_gram_workspace_bytes would report 0 because the
     * one-step kernels are faster.  For callers whose alternative is not those kernels: the
     * product of a kernel matrix with coefficients taken panel by panel competes with the fused
     * kernel of kmc_kernel_times_coefficients, which walks the matrix several times more slowly. */
    KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE = 256,
    /* kmc_build_kernel, inner_operator DIFF with inner_power ABS (sums of absolute differences: the
     * L1 norm, Laplace-L1), with gram_workspace: large problems are summed on 32-bit fixed point.
     * Both operands are rounded once to a common grid (one power-of-two step per batch entry, from
     * the largest magnitude in both panels; 22 bits for k > 256, 24 for k <= 256, 26 for k <= 64) and
     * the walk adds |qb - qa| with one integer instruction (v_sad_u32) where fp32 takes two; integer
     * sums are exact.  An element is off by at most k grid steps; one whose sum is below
     * k / tolerance steps is not trusted (tolerance = gram_trust when 0 < gram_trust < 1, else 8e-6),
     * its 128 x 128 tile is stamped and the direct kernel recomputes the stamped tiles right behind,
     * as for KMC_FLAG_L2_GRAM.  Data with a NaN or an infinity, and data where a sample of 1024
     * pairs has more than one in 64 below the threshold (outliers that stretch the grid, sets of
     * near-duplicates), go to the direct kernel whole.  Trusted elements carry a relative error
     * below the tolerance; on spread-out data far less than the fp32 kernel's own rounding.
     * kmc_gram_workspace_bytes says which problems take the route (2048 tiles of 128 x 128 over the
     * batch and k >= 128; KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE: any) and how much memory it wants
     * (4 bytes per element of the padded operands).  Without a workspace, or for a problem the
     * query reports 0 for, the direct kernel runs.  Not with k_total.
     * The reference has no such path (include/build_a_kernel.cuh:339-370 is fp32 only). */
    KMC_FLAG_L1_FIXED = 512,
    /* Matrix-core launches for squared differences that are given a workspace first take a sample of
     * the result from the operands (one small launch): 256 tiles of 128 x 128 over the batch, 256
     * pairs (m, n) of each, judged by the trust rule on up to 128 of the k.  Pairs below the
     * threshold that are spread over the sampled tiles mean that nearly every part of the result
     * holds such a pair and would be recomputed by the direct kernel anyway (sets of near-duplicates,
     * tight clusters in any order): from 2 in 16384 on, the matrix-core kernel only stamps its parts
     * and the call costs the direct kernel's time plus little (at M = N = 30000, K = 1024: 32.5 ms
     * instead of 6 + 32; at 2048 x 2048 x 1024 0.19 instead of 0.37 ms).  Pairs packed into few tiles
     * (points stored cluster by cluster) leave the call on the matrix cores.  This flag leaves the
     * sample out: every part is multiplied, checked and, if need be, recomputed. */
    KMC_FLAG_NO_PROBE = 1024,
    /* kmc_build_kernel, inner_operator DIFF with inner_power ABS, SQUARE or a scalar exponent of 3 or 4 on the direct kernel (none of the
     * flags above), with gram_workspace: the fastest direct kernel for large problems (b in scalar registers)
     * takes its operands as k-major panels (rows contiguous, 16-byte aligned, k a multiple of 16, n a multiple
     * of 16).  With this flag the library copies operands stored any other way -- k contiguous as torch
     * allocates them, misaligned views, other k or n -- into such panels in the workspace (padded with zeros:
     * a zero in both operands adds nothing to a sum, padded columns are not stored) and runs that kernel on
     * the copies: one read and one write of each copied operand against 5 to 7 % of the kernel's time.  The
     * sums are the direct kernel's bit for bit.  kmc_gram_workspace_bytes says which calls take the route
     * (5400 tiles of 256 x 64 per batch entry -- 16000 tiles of one triangle for a panel against itself, which
     * is copied once --, k >= 64, an operand that needs a copy, 16-byte aligned c; KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE: any size) and how much memory it wants
     * (4 bytes per element of the padded copies).  Without a workspace, or for a call the query reports 0
     * for, the direct kernels run on the operands as they are.  The reference has one kernel for all
     * storage orders (include/build_a_kernel.cuh:484-539). */
    KMC_FLAG_DIRECT_PANELS = 2048
};

/*
 * Arguments of the fused pairwise-reduction kernel.  Mirrors, field for field,
 * the 21 launch arguments of cute_build_kernel
 * (include/build_a_kernel.cuh:554-566, marshalled at
 * src/kermac/build_a_kernel.py:378-390) plus the 8 template parameters that the
 * reference passes in the kernel name (src/kermac/build_a_kernel.py:52-71).
 *
 *   C[m + n*c_ld + l*c_bs] =
 *       kernel_fn( outer( sum_k inner( B(n,k,l) (-|*) A(m,k,l) ) ) )
 *
 * A(m,k,l) = a[m*1 + k*a_ld + l*a_bs] when a_majorness == KMC_COL_MAJOR,
 *            a[m*a_ld + k*1 + l*a_bs] when KMC_ROW_MAJOR; likewise B.
 * C is always written with m contiguous.  A batch stride of 0 broadcasts.
 *
 * Hyper-parameters (inner power, outer power, bandwidth, regularisation) are
 * either a device pointer read at [l * stride] or, when the pointer is NULL,
 * the by-value field next to it.
 */
typedef struct kmc_build_kernel_params {
    int32_t inner_operator;     /* enum kmc_inner_operator */
    int32_t inner_power;        /* enum kmc_power_type */
    int32_t outer_power;        /* enum kmc_power_type */
    int32_t kernel_type;        /* enum kmc_kernel_type */
    int32_t a_majorness;        /* enum kmc_majorness */
    int32_t b_majorness;
    int32_t flags;              /* enum kmc_flags */
    int32_t m, n, k, l;
    const float *a; int64_t a_ld; int64_t a_bs;
    const float *b; int64_t b_ld; int64_t b_bs;
    float *c;       int64_t c_ld; int64_t c_bs;
    const float *p_inner;        int64_t p_inner_bs;        float p_inner_value;
    const float *p_outer;        int64_t p_outer_bs;        float p_outer_value;
    const float *bandwidth;      int64_t bandwidth_bs;      float bandwidth_value;
    const float *regularization; int64_t regularization_bs; float regularization_value;
    int32_t regularization_offset_x;
    int32_t regularization_offset_y;
    float epsilon;
    float gram_trust;           /* used with KMC_FLAG_L2_GRAM; <= 0 selects 0.25 */
    /* 0, or the length of one contraction whose consecutive ranges are the batch
     * entries of this launch (see kmc_build_kernel_finish): entry l then walks the k
     * terms from l*k on, the last entry only the k_total - (l-1)*k that are left
     * (1 .. k of them; l must be ceil(k_total / k)).  kmc_build_kernel only, not with
     * the matrix-core flags.  No counterpart in the reference. */
    int32_t k_total;
    /* With the matrix-core flags only (ignored otherwise): a point c[k] that is subtracted from
     * both operands while they are staged, read at gram_centre[l * gram_centre_bs + k].
     * Distances do not change; what changes is how much |a|^2 + |b|^2 - 2 a.b cancels, which is
     * in proportion to the norms: with a centre near the data (its mean: kmc_sample_mean) the
     * norms are those of the spread of the data, not of its offset from the origin, and tiles of
     * data with a common offset stay trusted instead of being recomputed.  16-byte aligned, the
     * stride a multiple of 4; each vector is padded with zeros to a multiple of 64 floats and
     * followed by one float that says whether to subtract at all (0: this batch entry is taken
     * as it is; kmc_sample_mean writes all of this).  NULL: nothing is subtracted. */
    const float *gram_centre;
    int64_t gram_centre_bs;
    /* With KMC_FLAG_L2_GRAM_BF16, KMC_FLAG_DOT_PIECES or KMC_FLAG_L1_FIXED (ignored otherwise): device memory the call may use, 256-byte
     * aligned, of at least the size kmc_gram_workspace_bytes reports for these parameters.  With
     * it, large problems take a faster route in three steps (statistics per row, both operands
     * split once into two fp16 pieces per value in the order the matrix instruction reads them,
     * then 256 x 256 tiles on the fp16 matrix instruction; same trust rule, same repair launch,
     * same tolerance: at M = N = 30000, K = 1024 6.1 ms instead of 10).  NULL, too small, or a
     * problem for which kmc_gram_workspace_bytes reports 0: the one-step kernel runs.  The
     * contents after the call do not matter; calls that share a workspace must be ordered.
     * With KMC_FLAG_L2_GRAM or KMC_FLAG_L2_GRAM_BF16 on a problem that runs a one-step kernel, a
     * workspace of at least KMC_SAMPLE_BYTES lets the library look before it multiplies (see
     * KMC_FLAG_NO_PROBE); kmc_gram_workspace_bytes does not ask for it, a caller who wants the
     * sample for every size hands over max(KMC_SAMPLE_BYTES, what the query reports). */
    void *gram_workspace;
    int64_t gram_workspace_bytes;
} kmc_build_kernel_params;

/* Bytes of gram_workspace that kmc_build_kernel would use for these parameters, 0 when it would
 * not use one: none of KMC_FLAG_L2_GRAM_BF16 with squared differences, KMC_FLAG_DOT_PIECES with
 * products and KMC_FLAG_L1_FIXED with absolute differences, or a problem too small to gain by the
 * library's rule for that route.  The rules weigh the tiles over the batch (of a panel against
 * itself: those on and below the diagonal; the panel is split once), the contraction length, tiles
 * in both directions of every batch entry, the share of padding, and whether k is the contiguous
 * index of both operands; their thresholds are the table that kmc_dispatch_rules() prints, the
 * only place where those numbers are kept.  KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE sets the size rules
 * aside.  About 1.1 times the bytes of the operands.  No counterpart in the reference. */
int kmc_gram_workspace_bytes(const kmc_build_kernel_params *params, int64_t *bytes);

/* Stands in for launch(stream, config, cute_build_kernel<...>, *args)
 * (src/kermac/build_a_kernel.py:339-392).  Returns
 * KMC_ERR_UNSUPPORTED_VARIANT when the (inner_operator, inner_power) pair is
 * not among the ahead-of-time compiled ones. */
int kmc_build_kernel(const kmc_build_kernel_params *params, void *stream);

/*
 * Second step of a contraction that the caller cut over k (no counterpart in the
 * reference, whose kernel walks all of k in one workgroup per tile: a 100 x 100
 * result over k = 100000 is a single workgroup there and here).  The caller launches
 * kmc_build_kernel on `slices` ranges of k with outer_power = KMC_POW_NOOP and
 * kernel_type = KMC_KERNEL_NONE into partial results
 *   partials[m + n*partial_ld + l*partial_bs + s*partial_slice]
 * (a batched launch over strided views does all slices at once, with k_total for a
 * shorter last range); this entry point
 * adds the partial results in slice order and applies outer power, epsilon mask,
 * kernel function and regularised diagonal of `params` exactly like
 * kmc_build_kernel, writing C.  `a`, `b` and `k` of `params` are not read.
 */
int kmc_build_kernel_finish(const kmc_build_kernel_params *params, const float *partials, int64_t partial_ld,
                            int64_t partial_bs, int64_t partial_slice, int32_t slices, void *stream);

/*
 * mean[l*mean_bs + k] = the mean over (a sample of) the rows of the panel x (addressed like the a
 * operand of kmc_build_kernel: majorness, ld, batch stride bs), for use as gram_centre.  Panels
 * of up to 4096 rows are averaged whole, longer ones over 16 evenly spaced runs of 256 rows;
 * the sums run in a fixed order.  Per batch entry the call writes 2 * roundup(k, 64) + 64 floats
 * (mean_bs must be at least that for l > 1): the mean padded with zeros to a multiple of 64, a
 * flag in the next float -- 1, or 0 when the mean is so close to the origin against the spread of
 * the rows around it (|mean|^2 <= variance / 64) that subtracting it would change nothing worth
 * its cost; the matrix-core kernels read it -- then 63 unused floats and the variance per k.
 * Two small launches on the stream.  No counterpart in the reference.
 */
int kmc_sample_mean(const float *x, int32_t majorness, int32_t rows, int32_t k, int64_t ld, int64_t bs, int32_t l,
                    float *mean, int64_t mean_bs, void *stream);

/*
 * The cut over k above as one call that allocates nothing.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  `params` describes the
 * whole problem exactly as for kmc_build_kernel (l must be 1, k_total 0, no matrix-core
 * flags, an ahead-of-time compiled (inner_operator, inner_power) pair); k is cut into at
 * most `ranges` ranges of whole 16-term slices, kmc_build_kernel computes their plain sums
 * and kmc_build_kernel_finish adds them in range order and applies the epilogue -- the same
 * two launches, the same bits, as the two-call form with a caller-supplied buffer.  The
 * partial sums live in a static device array of the library: KMC_STATIC_SCRATCH_BYTES on
 * every GPU that runs the library, held until the process ends.  A call whose
 * ceil(k / depth) * n * (m rounded up to 4) floats do not fit is rejected with
 * KMC_ERR_INVALID_ARGUMENT before anything is launched.  No hipMalloc, hipFree or other
 * allocating call is made.  All calls on one GPU share the array: calls on one stream are
 * ordered, calls that overlap on one GPU (two streams, two host threads) race.  The first call on
 * a device looks up the array's address there (once, under a lock): make one eager call per device
 * before capturing calls into a HIP graph.  The stream must belong to the current device.
 */
#define KMC_STATIC_SCRATCH_BYTES (64u << 20)

/* What the sample in front of a matrix-core launch for squared differences takes of gram_workspace
 * (KMC_FLAG_NO_PROBE); the route through the workspace counts it in what kmc_gram_workspace_bytes
 * reports, the one-step kernels use it when the caller hands it over. */
#define KMC_SAMPLE_BYTES 1024
int kmc_build_kernel_cut_static(const kmc_build_kernel_params *params, int32_t ranges, void *stream);

/*
 * Arguments of the fused kernel-gradient contraction; mirrors the 24 launch
 * arguments of cute_norm_kernel_gradient (include/p_norm_gradient.cuh:413-422,
 * marshalled at src/kermac/cdist_grad.py:226-235).
 *
 *   E[m + n*e_ld_n + o*e_ld_o + l*e_bs] =
 *       sum_k C[o*c_ld + k + l*c_bs] * A[m + k*a_ld + l*a_bs]
 *             * g( D[m + n*d_ld + l*d_bs] - B[n*b_ld + k + l*b_bs] )
 *   g(x) = copysign(1,x) (L1), x (L2), copysign(1,x)*|x|^(p-1) (P)
 *
 * p is a device pointer read at [l * p_bs], or by value when NULL.
 */
typedef struct kmc_norm_gradient_params {
    int32_t norm_type;          /* enum kmc_norm_type */
    int32_t flags;
    int32_t m, n, o, k, l;
    const float *a; int64_t a_ld; int64_t a_bs;   /* [k, m], m contiguous */
    const float *b; int64_t b_ld; int64_t b_bs;   /* [n, k], k contiguous */
    const float *c; int64_t c_ld; int64_t c_bs;   /* [o, k], k contiguous */
    const float *d; int64_t d_ld; int64_t d_bs;   /* [n, m], m contiguous */
    float *e; int64_t e_ld_n; int64_t e_ld_o; int64_t e_bs; /* [o, n, m], m contiguous */
    const float *p; int64_t p_bs; float p_value;
    /* KMC_NORM_L1 and KMC_NORM_L2 (ignored otherwise): device memory the call may use, 256-byte
     * aligned, of at least the size kmc_norm_gradient_workspace_bytes reports for these parameters.
     * With it, large problems run on the fp16 matrix instruction.  KMC_NORM_L1: a and c are split once into two fp16 pieces per
     * value (a power-of-two scale per row m of a and per row o of c), the sign of d - b is put on
     * the pieces of a exactly, and the contraction takes 3 matrix instructions per 32 k where the
     * fp32 kernel issues 8 of twice the duration.  Error of e from the pieces below
     * 3 * 2^-22 sum_k |c a|, beside the rounding of the fp32 accumulation that both kernels have.
     * KMC_NORM_L2 with e_ld_o = n * e_ld_n (the planes of e one matrix of o * n rows): large problems
     * run as e = (d - s) g - p a with g[m][o] = sum_k a c, p[o n_rows + n][k] = c[o][k] (b[n][k] - s[n])
     * and s[n] the mean of row n of b (any s gives the same e; this one keeps both terms as small
     * as the data allows): p and a are split once into two fp16 pieces per value with a scale per
     * row and multiplied in 256 x 256 tiles on the fp16 matrix instruction, g comes from the fp32
     * matrix instruction; the workspace also holds p in fp32.  Error of the product from the pieces
     * below 3 * 2^-22 sum_k |c a (b - s)| + k * 2^-38 max_k|a[k][m]| max_k|p[r][k]|.
     * NULL, too small, or a problem for which the query reports 0: the fp32 kernels run. */
    void *workspace;
    int64_t workspace_bytes;
} kmc_norm_gradient_params;

/* Bytes of workspace that kmc_norm_kernel_gradient would use for these parameters, 0 when it would
 * not use one.  KMC_NORM_L1: enough outputs, columns n and terms m * n * k * l (the GRADIENT_F16 lines
 * of kmc_dispatch_rules(); 4e8 terms at 16 outputs), and n within one grid dimension; about 1.1 times the
 * bytes of a, b and c.  KMC_NORM_L2:
 * when a model of both times favours the route by 15 % (tiles of 256 x 256 over m and o * n, in
 * both directions, and a contraction of about 512 or more); about 4 (m + 2 o n) k bytes.
 * KMC_NORM_P: never.  No counterpart in the reference. */
int kmc_norm_gradient_workspace_bytes(const kmc_norm_gradient_params *params, int64_t *bytes);

/* Stands in for launch(stream, config, cute_norm_kernel_gradient<NormType>, *args)
 * (src/kermac/cdist_grad.py:192-237). */
int kmc_norm_kernel_gradient(const kmc_norm_gradient_params *params, void *stream);

/*
 * Fused kernel matrix x coefficients:
 *   out[m*out_ld + o + l*out_bs] = sum_n Kmat(m,n,l) * coef[n*coef_ld + o + l*coef_bs]
 * where Kmat(m,n,l) is exactly the value kmc_build_kernel would have stored at
 * C(m,n,l) for `kernel` (its c, c_ld, c_bs fields are ignored).  The m x n
 * matrix is never written to memory.  The reference has no such kernel
 * (its run_kernel always materialises out[L,M,N],
 * src/kermac/build_a_kernel.py:259,378-392); the semantics are those of
 * run_kernel(...) followed by a matmul with the coefficients.
 */
typedef struct kmc_kernel_coefficients_params {
    kmc_build_kernel_params kernel;
    int32_t o;                                    /* coefficient columns */
    const float *coef; int64_t coef_ld; int64_t coef_bs;  /* [n, o], o contiguous */
    float *out; int64_t out_ld; int64_t out_bs;           /* [m, o], o contiguous */
    /* 0 or 1: one launch computes the whole product.  R > 1: the n rows of b and coef (the
     * centres) are cut into R consecutive ranges of ceil(ceil(n / 128) / R) tiles of 128, every
     * range is walked by workgroups of its own and writes its partial product
     *   out[m*out_ld + o + l*out_bs + r*out_range_stride],
     * and the caller adds the R partial products (in a fixed order, for reproducible results).
     * A workgroup owns 128 rows m and walks every centre of its range, so few rows against
     * many centres, or a batch of problems that fills only two workgroup slots per CU, leave
     * the chip under-used unless the centres are cut.  Everything else, the regularised
     * diagonal included (it is addressed by the global index n), is unchanged. */
    int32_t n_ranges;
    int64_t out_range_stride;
} kmc_kernel_coefficients_params;

/* Coefficient columns are processed in chunks of up to 64 per workgroup (one chunk of 32 for o <= 32);
 * o > 64 works (the kernel values are then recomputed per chunk).  Returns
 * KMC_ERR_UNSUPPORTED_VARIANT when the (inner_operator, inner_power) pair is not
 * among the ahead-of-time compiled ones. */
int kmc_kernel_times_coefficients(const kmc_kernel_coefficients_params *params, void *stream);
/* 1 when (inner_operator, inner_power) is compiled ahead of time for the fused
 * coefficient kernel. */
int kmc_kernel_times_coefficients_has_variant(int32_t inner_operator, int32_t inner_power);
/* Launch a run-time compiled kmc::kernel_times_coefficients instantiation. */
int kmc_kernel_times_coefficients_jit(void *function, const kmc_kernel_coefficients_params *params, void *stream);

/*
 * A stored panel of the kernel matrix times coefficients:
 *   out[m*out_ld + o + l*out_bs] (+)= sum_n matrix[n*matrix_ld + m + l*matrix_bs] * coef[n*coef_ld + o + l*coef_bs]
 * The second half of the kernel matrix x coefficients product when the matrix is built in panels
 * of centres by kmc_build_kernel (c_ld = matrix_ld, m contiguous) instead of inside the fused
 * kernel: for squared differences the matrix-core routes of kmc_build_kernel build a panel
 * several times faster than kmc_kernel_times_coefficients walks it.  The sums run in a fixed
 * order: the same inputs give the same bits.  n = 0 without accumulate stores zeros.  The
 * reference has no such kernel (its run_kernel stops at the stored matrix out[L,M,N],
 * src/kermac/build_a_kernel.py:259,378-392); no library routine and no allocation here.
 */
typedef struct kmc_matrix_coefficients_params {
    int32_t m, n, o, l;
    const float *matrix; int64_t matrix_ld; int64_t matrix_bs;  /* [n, m], m contiguous */
    const float *coef; int64_t coef_ld; int64_t coef_bs;        /* [n, o], o contiguous */
    float *out; int64_t out_ld; int64_t out_bs;                 /* [m, o], o contiguous */
    int32_t accumulate;                                         /* 0: out = product, 1: out += product */
    /* 0 or 1: one product.  S > 1: the n rows are cut into S consecutive ranges, each walked by
     * workgroups of its own into a partial product of its own,
     *   out[m*out_ld + o + l*out_bs + s*out_split_stride],
     * and the caller adds the S partial products in a fixed order (as with n_ranges of
     * kmc_kernel_coefficients_params): a workgroup owns 512 rows m, so few rows against a long
     * panel leave the chip under-used unless the n are cut.  l * S may not exceed 65535. */
    int32_t n_splits;
    int64_t out_split_stride;
} kmc_matrix_coefficients_params;
int kmc_matrix_times_coefficients(const kmc_matrix_coefficients_params *params, void *stream);

/* ---- run-time compilation (stands in for cuda.core Program / ObjectCode:
 *      src/kermac/module_cache/module_cache.py:13-51, 219-239) ---- */

/* Compile `source` for the current device's architecture with hiprtc.
 * `headers`/`header_names` are in-memory include files.  On success *code is a
 * malloc'ed code object of *code_size bytes and lowered_names[i] (malloc'ed
 * strings) is the mangled symbol of name_expressions[i].  Free with
 * kmc_jit_free. */
int kmc_jit_compile(const char *source, const char *source_name,
                    int n_headers, const char *const *headers, const char *const *header_names,
                    int n_options, const char *const *options,
                    int n_names, const char *const *name_expressions,
                    void **code, size_t *code_size, char **lowered_names);
void kmc_jit_free(void *ptr);

/* hipModuleLoadData / hipModuleGetFunction / hipModuleUnload. */
int kmc_module_load(const void *code, size_t code_size, void **module);
int kmc_module_get_function(void *module, const char *lowered_name, void **function);
int kmc_module_unload(void *module);

/* Launch a run-time compiled instance of the kernels above.  `function` must be
 * an instantiation of kmc::build_kernel / kmc::norm_kernel_gradient from the
 * kernel headers shipped with this library, compiled for load modes
 * (load_a, load_b) as reported by kmc_build_kernel_load_modes. */
int kmc_build_kernel_jit(void *function, const kmc_build_kernel_params *params, void *stream);
/* The loader variants (0..3: col-vec, col-scalar, row-vec, row-scalar) that
 * kmc_build_kernel would pick for these operands. */
int kmc_build_kernel_load_modes(const kmc_build_kernel_params *params, int32_t *load_a, int32_t *load_b);

/* ---- misc ---- */
int kmc_abi_version(void);
/* The thresholds of the library's rules for its routes through a workspace (which
 * kmc_gram_workspace_bytes and kmc_norm_gradient_workspace_bytes apply) as text, one
 * "NAME = integer" per line, into buf (4096 bytes are enough).  A tile is 256 x 256 for the
 * matrix-core routes and 128 x 128 for the fixed-point one.  No counterpart in the reference. */
int kmc_dispatch_rules(char *buf, size_t buf_len);
/* Message of the last failing call on this thread ("" if none). */
const char *kmc_last_error(void);
/* gcnArchName of `device` (e.g. "gfx950:sramecc+:xnack-") into buf. */
int kmc_device_arch(int device, char *buf, size_t buf_len);
/* 1 when (inner_operator, inner_power) is compiled ahead of time. */
int kmc_build_kernel_has_variant(int32_t inner_operator, int32_t inner_power);

#ifdef __cplusplus
}
#endif
#endif /* KERMAC_AMD_H */
