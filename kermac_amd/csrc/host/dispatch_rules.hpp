// Every threshold by which the library decides, from the shape of a call alone, whether a route
// through a workspace applies, and which variant of the direct kernel is launched.  This table is the only place where these numbers live: the rules
// (launch_one in kernels/build_kernel_inst.hip, wide_pays in kernels/gram_f16_wide_inst.hip, fixed_pays in kernels/l1_fixed_inst.hip, f16_pays in
// kernels/norm_gradient_f16_inst.hip, gradient_l2_pays in kernels/gram_f16_wide_inst.hip) read them
// from here, kmc_dispatch_rules() prints them, and the Python layer builds its "which kernel runs
// when" table from that print-out.  Where each number comes from (the sweeps) is told next to the rule
// that uses it.  A "tile" is 256 x 256 for the matrix-core routes and 128 x 128 for the fixed-point one.
#pragma once

// X(name, value)
#define KMC_DISPATCH_RULES(X)                                                                           \
    /* squared differences through the workspace: tiles over the batch, contraction length */          \
    X(WIDE_MIN_K, 64)                                                                                   \
    X(WIDE_MIN_TILES, 128)                                                                              \
    X(WIDE_MIN_TILES_TIMES_K, 147456)      /* unless there are ... */                                   \
    X(WIDE_TILES_FOR_ANY_K, 768)           /* ... this many tiles */                                    \
    X(WIDE_MIN_TILES_PER_SIDE_X2, 5)       /* 2 tiles_m tiles_n >= 5 (tiles_m + tiles_n), per batch entry */ \
    X(WIDE_MAX_PADDING_PERCENT, 20)        /* of the tiles' area */                                     \
    /* ... both operands with k contiguous: the one-step kernels stage those slowly */                  \
    X(WIDE_K_CONTIGUOUS_MIN_K, 256)                                                                     \
    X(WIDE_K_CONTIGUOUS_MIN_TILES, 48)                                                                  \
    X(WIDE_K_CONTIGUOUS_MIN_TILES_TIMES_K, 36864)                                                       \
    X(WIDE_K_CONTIGUOUS_MIN_ROWS, 129)     /* in both directions */                                     \
    /* sums of products through the workspace (the alternative is the direct kernel) */                 \
    X(DOT_MIN_K, 128)                                                                                   \
    X(DOT_MIN_TILES, 64)                                                                                \
    X(DOT_MIN_TILES_TIMES_K, 65536)                                                                     \
    X(DOT_LONG_K, 256)                     /* from here on, whatever the padding: */                    \
    X(DOT_LONG_MIN_TILES_BATCHED, 32)                                                                   \
    X(DOT_LONG_MIN_TILES_SINGLE, 64)                                                                    \
    X(DOT_LONG_MIN_TILES_TIMES_K, 24576)                                                                \
    /* the sample of the result in front of the matrix-core kernels for squared differences */           \
    X(SAMPLE_TILES, 256)                   /* of 128 x 128, 256 pairs each */                           \
    X(SAMPLE_LEAVE_PER_16384, 2)           /* pairs below the trust threshold, spread over the tiles */ \
    /* the direct kernel compiled for four waves per SIMD (k-major panels, no fractional power) */       \
    X(DIRECT_FOUR_WAVES_MIN_K, 256)                                                                     \
    /* ... and the one with b in scalar registers (absolute and squared differences, K and N multiples of 16): */ \
    /* tiles of 256 x 64 in every batch entry */                                                         \
    X(DIRECT_SCALAR_B_MIN_TILES, 1800)                                                                  \
    X(DIRECT_SCALAR_B_MIN_K, 64)                                                                        \
    X(DIRECT_SCALAR_B_MIN_TILES_SYMMETRIC, 16000)    /* a panel against itself: the tiles of its triangle */ \
    /* ... on copies of operands in any other storage (KMC_FLAG_DIRECT_PANELS): the same tiles, per batch entry */ \
    X(DIRECT_PANELS_MIN_TILES, 5400)                                                                    \
    X(DIRECT_PANELS_MIN_K, 64)                                                                          \
    /* absolute differences on fixed point (KMC_FLAG_L1_FIXED): tiles of 128 x 128 over the batch */    \
    X(L1_FIXED_MIN_TILES, 2048)                                                                         \
    X(L1_FIXED_MIN_K, 128)                                                                              \
    /* the L1 gradient on the fp16 matrix instruction */                                                \
    X(GRADIENT_F16_MIN_OUTPUTS, 3)                                                                      \
    X(GRADIENT_F16_MIN_N, 24)                                                                           \
    X(GRADIENT_F16_MIN_TERMS_TIMES_OUTPUTS, 6400000000LL)     /* up to 16 outputs */                    \
    X(GRADIENT_F16_MANY_OUTPUTS_MIN_TERMS, 15000000)          /* more than 16 outputs */                \
    /* the L2 gradient as one product of pieces: taken when 1.15 x its modelled time is below the fp32 kernels' */ \
    X(GRADIENT_L2_ADVANTAGE_PERCENT, 15)

namespace kmc_rules {
#define KMC_DEFINE_RULE(name, value) constexpr long long name = value;
KMC_DISPATCH_RULES(KMC_DEFINE_RULE)
#undef KMC_DEFINE_RULE
}  // namespace kmc_rules
