"""Which kernel a call runs: every threshold, from the two places that own them, and one table.

The library owns the rules for its routes through a workspace (``kmc_gram_workspace_bytes`` and
``kmc_norm_gradient_workspace_bytes`` apply them; ``kmc_dispatch_rules`` prints their thresholds from the one
table they are kept in, ``csrc/host/dispatch_rules.hpp``).  The Python layer owns the choices among the kernels that need no
workspace and the rules of the coefficient product; their thresholds are the module constants named below.  Nothing is
restated here: ``rules()`` reads both, and ``table_markdown()`` fills the sentences of the table with what it read.

    python -m kermac_amd.dispatch          # prints the table
"""
from __future__ import annotations


def rules() -> dict:
    """{name: value}: the library's table (upper-case names) and the Python layer's constants (``module.NAME``)."""
    import importlib
    from . import _backend
    # (the package binds the names cdist_grad and scratch to functions: the modules are asked for by name)
    build_a_kernel, cdist_grad, kernel_coefficients = (importlib.import_module(f"{__package__}.{name}")
                                                       for name in ("build_a_kernel", "cdist_grad", "kernel_coefficients"))

    merged = dict(_backend.dispatch_rules())
    for module, prefixes in ((build_a_kernel, ("_AUTO_", "_CUT_", "_L2_")),
                             (cdist_grad, ("_SPLIT_",)),
                             (kernel_coefficients, ("_AUTO_", "_PANEL_", "_PIECES_", "_FUSED_", "_MANY_", "_SPLIT_"))):
        short = module.__name__.rsplit(".", 1)[-1]
        for name, value in vars(module).items():
            if name.startswith(prefixes) and isinstance(value, (int, float)) and not isinstance(value, bool):
                merged[f"{short}.{name.lstrip('_')}"] = value
    return merged


def _number(value) -> str:
    if isinstance(value, int) and value >= 10_000_000:
        value = float(value)
    if isinstance(value, float) and value == int(value) and abs(value) >= 1e5:
        mantissa, exponent = f"{value:.1e}".split("e")
        mantissa = mantissa.rstrip("0").rstrip(".")
        return f"{mantissa}e{int(exponent)}"
    if isinstance(value, float) and value == int(value):
        return str(int(value))
    return str(value)


_ROWS = (
    # (call, condition, kernel); {NAME} is replaced by the rule of that name
    ("`cdist(p=2)`, `run_kernel` of a DIFF + SQUARE descriptor (L2 norm, Laplace-L2, Gaussian) into a stored matrix; l2 mode "
     "`\"auto\"` (the default)",
     "K < {build_a_kernel.L2_DEFAULT_MIN_K}", "direct `build_kernel<DIFF, SQUARE>`"),
    ("",
     "the library's rule for the workspace route: K ≥ {WIDE_MIN_K}, ≥ {WIDE_MIN_TILES} tiles of 256 × 256 over the batch, "
     "tiles · K ≥ {WIDE_MIN_TILES_TIMES_K} or ≥ {WIDE_TILES_FOR_ANY_K} tiles, per batch entry 2 · tiles_m · tiles_n ≥ "
     "{WIDE_MIN_TILES_PER_SIDE_X2} · (tiles_m + tiles_n), ≤ {WIDE_MAX_PADDING_PERCENT} % of the tiles' area padding; with k contiguous in both "
     "operands instead: K ≥ {WIDE_K_CONTIGUOUS_MIN_K}, ≥ {WIDE_K_CONTIGUOUS_MIN_TILES} tiles, tiles · K ≥ {WIDE_K_CONTIGUOUS_MIN_TILES_TIMES_K}, M and N ≥ "
     "{WIDE_K_CONTIGUOUS_MIN_ROWS}",
     "`gram_row_stats_pair` + `gram_f16_split_pair` (both operands per launch), `gram_probe_operands`, `gram_f16_wide` (fp16 pieces, 256 × 256 tiles), repair launch "
     "of the direct kernel"),
    ("",
     "K ≥ {build_a_kernel.AUTO_ONE_STEP_MIN_K}, trust < 1, "
     "and not (a call the direct path would cut over k on fewer than {build_a_kernel.AUTO_UNCUT_MIN_TILES_K_CONTIGUOUS} tiles of 128 × 128, "
     "{build_a_kernel.AUTO_UNCUT_MIN_TILES} with the rows contiguous)",
     "one-step matrix-core kernel: `gram_l2_kernel` (fp32 matrix instruction) with k contiguous in an operand and K ≥ {build_a_kernel.AUTO_FP32_MIN_K} on "
     "{build_a_kernel.AUTO_FP32_MIN_TILES} … {build_a_kernel.AUTO_FP32_MAX_TILES} tiles over the batch and ≥ {build_a_kernel.AUTO_FP32_MIN_TILES_PER_ENTRY} per entry, "
     "or one dimension ≤ 128 with ≥ {build_a_kernel.AUTO_FP32_MIN_TILES} "
     "tiles; else `gram_bf16_l2_kernel` (three bf16 pieces); from M · N · K · L ≥ {build_a_kernel.L2_SAMPLE_MIN_TERMS} on `gram_probe_operands` in front "
     "of either; repair launch behind"),
    ("", "otherwise", "direct `build_kernel<DIFF, SQUARE>`"),
    ("", "whichever matrix-core kernel runs: the sample of `gram_probe_operands` ({SAMPLE_TILES} tiles of the result, 256 pairs each) shows "
     "{SAMPLE_LEAVE_PER_16384} pairs in 16384 below the trust threshold, spread over the sampled tiles and not packed into few of them",
     "the matrix-core kernel only stamps its parts: the repair launch, i.e. the direct kernel, computes everything"),
    ("`run_kernel` of DOT + NOOP (sums of products) into a stored matrix; l2 mode `\"auto\"`",
     "K ≥ {build_a_kernel.L2_DEFAULT_MIN_K} and the library's rule: K ≥ {DOT_MIN_K}, ≥ {DOT_MIN_TILES} tiles, tiles · K ≥ {DOT_MIN_TILES_TIMES_K}, "
     "≤ {WIDE_MAX_PADDING_PERCENT} % padding; or K ≥ {DOT_LONG_K}, tiles · K ≥ {DOT_LONG_MIN_TILES_TIMES_K}, ≥ {DOT_LONG_MIN_TILES_BATCHED} tiles "
     "over a batch ({DOT_LONG_MIN_TILES_SINGLE} of a single problem)",
     "the workspace route with `gram_f16_wide<GW_EPILOGUE_DOT>` (no trust check, no repair)"),
    ("", "otherwise", "direct `build_kernel<DOT, NOOP>`"),
    ("`cdist(p=1)`, `run_kernel` of DIFF + ABS (L1 norm, Laplace-L1)",
     "l1 mode `\"fixed\"` (opt-in) and ≥ {L1_FIXED_MIN_TILES} tiles of 128 × 128 over the batch, K ≥ {L1_FIXED_MIN_K}",
     "`l1_fixed_range`, `l1_fixed_sample`, `l1_fixed_convert`, `l1_fixed_kernel` (v_sad_u32), repair launch of the direct kernel"),
    ("", "otherwise (the default)", "direct `build_kernel<DIFF, ABS>`"),
    ("any other descriptor (fractional p, signed differences, …)", "always",
     "direct `build_kernel` (ahead of time for DIFF + NOOP/ABS/SQUARE/POW and DOT + NOOP, else compiled on first use); scalar p of 0.5, 1.5, 3, 4 on "
     "the exact-form variants"),
    ("every direct launch",
     "absolute differences, their squares, and the scalar exponents 3 and 4; both operands with m / n contiguous and 16-byte aligned, K and N multiples of 16, K ≥ {DIRECT_SCALAR_B_MIN_K}, "
     "≥ {DIRECT_SCALAR_B_MIN_TILES} tiles of 256 × 64 in every batch entry ({DIRECT_SCALAR_B_MIN_TILES_SYMMETRIC} tiles of one triangle for a set against itself), "
     "not ranges of one contraction, not a repair launch",
     "`build_kernel_scalar_b` (b in scalar registers, only a through LDS; 92 registers, four waves per SIMD)"),
    ("",
     "the same inner terms on operands that kernel cannot take as they are (k contiguous, misaligned, K or N not multiples of 16), "
     "K ≥ {DIRECT_PANELS_MIN_K}, ≥ {DIRECT_PANELS_MIN_TILES} tiles of 256 × 64 in every batch entry ({DIRECT_SCALAR_B_MIN_TILES_SYMMETRIC} of one triangle for a "
     "set against itself, which is copied once), result 16-byte aligned, not ranges of one contraction, and scratch memory allowed",
     "`panel_copy` of each such operand into padded k-major panels, then `build_kernel_scalar_b` on the copies"),
    ("",
     "both operands with m / n contiguous and 16-byte aligned, K ≥ {DIRECT_FOUR_WAVES_MIN_K}, inner power not fractional, not a repair launch",
     "`build_kernel_four_waves` (128 registers, four waves per SIMD; interior tiles copy their slices straight into LDS)"),
    ("", "otherwise", "`build_kernel` (three waves per SIMD; interior tiles of such operands copy straight into LDS all the same)"),
    ("every direct launch, unbatched",
     "fewer than {build_a_kernel.CUT_BELOW_TILES} tiles of 128 × 128 (of one triangle for a set against itself), K ≥ {build_a_kernel.CUT_MIN_K}, and the "
     "launch-time model promises {cut_percent} % (ranges of ≥ {build_a_kernel.CUT_MIN_DEPTH} k)",
     "`build_kernel` on ranges of k as a batch + `finish_partials`"),
    ("`cdist_grad`, p = 1",
     "O ≥ {GRADIENT_F16_MIN_OUTPUTS}, N ≥ {GRADIENT_F16_MIN_N}, terms · O ≥ {GRADIENT_F16_MIN_TERMS_TIMES_OUTPUTS}; with O > 16: terms ≥ "
     "{GRADIENT_F16_MANY_OUTPUTS_MIN_TERMS}",
     "split of a and c, `gradient_pad_b`, `norm_gradient_l1_f16` (64-, 32- or 16-output tiles)"),
    ("`cdist_grad`, p = 2", "a model of both times favours the route by {GRADIENT_L2_ADVANTAGE_PERCENT} %, and the planes of `out` form one matrix",
     "`gradient_l2_products`, splits, `gram_f16_wide<GW_EPILOGUE_GRADIENT_L2>`"),
    ("`cdist_grad`, otherwise", "O ≤ 8 / O > 8", "`norm_kernel_gradient` (vector ALU) / `norm_kernel_gradient_mfma` (fp32 matrix instruction), in runs of 32, 16 and ≤ 8 outputs; "
     "unbatched calls of fewer than {cdist_grad.SPLIT_BELOW_WORKGROUPS} workgroups are cut over k"),
    ("`run_kernel(..., coefficients=)`, squared differences, l2 mode `\"auto\"`",
     "K ≥ {kernel_coefficients.AUTO_PANEL_MIN_K} and (the library's workspace rule for a panel, or K ≥ {kernel_coefficients.AUTO_PANEL_LONG_K}, or K ≥ "
     "{kernel_coefficients.AUTO_PANEL_MID_K} with ≥ {kernel_coefficients.AUTO_PANEL_MID_TILES} tiles — both with {panel_used_percent} % of the tiles' area used — or "
     "O > {kernel_coefficients.AUTO_FUSED_MAX_COLUMNS} with K ≥ {kernel_coefficients.AUTO_PANEL_WIDE_K} and ≥ {kernel_coefficients.AUTO_PANEL_WIDE_TILES} tiles)",
     "panels of the matrix by the workspace route ({panel_mib} MiB, reused), each contracted by `matrix_times_coefficients` (from O ≥ "
     "{kernel_coefficients.PIECES_MIN_COLUMNS} and {kernel_coefficients.PIECES_MIN_TILES} tiles of (o, m) on as a product of fp16 pieces)"),
    ("", "K ≥ {kernel_coefficients.AUTO_FUSED_ANY_SIZE_MIN_K} with O ≤ {kernel_coefficients.AUTO_FUSED_MAX_COLUMNS} (from K = "
     "{kernel_coefficients.AUTO_FUSED_MIN_K} on above {build_a_kernel.L2_AUTO_MIN_TERMS} terms; with more columns only below "
     "{kernel_coefficients.AUTO_FUSED_SMALL_ELEMENTS} elements)", "fused `gram_times_coefficients` (fp32 matrix instruction, repair inside the kernel)"),
    ("", "otherwise", "fused `kernel_times_coefficients`"),
    ("`run_kernel(..., coefficients=)`, any other descriptor",
     "O > {kernel_coefficients.FUSED_COLUMNS_PER_WALK} and L · M · N ≥ {kernel_coefficients.MANY_COLUMNS_MIN_ELEMENTS}",
     "panels of the matrix by `kmc_build_kernel`, each contracted by `matrix_times_coefficients`"),
    ("", "otherwise", "fused `kernel_times_coefficients` (32 or 64 columns per workgroup), the centres in ranges where the launch-time model promises "
     "{ranges_percent} %"),
)


def table_markdown() -> str:
    """The "which kernel runs when" table, every number read from ``rules()``."""
    known = rules()
    known["cut_percent"] = round(100 * (1 - known["build_a_kernel.CUT_WORTH"]))
    known["ranges_percent"] = round(100 * (1 - known["kernel_coefficients.SPLIT_WORTH"]))
    known["panel_used_percent"] = round(100 * known["kernel_coefficients.AUTO_PANEL_MIN_USED"])
    known["panel_mib"] = known["kernel_coefficients.PANEL_BYTES"] >> 20

    import re

    def fill(text):
        def value_of(match):
            name = match.group(1)
            if name not in known:
                raise KeyError(f"the table names a rule that does not exist: {name}")
            return _number(known[name])
        return re.sub(r"\{([A-Za-z0-9_.]+)\}", value_of, text)

    lines = ["| call | condition (the first that holds) | what runs |", "|---|---|---|"]
    for call, condition, kernel in _ROWS:
        lines.append(f"| {call} | {fill(condition)} | {fill(kernel)} |")
    return "\n".join(lines)


if __name__ == "__main__":
    print(table_markdown())
