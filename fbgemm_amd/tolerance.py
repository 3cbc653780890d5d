"""The bound the tolerance-grade accumulate mode (FBGEMM_AMD_ACC_FAST) is held to, in one place
for the parity tests and for the gate of the benchmark.

The path states its tolerance element by element: fp32 output within 1e-5 relative, fp16 / bf16
output within one unit in the last place. That reading is applied to every element that is not a
cancellation, i.e. not far smaller than the largest |expected| of its bag's block of the output
("the block"). The floor comes from fp32 itself: a sum of n terms carries up to n * 2^-24 of the
magnitudes summed in rounding error whatever the order of the terms, so two orders of the same sum
differ by that much: for bags of tens of rows about 1e-6 of the block (measured for this mode:
6.5e-7), which is 1e-5 of an element an eighth of the block, and less than one unit in the last
place of a 16-bit output down to elements a thousandth of the block.
  fp32:        |got - expected| <= 1e-5 * max(|expected|, 2^-3 * block)
  fp16 / bf16: at most one unit in the last place where |expected| >= 2^-10 * block; below that
               one unit, or the fp32 floor |got - expected| <= 1e-5 * 2^-3 * block.
How many elements were cancellations, and how many of them needed the floor, is counted and reported.
"""
REL = 1e-5
CANCEL_FP32 = 2.0 ** -3    # fp32 output: elements from an eighth of the block on are held to 1e-5 of themselves
CANCEL_16BIT = 2.0 ** -10  # 16-bit output: elements from 2^-10 of the block on are held to one unit in the last place
FLOOR = REL * CANCEL_FP32  # the fp32 rounding floor, relative to the block


def _ordered(bits16, np):
    """16-bit float patterns as integers in value order (neighbours differ by one)."""
    b = bits16.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7fff), b)


def grade(got, want, out_ty, np):
    """got / want: [bags, columns of one table] of fp32 values (out_ty 0) or of uint16 patterns of
    fp16 (1) / bf16 (5). Returns a dict: ok; worst (relative error for fp32, units in the last
    place for 16-bit outputs, over the elements held to the element-wise bound); cancellations (how
    many elements are below the threshold of their output type); needed_block_clause (how many of
    those failed the element-wise bound and passed only by the floor); worst_block (their largest
    error relative to the block's magnitude)."""
    if out_ty == 0:
        g, w = got.astype(np.float64), want.astype(np.float64)
    elif out_ty == 1:
        g, w = got.view(np.float16).astype(np.float64), want.view(np.float16).astype(np.float64)
    else:
        g = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        w = (want.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    finite = np.isfinite(w)
    aw = np.where(finite, np.abs(w), 0.0)
    block = aw.max(axis=1, keepdims=True) if aw.size else aw
    err = np.where(finite, np.abs(np.where(finite, g, 0.0) - np.where(finite, w, 0.0)), 0.0)
    small = finite & (aw < (CANCEL_FP32 if out_ty == 0 else CANCEL_16BIT) * block)
    big = finite & ~small
    if out_ty == 0:
        with np.errstate(divide="ignore", invalid="ignore"):
            rel = np.where(aw > 0, err / np.where(aw > 0, aw, 1.0), np.where(err > 0, np.inf, 0.0))
        passes = rel <= REL
        worst = float(rel[big].max(initial=0.0))
    else:
        ulps = np.abs(_ordered(got, np) - _ordered(want, np))
        passes = ulps <= 1
        worst = int(ulps[big].max(initial=0))
    by_block = err <= FLOOR * block
    needed = small & ~passes
    ok = bool((passes | ~big).all() and (by_block | ~needed).all())
    with np.errstate(divide="ignore", invalid="ignore"):
        wb = np.where(block > 0, err / np.where(block > 0, block, 1.0), 0.0)
    return {"ok": ok, "worst": worst, "cancellations": int(small.sum()), "needed_block_clause": int(needed.sum()),
            "worst_block": float(np.where(needed, wb, 0.0).max(initial=0.0)), "elements": int(finite.sum())}
