"""y = x . W^T (+ b), W stored [out, in] as in the checkpoint (ginfer/core/layer/linear.cc:9-20).

32-bit: the package's own FMA kernel (no matrix unit, no reduced-precision mode).  bfloat16: the
package's matrix-core kernel for up to 64 rows (decode), the BLAS library for more rows (prefill), which
is where the reference calls its library (ginfer/core/op/kernels/cuda/gemm_kernel/gemm_kernel.cu:42-164);
both accumulate in 32-bit and add the bias before the one rounding.  From 17 rows on the library also takes
the products with a wide output, where it was measured faster; replays of recorded steps that hold
these calls are checked bit for bit against eager steps in the tests."""
import torch

from ..kernels import autotune, ops
from ..kernels.tuning import TUNING      # every threshold below is a field of this table, with what it was measured on


def linear(x, weight, bias=None, out_dtype=None, parts_ok=False):
    """x [M, K], weight [N, K], bias [N] | None -> [M, N] in x's dtype (or float32 on request).
    With parts_ok the result may instead be float32 [parts, M, N]: partial sums of a K-split product,
    which the norm that follows adds up in order.  x may be ops.ScaledRows, the rows of a folded norm."""
    if isinstance(x, ops.ScaledRows):
        return ops.gemm_skinny(x, weight, bias, out_dtype=out_dtype, nt=1)
    if x.dtype == torch.float32:
        return ops.gemm_nt(x, weight, bias)
    float32_out = out_dtype == torch.float32
    skinny_ok = ops.gemm_skinny_supported(x, weight)
    plan = None
    if autotune.active():
        key = ("linear", autotune.rows_class(x.shape[0]), weight.shape[0], x.shape[1], bias is not None, float32_out,
               bool(parts_ok), skinny_ok)
        plan = autotune.choose(key, (weight, bias))
    if plan is None:
        plan = linear_plan(x.shape[0], weight.shape[0], x.shape[1], bias is not None, float32_out, parts_ok, skinny_ok)
    return run_linear_plan(plan, x, weight, bias, out_dtype)


def linear_plan(rows, out_features, in_features, has_bias, float32_out, parts_ok, skinny_ok):
    """The way a bfloat16 product is done, by the rules: ("skinny", tiles of W per wavefront, parts of K) for the
    package's weight-streaming kernel, ("library", pieces of K) for the BLAS library.  More than one part or piece
    means float32 partial sums [parts, M, N] for the consumer to add."""
    may_split = parts_ok and not float32_out
    if may_split and not has_bias:
        measured = TUNING.measured_plans.get("%d,%d,%d" % (autotune.rows_class(rows), out_features, in_features))
        if measured is not None and (skinny_ok or measured[0] != "skinny"):
            return tuple(measured)
        pieces = _library_long_k_pieces(rows, out_features, in_features)
        if pieces > 1:
            return ("library", pieces)
    if skinny_ok and not _library_is_faster(rows, out_features):
        # tilings measured on MI355X (graph replays, weights not cache-resident): up to 16 rows one
        # 16-row tile of W per wavefront streams best; beyond, four tiles halve the re-reading of x; a
        # long K is split over workgroups where the consumer can add the parts
        if may_split and in_features >= TUNING.split_k_min_in_features:
            nt, splits = _split_plan(rows, out_features, in_features)
            if splits > 1:
                return ("skinny", nt, splits)
        return ("skinny", 4 if (rows > 16 and out_features >= TUNING.four_tiles_min_out_features) else 1, 1)
    if may_split and not has_bias:
        parts = _library_split(rows, out_features, in_features)
        if parts > 1:
            return ("library", parts)
    return ("library", 1)


def run_linear_plan(plan, x, weight, bias, out_dtype):
    if plan[0] == "skinny":
        _, nt, splits = plan
        if splits > 1:
            return ops.gemm_skinny(x, weight, bias, out_dtype=torch.float32, nt=nt, grid_splits=splits)
        return ops.gemm_skinny(x, weight, bias, out_dtype=out_dtype, nt=nt)
    _, parts = plan
    if parts > 1:
        # the library, once, over `parts` pieces of K side by side (a batched product over views of x and
        # the weight): float32 partial sums for the norm that follows, and work for all of the chip
        M, K = x.shape
        kc = K // parts
        xv = x.as_strided((parts, M, kc), (kc, x.stride(0), 1))
        wv = weight.as_strided((parts, kc, weight.shape[0]), (kc, 1, K))
        return torch.bmm(xv, wv, out_dtype=torch.float32)
    if out_dtype == torch.float32:
        y = torch.mm(x, weight.t(), out_dtype=torch.float32)
        if bias is not None:
            y += bias
        return y
    if bias is not None:
        return torch.addmm(bias, x, weight.t())
    return torch.mm(x, weight.t())


def linear_candidates(key):
    """Every plan that does the product of an autotune key; the plan by the rules first."""
    _, rows, out_features, in_features, has_bias, float32_out, parts_ok, skinny_ok = key
    plans = [linear_plan(rows, out_features, in_features, has_bias, float32_out, parts_ok, skinny_ok)]

    def add(plan):
        if plan not in plans:
            plans.append(plan)

    may_split = parts_ok and not float32_out
    if skinny_ok:
        tiles = (1, 4) if rows > 16 else (1,)
        for nt in tiles:
            add(("skinny", nt, 1))
        if may_split and in_features >= TUNING.split_k_min_in_features:
            steps = -(-in_features // 64)
            for parts in (2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16):
                if parts <= min(TUNING.max_split_k_parts, steps // 8) and steps % parts == 0:
                    for nt in tiles:
                        add(("skinny", nt, parts))
    add(("library", 1))
    if may_split and not has_bias:
        for parts in (2, 3, 4, 5, 7, 8, 10, 14, 16):
            if in_features % parts == 0 and (in_features // parts) % 8 == 0 and in_features // parts >= 512:
                add(("library", parts))
    return plans


def _linear_timing(key, operands, device):
    """For the tuner: the product on random rows, followed, where it may come in parts, by the norm that adds them
    (more parts cost that norm more to read)."""
    _, rows, out_features, in_features, _, float32_out, parts_ok, _ = key
    x = (torch.randn((rows, in_features), device=device) * 0.5).to(torch.bfloat16)
    residual = torch.zeros((rows, out_features), dtype=torch.float32, device=device) if parts_ok else None
    gain = torch.ones((out_features,), dtype=torch.bfloat16, device=device) if parts_ok else None

    def run(plan, i):
        weight, bias = operands[i]
        y = run_linear_plan(plan, x, weight, bias, torch.float32 if float32_out else None)
        if parts_ok:
            ops.add_rmsnorm(residual, y, gain, 1e-6, torch.bfloat16)
    return run


autotune.register_kind("linear", linear_candidates, _linear_timing)


def _split_plan(rows, out_features, in_features):
    """(tiles of W per wavefront, parts of K) for a product whose consumer adds partial sums.  Measured on
    MI355X at the sizes of a 1.5B and a 7B model: the kernel wants some 250 workgroups with four tiles per
    wavefront (more than 16 rows, and enough columns) or some 500 with one, and parts of equal length: the count
    of parts divides K's steps of 64 (down projection of the 1.5B shape at 64 rows: 10 parts 14 us, 11 parts
    23 us).  That gives 10 parts at 64 rows and 5 at 8 for the 1.5B shape's down projection, 4 for the 7B
    shape's; a product with a short K and few columns keeps 2 parts."""
    steps = -(-in_features // 64)
    cap = max(1, min(TUNING.max_split_k_parts, steps // 8))       # parts that leave every wavefront a step
    tiles4 = -(-out_features // 64)
    if rows > 16 and tiles4 * cap >= 192:
        return 4, _nearest_divisor(steps, 256.0 / tiles4, cap)
    if in_features < TUNING.split_k_from:
        return 1, min(2, cap)
    return 1, _nearest_divisor(steps, 512.0 / -(-out_features // 16), cap)


def _nearest_divisor(n, target, cap):
    """The divisor of n in 1..cap nearest to target (the smaller of two equally near)."""
    best = 1
    for d in range(1, cap + 1):
        if n % d == 0 and abs(d - target) < abs(best - target):
            best = d
    return best


def _library_is_faster(rows, out_features):
    """Measured on MI355X: from 17 rows on, products with a wide output (the gate-up product, the head) run
    faster in the BLAS library than in the weight-streaming kernel, which re-reads x once per 64 outputs."""
    return rows > TUNING.library_from_rows and out_features >= TUNING.library_min_out_features


def _library_long_k_pieces(rows, out_features, in_features):
    """Into how many pieces of K the library's product of a few rows is cut where its one product is slow because K
    is long, or 1 where this rule has nothing to say (measured on MI355X at the layer sizes of models from 3B to 72B;
    the figures stand beside the thresholds in kernels/tuning.py)."""
    T = TUNING
    if rows <= T.library_from_rows or rows > T.library_split_max_rows:
        return 1
    if in_features >= T.library_long_k_from and in_features >= 2 * out_features:
        if out_features < T.library_long_k_min_out_features:
            return 1
        if rows <= T.library_long_k_few_rows:                # the fewest rows: two pieces, and only where the library is taken anyway
            halves = in_features >= T.library_long_k_few_rows_from and out_features >= T.library_min_out_features
            return 2 if halves and in_features % 16 == 0 else 1
        tries = (T.library_long_k_pieces, T.library_long_k_pieces - 1)
        for pieces in tries:                                   # whole steps of 64 first
            if pieces > 1 and in_features % (pieces * 64) == 0:
                return pieces
        for pieces in tries + (5, 4, 2):
            if pieces > 1 and in_features % (pieces * 8) == 0:
                return pieces
        return 1
    if min(out_features, in_features) >= T.library_square_min_features and rows > T.library_long_k_few_rows:
        if out_features < T.library_square_max_out_features:
            tries = (8, 4, 2)
        elif rows >= T.library_square_many_rows:
            tries = (4, 2)
        else:
            return 1
        for pieces in tries:
            if in_features % (pieces * 8) == 0:
                return pieces
    return 1


def _library_split(rows, out_features, in_features):
    """Into how many pieces of K the library's product is cut.  Measured on MI355X: with up to 256 rows, few
    output columns and a long K (the down projection of a busy decode step) the library's single product leaves
    a quarter of the chip idle and takes 31 us where five pieces side by side take 23.  A prompt portion's rows
    gain less, while the float32 parts cost the norm more to read: four pieces take the down projection of the 1.5B
    shape and the norm after it from 50.7 to 39.0 us at 1,024 rows and from 76.0 to 69.8 at 2,048 (the library's one
    product makes 264 tiles for 256 compute units there); at 4,096 rows nothing is gained."""
    if in_features >= TUNING.split_k_from and out_features > TUNING.library_split_max_out_features:
        # more columns than that: only a long K, and only the shorter portions, in halves (5,120 columns of a K of 13,824:
        # 512 rows 127 -> 98 us, 1,024 rows 168 -> 143; 8,192 columns of a K of 29,568: 347 -> 256 and 381 -> 378;
        # at 2,048 rows one product is the fastest of all)
        long_k = in_features >= TUNING.library_long_k_from and in_features >= 2 * out_features
        if long_k and TUNING.library_split_max_rows < rows <= TUNING.library_split_wide_max_rows and in_features % 16 == 0:
            return 2
        return 1
    if not (in_features >= TUNING.split_k_from and out_features <= TUNING.library_split_max_out_features):
        return 1
    if TUNING.library_split_min_rows <= rows <= TUNING.library_split_max_rows:
        tries = (5, 4, 2)
    elif TUNING.library_split_max_rows < rows <= TUNING.library_split_portion_max_rows:
        tries = (4, 2)
    else:
        return 1
    for parts in tries:
        if in_features % parts == 0 and (in_features // parts) % 8 == 0:
            return parts
    return 1


def linear_into_norm(x, weight, bias, residual, norm):
    """residual += x . W^T (+ b) in place, and the rows of `norm` over the new residual as ops.ScaledRows: the
    product's kernel folds the add and the norm, so neither makes a pass over memory of its own.  None where
    the kernel does not take these operands (more than 16 rows, 32-bit, odd sizes, a norm that is no plain
    root-mean-square norm with a gain): the caller then takes the ordinary way."""
    if not getattr(norm, "foldable", False) or x.dtype != torch.bfloat16 or residual is None:
        return None
    if (x.shape[1] >= TUNING.split_k_from and x.shape[0] > TUNING.fold_long_k_up_to_rows
            and weight.shape[0] < 16 * TUNING.fold_min_workgroups):
        return None      # a long K and few columns: the split over workgroups is worth more than the folded norm
    if not ops.folded_norm_supported(x, weight, residual, norm.weight):
        return None
    return ops.gemm_skinny(x, weight, bias, into_norm=(residual, norm.weight, norm.eps))


def gated_linear(x, weight_gate_up):
    """silu(x . Wg^T) * (x . Wu^T) with Wg over Wu stacked in one matrix [2I, K] -> [M, I].  x may be
    ops.ScaledRows."""
    if isinstance(x, ops.ScaledRows):
        return ops.gemm_skinny(x, weight_gate_up, gated=True)
    skinny_ok = x.dtype == torch.bfloat16 and ops.gemm_skinny_supported(x, weight_gate_up)
    transposable = _transposable(x, weight_gate_up)
    plan = None
    if autotune.active() and x.dtype == torch.bfloat16:
        key = ("gated", autotune.rows_class(x.shape[0]), weight_gate_up.shape[0], x.shape[1], skinny_ok, transposable)
        plan = autotune.choose(key, (weight_gate_up,))
    if plan is None:
        plan = gated_plan(x.shape[0], weight_gate_up.shape[0], skinny_ok, transposable)
    return run_gated_plan(plan, x, weight_gate_up)


def gated_plan(rows, out_features, skinny_ok, transposable):
    """By the rules: ("skinny",) the weight-streaming kernel with the activation in its epilogue; ("transposed",) the
    library with the weights as its first operand, which leaves the product transposed, [2I, M], and the activation on
    that; ("library",) the usual product and the activation."""
    if skinny_ok and not _library_is_faster(rows, out_features):
        return ("skinny",)
    if transposable and _transposed_product_is_faster(rows):
        return ("transposed",)
    return ("library",)


def run_gated_plan(plan, x, weight_gate_up):
    if plan[0] == "skinny":
        return ops.gemm_skinny(x, weight_gate_up, gated=True)
    if plan[0] == "transposed":
        return ops.silu_mul_transposed(torch.mm(weight_gate_up, x.t()))
    return ops.silu_mul(linear(x, weight_gate_up))


def gated_candidates(key):
    _, rows, out_features, _, skinny_ok, transposable = key
    plans = [gated_plan(rows, out_features, skinny_ok, transposable)]
    for plan, ok in ((("skinny",), skinny_ok), (("library",), True), (("transposed",), transposable)):
        if ok and plan not in plans:
            plans.append(plan)
    return plans


def _gated_timing(key, operands, device):
    _, rows, _, in_features, _, _ = key
    x = (torch.randn((rows, in_features), device=device) * 0.5).to(torch.bfloat16)
    return lambda plan, i: run_gated_plan(plan, x, operands[i][0])


autotune.register_kind("gated", gated_candidates, _gated_timing)


def _transposable(x, weight):
    """Whether the library can take the weights as its first operand for these operands (any row count)."""
    return (x.dtype == torch.bfloat16 and x.is_contiguous() and weight.shape[0] % 16 == 0 and x.shape[1] % 8 == 0
            and x.shape[0] % 8 == 0)


def _transposed_product_is_faster(rows):
    """Measured on MI355X at the 1.5B, 7B and 72B shapes' gate-up product: with a number of rows that is a multiple of
    256 (the portions that a token budget of 2,048 cuts) the library's tiles fit the rows when the weights are its
    first operand: level to 15 % faster (2,048 rows of the 1.5B shape: 115 -> 98 us; 256 rows, a decode step of 256
    requests: 3 to 8 %); with other row counts it is up to 20 % slower, so they keep the usual product."""
    every = TUNING.transposed_gate_up_row_multiple
    return rows >= every and rows % every == 0
