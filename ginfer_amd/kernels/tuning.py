"""Where a step's work goes: every threshold by which a part or a kernel dispatcher chooses between two ways of doing
the same thing lives here, in one table, with what it was measured on.  They decide speed only, never results (beyond
rounding in bfloat16): any setting gives right answers.  The values were measured on one MI355X (256 compute units) at
the layer sizes of a 1.5B and a 7B model; a model of other sizes may want others:

    from ginfer_amd.kernels.tuning import TUNING
    TUNING.library_from_rows = 32                       # for the process
    GINFER_AMD_TUNING='{"library_from_rows": 32}'       # or from the environment, as JSON

No part or dispatcher in Python holds such a number of its own.  What the kernels fix when they are compiled is not in
this table: the wavefronts of an attention workgroup (`PREFILL_WAVES`, `DEC_WAVES`), how late the running maximum of the
softmax is raised (`LAZY_MAX`) and the like are macros at the top of the source that uses them, each with its
measurement; and how a launcher lays ONE kernel over the chip for the sizes it is given (packed tiles, the columns a
workgroup owns where a product is dealt evenly to the compute units: `auto_pack`, `fold_cols`, `gated_even_workgroups`
in csrc/gemm_skinny.hip) is a rule in that source, beside the figures it was measured with.
"""
import json
import os
from dataclasses import dataclass, field, fields


@dataclass
class Tuning:
    # ---- bfloat16 products (parts/linear.py).  Up to 64 rows the package's weight-streaming kernel can take a product,
    # beyond that only the BLAS library.
    # From more rows than this, products with at least `library_min_out_features` output columns (gate-up, the head) go
    # to the library: the streaming kernel re-reads the rows once per 64 columns.
    library_from_rows: int = 16
    library_min_out_features: int = 4096
    # With more than 16 rows and at least this many output columns the streaming kernel takes four tiles of the weight
    # per wavefront, which halves the re-reading of the rows.
    four_tiles_min_out_features: int = 4096
    # A product whose consumer can add partial sums splits a K of at least `split_k_min_in_features` over workgroups
    # (a shorter K only in two parts); at most `max_split_k_parts` parts.
    split_k_from: int = 4096
    split_k_min_in_features: int = 1024
    max_split_k_parts: int = 16
    # A product that folds the norm after it cannot split K over workgroups.  With a K of `split_k_from` or more it still
    # folds up to this many rows (packed tiles fill the chip), and beyond only if its full tiles make at least
    # `fold_min_workgroups` workgroups.
    fold_long_k_up_to_rows: int = 8
    fold_min_workgroups: int = 192
    # The library's product of 65 to 256 rows with a K of at least `split_k_from` and at most this many output columns
    # is cut into pieces of K side by side (a batched product): one product leaves a quarter of the chip idle.
    library_split_min_rows: int = 65
    library_split_max_rows: int = 256
    library_split_max_out_features: int = 4096
    # From more than `library_from_rows` rows on, the library's one product is slow where K is long and the rows are few (it
    # does not split K by itself: 5,120 columns of a K of 27,648 at 64 rows 173 us, in eight pieces 75).  A long K (at
    # least `library_long_k_from`, and twice the columns or more) with at least `library_long_k_min_out_features` columns
    # goes to the library in `library_long_k_pieces` pieces (or one fewer where only that cuts K into whole steps of 64),
    # also where the streaming kernel would take it (2,048 columns of a K of 11,008 at 64 rows: 39 -> 30 us); up to
    # `library_long_k_few_rows` rows only a K of `library_long_k_few_rows_from` or more with `library_min_out_features`
    # columns, and in two pieces (5,120 columns of a K of 27,648 at 32 rows: 163 -> 94 us; more pieces lose there).  Measured at the down projections
    # of the 3B, 7B, 14B, 32B and 72B shapes at 32 to 256 rows: 5 to 64 % less time than the plan before, the 7B shape's
    # 64 rows aside (59 against 60 us; its own best is below).  A product about as long as it is wide with
    # `library_square_min_features` columns and elements of K or more takes eight pieces beyond `library_long_k_few_rows`
    # rows while it has under `library_square_max_out_features` columns, and four pieces from 128 rows on beyond that
    # (5,120 squared: 5 to 34 % less; 8,192 squared at 256 rows 91 -> 62 us).
    library_long_k_from: int = 8192
    library_long_k_min_out_features: int = 2048
    library_long_k_pieces: int = 8
    library_long_k_few_rows: int = 32
    library_long_k_few_rows_from: int = 16384
    library_square_min_features: int = 4096
    library_square_max_out_features: int = 8192
    library_square_many_rows: int = 128
    # Sizes at which the library's own choice of kernel makes an exception of one plan: "class of the row count,output
    # columns,elements of K" of a product whose consumer adds partial sums -> the plan measured fastest there, which
    # stands before the rules (found with --autotune at the 7B shape: decode at batch 64 7.57 -> 7.20 ms a step).
    measured_plans: dict = field(default_factory=lambda: {
        "64,3584,18944": ("library", 2), "64,3584,3584": ("library", 2), "128,3584,3584": ("library", 2)})
    # The same for the rows of prompt portions up to this many, in four pieces (the float32 parts cost the norm that
    # adds them more to read, so the gain is smaller and ends at 4,096 rows).
    library_split_portion_max_rows: int = 2048
    # with more output columns than `library_split_max_out_features`, a long K (as above) goes in halves up to this many rows
    library_split_wide_max_rows: int = 1024
    # The gate-up product lies transposed (weights as the library's first operand) for row counts from this on that
    # are a multiple of it: the library's tiles then fit the rows.
    transposed_gate_up_row_multiple: int = 256
    # ---- the fused q|k|v projection + rotation + cache write (parts/attention.py): from more rows than this and a K
    # of at least that, the library's product followed by the rotation kernel is faster (the fused kernel cannot split K).
    fused_qkv_up_to_rows: int = 16
    fused_qkv_unless_in_features: int = 3072
    # With a shorter K than that, from this many rows on the product goes to the weight-streaming kernel with K split over
    # workgroups, into K // `qkv_in_parts_min_k` parts (at most `qkv_in_parts_most`), which the rotation kernel adds up
    # (2,048 columns of a K of 1,536 in a decode step of 64 rows: the fused kernel 13.6 us, product 6.7 + rotation over the
    # parts 5.9; decode at batch 64 18,340 -> 18,450 tok/s, at batch 48 15,760 -> 15,900).
    qkv_in_parts_from_rows: int = 48
    qkv_in_parts_min_k: int = 384
    qkv_in_parts_most: int = 4
    # ---- attention on the matrix cores (kernels/ops.py)
    decode_target_workgroups: int = 256      # key splits are chosen so that a decode step makes about this many workgroups
    decode_min_split_keys: int = 128         # one tile of 32 keys for each wavefront of a workgroup
    decode_max_splits: int = 256
    # tokens in a step from which prompt rows go 32 to a wavefront (12 heads in 2 groups of 128, one prompt alone: 1,024
    # tokens 20.9 us with 16 rows, 24.8 with 32; 1,536: 27.2 and 29.8; 2,048: 39.4 and 38.1; 4,096: 110 and 82)
    prefill_wide_tiles_from: int = 2048
    # heads of a kv group go side by side into a prefill workgroup only while the step still makes `prefill_fill_workgroups`
    # workgroups; among the groupings that do, the one with the most heads that still makes `prefill_prefer_workgroups`
    # (one and a half rounds of the chip), else the one with the fewest heads
    prefill_fill_workgroups: int = 256
    prefill_prefer_workgroups: int = 384
    # The keys of a step's heaviest prompt tiles can be dealt to several workgroups (merged by a second kernel): when the
    # step makes at most `prefill_split_max_workgroups` workgroups, the heaviest tile's walk is at least
    # `prefill_split_min_key_tiles` tiles of 32 keys long per stream of its workgroup, and longer than
    # `prefill_split_imbalance` times a compute unit's mean share.  0 (the default): never.  Measured with 1.5 at one prompt
    # alone in a step, 12 heads in 2 groups of 128: 2,048 tokens 40.8 us whole, 45.6 in parts; 7B's heads 69.4 and 70.6.
    prefill_split_max_workgroups: int = 512
    prefill_split_min_key_tiles: int = 12
    prefill_split_imbalance: float = 0.0
    # ---- the general attention kernels (the 32-bit path, odd head or page sizes; csrc/attention_generic.hip).  A step that
    # makes no more workgroups of a token and a kv head than this goes whole to the kernel for single tokens (measured at
    # contexts of 512 and 4,096: 12 heads in 2 groups up to 256 tokens); the kernel for portions takes as many wavefronts
    # to a workgroup as still leave `generic_fill_workgroups` workgroups (one and a half to a compute unit).
    generic_few_tokens_workgroups: int = 512
    generic_fill_workgroups: int = 384
    # ---- recorded steps (engine/runner.py): steps with prompt portions are laid into recorded steps of padded sizes up
    # to `mixed_graph_max_tokens` rows, fewer for large models: padding pays while rows x weights stays under what the
    # device does in the time the host needs to launch a step kernel by kernel.
    mixed_graph_max_tokens: int = 512
    padded_rows_times_weights: float = 1.5e12
    # decode batches up to `graph_max_rows` requests are recorded, a shape the `graph_after`-th time it is seen, and the
    # `graph_keep` most recently used recorded shapes are kept
    graph_max_rows: int = 256
    graph_after: int = 2
    graph_keep: int = 128
    # ---- the engine's warm-up (engine/engine.py): prompt portions of these lengths run once before the first request
    # (the BLAS library picks other kernels for other numbers of rows and loads each at its first use); the ones under
    # `warmup_record_below` run three times, so that the padded step a lone prompt of about that length is laid into is
    # recorded and replayed before a request pays for it
    warmup_portion_lengths: tuple = (2048, 1024, 512, 400, 256, 160, 96, 48, 8)
    warmup_record_below: int = 512

    def update(self, values):
        known = {f.name: f.type for f in fields(self)}
        for k, v in values.items():
            if k not in known:
                raise KeyError("no tuning value %r (known: %s)" % (k, ", ".join(sorted(known))))
            if isinstance(getattr(self, k), dict):
                v = {str(size): tuple(plan) for size, plan in dict(v).items()}
            setattr(self, k, type(getattr(self, k))(v))


TUNING = Tuning()
if os.environ.get("GINFER_AMD_TUNING"):
    TUNING.update(json.loads(os.environ["GINFER_AMD_TUNING"]))
