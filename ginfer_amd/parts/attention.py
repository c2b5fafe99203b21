"""Attention over the paged cache: grouped queries, rotary positions, all keys or a window."""
import math

import torch

from ..kernels import ops
from ..kernels.tuning import TUNING
from ..weights.loader import WeightSpec
from .base import Part, KVCacheSpec
from .linear import linear, linear_into_norm
from .registry import register_mixer


def _library_then_rotation_is_faster(rows, in_features):
    """The fused projection kernel cannot split K over workgroups (its epilogue needs whole sums).  Measured on
    MI355X at a 7B model's sizes (K 3584, 4608 outputs): from 17 rows on the BLAS library's product followed by
    the rotation kernel is faster (32 rows: 17.6 us against 20.6; 64 rows: 23.4 against 28.1); at a 1.5B model's
    (K 1536) the fused kernel stays ahead or level up to 64 rows."""
    return rows > TUNING.fused_qkv_up_to_rows and in_features >= TUNING.fused_qkv_unless_in_features


def _projection_in_parts(x, w_qkv, head_dim, rotary_dim):
    """Into how many parts of K the q|k|v product of these rows is split, its parts to be added by the rotation kernel;
    0: not this way.  The fused kernel cannot split K, and each of its workgroups reads all rows of x, which from some
    48 rows on is most of what it reads.  Measured on MI355X in a decode step of 64 rows (2,048 columns of a K of 1,536):
    the fused kernel 13.6 us, the product in four parts 6.7 + the rotation kernel over them 5.9; with fewer rows the fused
    kernel's time falls faster than the pair's (32 rows: 9.2 us)."""
    if isinstance(x, ops.ScaledRows) or x.dtype != torch.bfloat16:
        return 0
    rows, K = x.shape
    if not (TUNING.qkv_in_parts_from_rows <= rows <= ops.SKINNY_MAX_ROWS) or K >= TUNING.fused_qkv_unless_in_features:
        return 0
    if not ops.gemm_skinny_supported(x, w_qkv) or (rotary_dim // 2) % 4 or (head_dim - rotary_dim) % 4 or head_dim % 4:
        return 0
    parts = min(TUNING.qkv_in_parts_most, 8, K // TUNING.qkv_in_parts_min_k)
    return parts if parts >= 2 else 0


@register_mixer("attention")
class Attention(Part):
    """q/k/v projections (one fused product over the stacked weights; results equal the three separate
    ones of ginfer/core/layer/transformer/attention.cc:61-63), rotation of q and k and the cache write
    (:69-72, :32-33), attention over the request's pages (:34), output projection (:80-81).
    score scale 1/sqrt(head_dim) unless `scale` is given; `window` None attends to all earlier keys."""

    capturable = True
    takes_scaled_rows = True
    folds_norm = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, qkv_bias, out_bias, window, position,
                 scale, dtype, device):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads %d is not a multiple of num_kv_heads %d" % (num_heads, num_kv_heads))
        if not 0 < head_dim <= 256:
            raise ValueError("head_dim %d is not supported: the attention kernels take head sizes up to 256 "
                             "(the matrix-core kernels multiples of 16, the general kernel the others)" % head_dim)
        self.hidden_size, self.nh, self.nkv, self.hd = hidden_size, num_heads, num_kv_heads, head_dim
        self.qkv_bias, self.out_bias = bool(qkv_bias), bool(out_bias)
        self.window = int(window) if window else None
        self.position = position
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.dtype, self.device = dtype, device
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    def cache_spec(self):
        return KVCacheSpec(self.nkv, self.hd, self.window)

    def weight_specs(self):
        H, q, kv = self.hidden_size, self.nh * self.hd, self.nkv * self.hd
        specs = {"q_proj.weight": WeightSpec((q, H)), "k_proj.weight": WeightSpec((kv, H)),
                 "v_proj.weight": WeightSpec((kv, H)), "o_proj.weight": WeightSpec((H, q))}
        if self.qkv_bias:
            specs.update({"q_proj.bias": WeightSpec((q,)), "k_proj.bias": WeightSpec((kv,)),
                          "v_proj.bias": WeightSpec((kv,))})
        if self.out_bias:
            specs["o_proj.bias"] = WeightSpec((H,))
        return specs

    def bind_weights(self, t):
        self.w_qkv = torch.cat([t["q_proj.weight"], t["k_proj.weight"], t["v_proj.weight"]], dim=0).contiguous()
        self.b_qkv = (torch.cat([t["q_proj.bias"], t["k_proj.bias"], t["v_proj.bias"]], dim=0).contiguous()
                      if self.qkv_bias else None)
        self.w_o = t["o_proj.weight"]
        self.b_o = t.get("o_proj.bias") if self.out_bias else None

    def kernel_modules(self):
        mods = ["rope_kv", "attention_generic", "gemm"]
        if self.dtype == torch.bfloat16:
            mods += ["gemm_skinny"]
            if self.hd in ops.MFMA_HEAD_DIMS:
                mods += [("attention_mfma", {"HEAD_DIM": self.hd})]
        return mods

    def forward(self, x, step, cache, into_norm=None):
        """into_norm = (residual, norm): where the output projection's kernel can, the result is added to the
        residual here and the rows of `norm` come back as ops.ScaledRows; else the result comes back as ever."""
        cos, sin = self.position.tables()
        parts = _projection_in_parts(x, self.w_qkv, self.hd, self.position.rotary_dim)
        if parts:
            # a decode step of many rows: the product with K split over workgroups (every workgroup then reads a share
            # of the rows only), its 32-bit parts added up by the kernel that rotates and writes the cache
            sums = ops.gemm_skinny(x, self.w_qkv, None, out_dtype=torch.float32, nt=2, grid_splits=parts)
            qkv = ops.rope_kv_from_parts(sums, self.b_qkv, step.positions, cos, sin, cache.slot_mapping, cache.k_pages,
                                         cache.v_pages, self.nh, self.nkv, self.hd, write_kv=cache.owner)
        elif (ops.qkv_rope_skinny_supported(x, self.w_qkv, self.hd, self.position.rotary_dim)
                and not _library_then_rotation_is_faster(x.shape[0], x.shape[1])):
            # few rows (decode): projection, rotation and cache write in one kernel
            qkv = ops.qkv_rope_skinny(x, self.w_qkv, self.b_qkv, step.positions, cos, sin, cache.slot_mapping,
                                      cache.k_pages, cache.v_pages, self.nh, self.nkv, self.hd, write_kv=cache.owner)
        else:
            qkv = linear(x, self.w_qkv, self.b_qkv)
            ops.rope_kv_write(qkv, step.positions, cos, sin, cache.slot_mapping, cache.k_pages, cache.v_pages,
                              self.nh, self.nkv, self.hd, write_kv=cache.owner)
        a = ops.paged_attention(qkv, cache.k_pages, cache.v_pages, cache.block_table, step, self.nh, self.nkv,
                                self.hd, self.scale, self.window)
        if into_norm is not None:
            folded = linear_into_norm(a, self.w_o, self.b_o, *into_norm)
            if folded is not None:
                return folded
        return linear(a, self.w_o, self.b_o, parts_ok=True)
