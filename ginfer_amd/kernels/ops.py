"""Python faces of the HIP kernels.

Every function checks on the host what its kernel and launch grid assume (devices, dtypes,
contiguity, matching sizes) and raises a clear error instead of launching with operands that do not
fit; a kernel never sees a shape it was not written for.  Tensors are torch tensors on the GPU;
kernels run on torch's current stream.
"""
import ctypes

import torch

from . import build
from .tuning import TUNING

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_f = ctypes.c_float


class KernelError(RuntimeError):
    pass


def _ptr(t):
    return _vp(t.data_ptr()) if t is not None else _vp(0)


def _stream():
    """The raw handle of torch's current stream on the current device (the recording stream while a step is
    being recorded)."""
    return _vp(_raw_stream(_current_device()))


_raw_stream = torch._C._cuda_getCurrentRawStream
_current_device = torch.cuda.current_device


def _check(rc, name):
    if rc != 0:
        raise KernelError("kernel %s failed to launch (code %d)" % (name, rc))


def _need(cond, msg, *args):
    """Raises KernelError(msg % args) unless cond holds; the message is put together only then."""
    if not cond:
        raise KernelError(msg % args if args else msg)


def _dev(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU (got a %s tensor)" % t.device)
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel operands lie on different devices")


def _is_bf16(dtype):
    if dtype is torch.bfloat16:
        return 1
    _need(dtype is torch.float32, "compute dtype must be float32 or bfloat16, got %s", dtype)
    return 0


def embedding_gather(table, ids, out=None):
    """table [V, H] (float32 or bfloat16), ids [T] int32 in [0, V) -> float32 [T, H]."""
    _dev(table, ids, out)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [V, H]")
    _need(ids.dtype == torch.int32 and ids.dim() == 1 and ids.is_contiguous(), "ids must be contiguous int32 [T]")
    T, H = ids.shape[0], table.shape[1]
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (T, H) and out.is_contiguous(), "out must be contiguous float32 [T, H]")
    lib = build.load("embedding")
    _check(lib.ga_embedding_gather(_ptr(out), _ptr(table), _ptr(ids), _i(T), _i(H),
                                   _i(_is_bf16(table.dtype)), _stream()), "embedding_gather")
    return out


def add_rmsnorm(residual, delta, gain, eps, dtype, rows=None, out=None):
    """residual float32 [T, H] (updated in place with + delta unless rows is given); delta [T, H] in
    `dtype`, or float32 [parts, T, H] (partial sums of a K-split product, added in order), or None;
    gain [H] in `dtype` (or float32); rows int32 [R] or None -> normed [R or T, H]."""
    _dev(residual, delta, gain, rows, out)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    T, H = residual.shape
    parts = 0
    if delta is not None and delta.dim() == 3:
        _need(delta.dtype == torch.float32 and delta.shape[1:] == (T, H) and delta.is_contiguous() and delta.shape[0] >= 1,
              "partial sums must be contiguous float32 [parts, %d, %d], got %s %s",
              T, H, delta.dtype, tuple(delta.shape))
        parts = delta.shape[0]
    elif delta is not None:
        _need(delta.dtype == dtype and delta.shape == (T, H) and delta.is_contiguous(),
              "delta must be contiguous %s [%d, %d], got %s %s",
              dtype, T, H, delta.dtype, tuple(delta.shape))
    _need(gain.shape == (H,) and gain.is_contiguous() and gain.dtype in (dtype, torch.float32),
          "gain must be contiguous [%d] in %s or float32",
          H, dtype)
    R = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be contiguous int32 [R]")
        R = rows.shape[0]
    if out is None:
        out = torch.empty((R, H), dtype=dtype, device=residual.device)
    _need(out.dtype == dtype and out.shape == (R, H) and out.is_contiguous(), "out must be contiguous [R, H]")
    lib = build.load("norm")
    _check(lib.ga_add_rmsnorm(_ptr(out), _ptr(residual), _ptr(delta), _i(parts), _i(T), _ptr(gain), _ptr(rows), _i(R), _i(H),
                              _f(eps), _i(_is_bf16(dtype)),
                              _i(1 if (gain.dtype == torch.float32 and dtype != torch.float32) else 0),
                              _stream()), "add_rmsnorm")
    return out


def silu_mul(gate_up, out=None):
    """gate_up [T, 2I] -> [T, I]: silu(gate) * up with gate = [:, :I], up = [:, I:]."""
    _dev(gate_up, out)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0,
          "gate_up must be contiguous [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.dtype == gate_up.dtype and out.shape == (T, I) and out.is_contiguous(), "out must be contiguous [T, I]")
    lib = build.load("activation")
    _check(lib.ga_silu_mul(_ptr(out), _ptr(gate_up), _i(T), _i(I), _i(_is_bf16(gate_up.dtype)), _stream()),
           "silu_mul")
    return out


def silu_mul_transposed(gate_up_t, out=None):
    """gate_up_t [2I, T] (the gate-up product lying transposed) -> [T, I]: silu(gate) * up."""
    _dev(gate_up_t, out)
    _need(gate_up_t.dim() == 2 and gate_up_t.is_contiguous() and gate_up_t.dtype == torch.bfloat16
          and gate_up_t.shape[0] % 16 == 0 and gate_up_t.shape[1] % 8 == 0,
          "gate_up_t must be contiguous bfloat16 [2I, T] with I and T multiples of 8")
    I, T = gate_up_t.shape[0] // 2, gate_up_t.shape[1]
    if out is None:
        out = torch.empty((T, I), dtype=torch.bfloat16, device=gate_up_t.device)
    _need(out.dtype == torch.bfloat16 and out.shape == (T, I) and out.is_contiguous(), "out must be contiguous bfloat16 [T, I]")
    lib = build.load("activation")
    _check(lib.ga_silu_mul_transposed(_ptr(out), _ptr(gate_up_t), _i(T), _i(I), _stream()), "silu_mul_transposed")
    return out


def rope_kv_write(qkv, positions, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads,
                  head_dim, write_kv=True):
    """Rotates q and k inside qkv [T, (nh + 2 nkv) hd] in place and writes k, v to the paged cache
    (k [pages, nkv, page_size, hd], v [pages, nkv, hd, page_size]) at slot_mapping [T] int64 (-1: skip).  cos, sin: float32
    [positions, rotary_dim / 2]."""
    _dev(qkv, positions, cos, sin, slot_mapping, k_pages, v_pages)
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(qkv.dim() == 2 and qkv.shape[1] == width and qkv.is_contiguous(),
          "qkv must be contiguous [T, %d]",
          width)
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(),
          "positions must be contiguous int32 [T]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape and cos.dim() == 2
          and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, rotary_dim/2]")
    rotary_dim = 2 * cos.shape[1]
    _need(0 < rotary_dim <= head_dim,
          "rotary_dim %d must lie in (0, head_dim %d]",
          rotary_dim, head_dim)
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [T]")
        page_size = _check_pages(k_pages, v_pages, qkv.dtype, num_kv_heads, head_dim)
    lib = build.load("rope_kv")
    _check(lib.ga_rope_kv_write(_ptr(qkv), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
                                _ptr(k_pages), _ptr(v_pages), _i(T), _i(num_heads), _i(num_kv_heads),
                                _i(head_dim), _i(rotary_dim), _i(page_size), _i(1 if write_kv else 0),
                                _i(_is_bf16(qkv.dtype)), _stream()), "rope_kv_write")


def rope_kv_from_parts(parts, bias, positions, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads, head_dim,
                       write_kv=True):
    """The epilogue of a q|k|v projection that arrives as float32 partial sums [parts, T, (nh + 2 nkv) hd] of a product
    whose K was split over workgroups: the parts added in order, the bias (bfloat16 [width] or None), q and k rotated on
    the 32-bit sums; returns q [T, nh*hd] in bfloat16 and writes k and v into the paged cache at slot_mapping."""
    _dev(parts, bias, positions, cos, sin, slot_mapping, k_pages, v_pages)
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[2] == width and parts.is_contiguous(),
          "parts must be contiguous float32 [parts, T, %d]",
          width)
    T = parts.shape[1]
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(),
          "positions must be contiguous int32 [T]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape and cos.dim() == 2
          and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, rotary_dim/2]")
    rotary_dim = 2 * cos.shape[1]
    _need(0 < rotary_dim <= head_dim and (rotary_dim // 2) % 4 == 0 and (head_dim - rotary_dim) % 4 == 0 and head_dim % 4 == 0,
          "this kernel takes rotary_dim / 2, head_dim - rotary_dim and head_dim in multiples of 4; got %d of %d",
          rotary_dim, head_dim)
    _need(1 <= parts.shape[0] <= 8, "this kernel adds up to 8 parts, got %d", parts.shape[0])
    if bias is not None:
        _need(bias.dtype == torch.bfloat16 and bias.shape == (width,) and bias.is_contiguous(),
              "qkv bias must be bfloat16 [%d]",
              width)
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [T]")
        page_size = _check_pages(k_pages, v_pages, torch.bfloat16, num_kv_heads, head_dim)
    q = torch.empty((T, num_heads * head_dim), dtype=torch.bfloat16, device=parts.device)
    lib = build.load("rope_kv")
    _check(lib.ga_rope_kv_from_parts(_ptr(q), _ptr(parts), _i(parts.shape[0]), _ptr(bias), _ptr(positions), _ptr(cos),
                                     _ptr(sin), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), _i(T), _i(num_heads),
                                     _i(num_kv_heads), _i(head_dim), _i(rotary_dim), _i(page_size),
                                     _i(1 if write_kv else 0), _stream()), "rope_kv_from_parts")
    return q


def _check_pages(k_pages, v_pages, dtype, nkv, hd):
    """k_pages [pages, nkv, page_size, hd], v_pages [pages, nkv, hd, page_size] (values transposed)."""
    _need(k_pages is not None and v_pages is not None, "cache pages are missing")
    for p in (k_pages, v_pages):
        _need(p.dtype == dtype and p.dim() == 4 and p.is_contiguous() and p.shape[1] == nkv,
              "cache pages must be contiguous %s with %d kv heads",
              dtype, nkv)
    ps = k_pages.shape[2]
    _need(k_pages.shape[3] == hd and tuple(v_pages.shape) == (k_pages.shape[0], nkv, hd, ps),
          "cache pages must be k [pages, %d, page_size, %d] and v [pages, %d, %d, page_size], got %s and %s",
          nkv, hd, nkv, hd, tuple(k_pages.shape), tuple(v_pages.shape))
    return ps


def _check_attention_operands(q, k_pages, v_pages, block_table, token_entry, positions, nh, nkv, hd):
    _dev(q, k_pages, v_pages, block_table, token_entry, positions)
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd, "q must be [T, >= nh*hd] with unit inner stride")
    _need(nkv > 0 and nh % nkv == 0,
          "num_heads %d is not a multiple of num_kv_heads %d",
          nh, nkv)
    _check_pages(k_pages, v_pages, q.dtype, nkv, hd)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [entries, width]")
    for name, x in (("token_entry", token_entry), ("positions", positions)):
        _need(x.dtype == torch.int32 and x.shape == (T,) and x.is_contiguous(),
              "%s must be contiguous int32 [T]",
              name)
    return T


def paged_attention_generic(q, k_pages, v_pages, block_table, token_entry, positions, num_heads, num_kv_heads,
                            head_dim, scale, window=None, out=None, tokens_per_workgroup=0):
    """q: rows of the fused projection ([T, >= nh*hd]; the first nh*hd columns are the queries).
    Token t attends to the keys of request token_entry[t] at positions
    [max(0, p - window + 1), p], p = positions[t].  Returns [T, nh*hd].  tokens_per_workgroup: how many neighbouring
    tokens share a workgroup and (where they are of one request) its tiles of keys and values; 1 suits steps of
    single tokens, 0 leaves it to the library (from 32 tokens on: the matrix cores for a request's 8 tokens and more,
    a second kernel for the requests with fewer), -1 says besides that every request has at least 8 tokens in the
    step; no token's result depends on it."""
    T = _check_attention_operands(q, k_pages, v_pages, block_table, token_entry, positions, num_heads,
                                  num_kv_heads, head_dim)
    _need(0 < head_dim <= 256,
          "head_dim %d is not supported by the general attention kernel (up to 256)",
          head_dim)
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    _need(out.dtype == q.dtype and out.shape == (T, num_heads * head_dim) and out.stride(1) == 1, "out must be [T, nh*hd]")
    lib = build.load("attention_generic")
    _check(lib.ga_paged_attention_generic(
        _ptr(out), _i64(out.stride(0)), _ptr(q), _i64(q.stride(0)), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        _i(block_table.shape[1]), _ptr(token_entry), _ptr(positions), _i(T), _i(num_heads), _i(num_kv_heads),
        _i(head_dim), _i(k_pages.shape[2]), _i(int(window) if window else 0), _f(scale), _i(_is_bf16(q.dtype)),
        _i(int(tokens_per_workgroup)), _i(TUNING.generic_few_tokens_workgroups), _i(TUNING.generic_fill_workgroups),
        _stream()), "paged_attention_generic")
    return out


def gemm_nt(a, w, bias=None, out=None, out_dtype=None):
    """a [M, K] . w [N, K]^T (+ bias [N]) -> [M, N]; 32-bit accumulation, plain FMA.  a and w share a
    dtype (float32 or bfloat16); out is that dtype or float32."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          "gemm_nt: a [M, K] and w [N, K] do not agree: %s, %s",
          tuple(a.shape), tuple(w.shape))
    _need(a.dtype == w.dtype and a.stride(1) == 1 and w.is_contiguous(), "gemm_nt: a and w must share a dtype; w contiguous")
    M, K = a.shape
    N = w.shape[0]
    if bias is not None:
        _need(bias.dtype == w.dtype and bias.shape == (N,) and bias.is_contiguous(), "gemm_nt: bias must be [N] in w's dtype")
    out_dtype = out_dtype or (out.dtype if out is not None else a.dtype)
    _need(out_dtype in (a.dtype, torch.float32), "gemm_nt: out dtype must be the operands' or float32")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    _need(out.shape == (M, N) and out.dtype == out_dtype and out.stride(1) == 1, "gemm_nt: out must be [M, N]")
    lib = build.load("gemm")
    _check(lib.ga_gemm_nt(_ptr(out), _i64(out.stride(0)), _ptr(a), _i64(a.stride(0)), _ptr(w), _ptr(bias), _i(M), _i(N),
                          _i(K), _i(_is_bf16(a.dtype)), _i(1 if out_dtype == torch.bfloat16 else 0), _stream()),
           "gemm_nt")
    return out


def sample_rows(logits, temperature=None, uniform=None, out=None):
    """logits float32 [R, V] -> int32 [R].  Rows with temperature 0 (or all rows, without
    temperature) take the argmax with the lowest index among equals; others draw by inverse CDF from
    softmax(logits / temperature) with the given uniform numbers in [0, 1)."""
    _dev(logits, temperature, uniform, out)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1, "logits must be float32 [R, V]")
    R, V = logits.shape
    if temperature is not None:
        _need(uniform is not None, "temperature sampling needs uniform numbers")
        for name, x in (("temperature", temperature), ("uniform", uniform)):
            _need(x.dtype == torch.float32 and x.shape == (R,) and x.is_contiguous(),
                  "%s must be contiguous float32 [R]",
                  name)
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out.dtype == torch.int32 and out.shape == (R,) and out.is_contiguous(), "out must be contiguous int32 [R]")
    _need(R <= 65535, "at most 65535 rows a call")
    lib = build.load("sampling")
    lib.ga_sample_scratch_floats.restype = ctypes.c_int64
    scratch = torch.empty((max(1, lib.ga_sample_scratch_floats(_i(R), _i(V))),), dtype=torch.float32, device=logits.device)
    _check(lib.ga_sample_rows(_ptr(out), _ptr(logits), _i64(logits.stride(0)), _i(R), _i(V), _ptr(temperature),
                              _ptr(uniform), _ptr(scratch), _stream()), "sample_rows")
    return out


def random_normal_fill(out, key, mean, std):
    """out[i] = mean + std * normal(key, i) over out's elements in memory order (float32 or bfloat16, contiguous): the
    counter-based generator that the host shares, so the same key gives the same bits there."""
    _dev(out)
    _need(out.is_contiguous() and out.dtype in (torch.float32, torch.bfloat16), "random fill takes a contiguous float32 or "
          "bfloat16 tensor")
    lib = build.load("random_fill")
    _check(lib.ga_random_normal_fill(_ptr(out), _i64(out.numel()), ctypes.c_uint64(int(key)), _f(mean), _f(std),
                                     _i(_is_bf16(out.dtype)), _stream()), "random_normal_fill")
    return out


SKINNY_MAX_ROWS = 64
FOLDED_NORM_MAX_ROWS = 16


class ScaledRows:
    """The rows of a root-mean-square norm in two factors, as the products around a folded norm hand them on:
    `scaled` = h * g (bfloat16 [M, H]) and `sumsq` (float32 [M, parts]), partial sums of h^2 over the columns;
    the normalised row is scaled / sqrt(sum(sumsq) / H + eps).  A product that takes them multiplies its
    32-bit sums by the rows' factors, which gives what the normalised rows would."""

    __slots__ = ("scaled", "sumsq", "eps")

    def __init__(self, scaled, sumsq, eps):
        self.scaled, self.sumsq, self.eps = scaled, sumsq, float(eps)

    @property
    def shape(self):
        return self.scaled.shape

    @property
    def dtype(self):
        return self.scaled.dtype

    def rows(self):
        """The normalised rows themselves (for checks; the kernels never build them)."""
        rstd = torch.rsqrt(self.sumsq.double().sum(dim=1, keepdim=True) / self.scaled.shape[1] + self.eps)
        return (self.scaled.double() * rstd).float()


class _SkinnyNorm(ctypes.Structure):
    _fields_ = [("in_sumsq", _vp), ("in_parts", _i), ("inv_width", _f), ("eps", _f), ("residual", _vp), ("ldr", _i64),
                ("gain", _vp), ("gain_f32", _i), ("scaled", _vp), ("lds", _i64), ("out_sumsq", _vp)]


def _norm_in(norm, a):
    """Fills the in_ fields from ScaledRows; returns the rows the product runs on."""
    _need(a.scaled.dtype == torch.bfloat16 and a.scaled.dim() == 2 and a.scaled.shape[0] <= FOLDED_NORM_MAX_ROWS,
          "rows of a folded norm are bfloat16 [M <= %d, H]",
          FOLDED_NORM_MAX_ROWS)
    M, H = a.scaled.shape
    _need(a.sumsq.dtype == torch.float32 and a.sumsq.dim() == 2 and a.sumsq.shape[0] == M and a.sumsq.is_contiguous()
          and 1 <= a.sumsq.shape[1] <= 512, "partial sums of a folded norm are contiguous float32 [M, parts <= 512]")
    norm.in_sumsq, norm.in_parts = a.sumsq.data_ptr(), a.sumsq.shape[1]
    norm.inv_width, norm.eps = 1.0 / H, a.eps
    return a.scaled


def folded_norm_supported(a, w, residual, gain):
    """Whether a [M, K] . w [N, K]^T can add itself to `residual` and hand on the rows of the norm with `gain`
    in two factors (ScaledRows)."""
    x = a.scaled if isinstance(a, ScaledRows) else a
    N = w.shape[0]
    return (gemm_skinny_supported(x, w) and x.shape[0] <= FOLDED_NORM_MAX_ROWS and N % 8 == 0
            and build.load("gemm_skinny").ga_skinny_norm_parts(_i(x.shape[0]), _i(N)) <= 512
            and residual.dtype == torch.float32 and residual.shape == (x.shape[0], N) and residual.stride(1) == 1
            and gain.dtype in (torch.bfloat16, torch.float32) and gain.shape == (N,) and gain.is_contiguous())


def gemm_skinny_supported(a, w):
    """Whether the matrix-core kernel for few rows takes these operands."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and 0 < a.shape[0] <= SKINNY_MAX_ROWS
            and a.shape[1] % 8 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0)


def gemm_skinny(a, w, bias=None, out=None, out_dtype=None, nt=0, ks=0, grid_splits=1, gated=False, into_norm=None,
                pack=0):
    """a [M <= 64, K] . w [N, K]^T (+ bias) -> [M, N] in bfloat16 (or float32): the decode step's products,
    weights streamed once through the matrix cores.  grid_splits > 1: K is split over workgroups too and
    the result is float32 [grid_splits, M, N], parts for the consumer to add.  gated: w is [2N, K] (gate
    over up) and the result is silu(a.gate^T) * (a.up^T).
    pack = 2 (at most 8 rows): a tile of the matrix cores holds 8 rows of w twice, for the two halves of K,
    so that twice the workgroups stream the weights.
    a may be ScaledRows (at most 16 rows): the rows of a norm in two factors.  into_norm = (residual, gain, eps):
    the product is added to the float32 residual [M, N] in place and the rows of the norm that follows come
    back as ScaledRows instead of the product."""
    norm = None
    if isinstance(a, ScaledRows):
        norm = _SkinnyNorm()
        a = _norm_in(norm, a)
    if into_norm is not None:
        residual, gain, eps = into_norm
        _need(folded_norm_supported(a, w, residual, gain) and not gated and grid_splits == 1 and out is None,
              "a product folds the norm after it for at most %d bfloat16 rows, a float32 residual [M, N] and a "
              "gain [N], N a multiple of 8 with at most 512 partial sums a row",
              FOLDED_NORM_MAX_ROWS)
        _dev(residual, gain)
        norm = norm or _SkinnyNorm()
        M, N = residual.shape
        lib = build.load("gemm_skinny")
        scaled = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
        sumsq = torch.empty((M, lib.ga_skinny_norm_parts(_i(M), _i(N))), dtype=torch.float32, device=a.device)
        norm.residual, norm.ldr = residual.data_ptr(), residual.stride(0)
        norm.gain, norm.gain_f32 = gain.data_ptr(), 1 if gain.dtype == torch.float32 else 0
        norm.scaled, norm.lds, norm.out_sumsq = scaled.data_ptr(), scaled.stride(0), sumsq.data_ptr()
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          "gemm_skinny: a [M, K] and w [N, K] do not agree: %s, %s",
          tuple(a.shape), tuple(w.shape))
    _need(gemm_skinny_supported(a, w),
          "gemm_skinny takes bfloat16, at most %d rows, K a multiple of 8 and 16-byte "
          "aligned rows; got a %s %s, w %s %s",
          SKINNY_MAX_ROWS, a.dtype, tuple(a.shape), w.dtype, tuple(w.shape))
    M, K = a.shape
    N = w.shape[0]
    if gated:       # w stacks gate over up: the result has half as many columns
        _need(N % 2 == 0 and bias is None and grid_splits == 1, "gated product: w must be [2N, K], without bias or split")
        N //= 2
    if bias is not None:
        _need(bias.dtype == torch.bfloat16 and bias.shape == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be bfloat16 [N]")
    if into_norm is not None:
        _check(lib.ga_gemm_skinny(_vp(0), _i64(0), _ptr(a), _i64(a.stride(0)), _ptr(w), _ptr(bias), _i(M), _i(N), _i(K),
                                  _i(0), _i(1), _i(8), _i(1), _i(0), _i(0), ctypes.byref(norm), _stream()), "gemm_skinny")
        return ScaledRows(scaled, sumsq, eps)
    out_dtype = out_dtype or (out.dtype if out is not None else torch.bfloat16)
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_skinny: out dtype must be bfloat16 or float32")
    if grid_splits > 1:
        _need(out_dtype == torch.float32, "gemm_skinny: parts of a split product are float32")
        if out is None:
            out = torch.empty((grid_splits, M, N), dtype=torch.float32, device=a.device)
        _need(out.shape == (grid_splits, M, N) and out.dtype == torch.float32 and out.is_contiguous(),
              "gemm_skinny: parts must be contiguous float32 [splits, M, N]")
        ldc = N
    else:
        if out is None:
            out = torch.empty((M, N), dtype=out_dtype, device=a.device)
        _need(out.shape == (M, N) and out.dtype == out_dtype and out.stride(1) == 1, "gemm_skinny: out must be [M, N]")
        ldc = out.stride(0)
    lib = build.load("gemm_skinny")
    _check(lib.ga_gemm_skinny(_ptr(out), _i64(ldc), _ptr(a), _i64(a.stride(0)), _ptr(w), _ptr(bias), _i(M), _i(N),
                              _i(K), _i(1 if out_dtype == torch.float32 else 0), _i(nt), _i(ks), _i(grid_splits),
                              _i(1 if gated else 0), _i(pack), ctypes.byref(norm) if norm is not None else _vp(0),
                              _stream()), "gemm_skinny")
    return out


def qkv_rope_skinny_supported(x, w, head_dim, rotary_dim):
    """Whether the fused projection + rotation + cache-write kernel takes these operands."""
    if isinstance(x, ScaledRows):
        x = x.scaled
    return gemm_skinny_supported(x, w) and head_dim % 32 == 0 and rotary_dim == head_dim


def qkv_rope_skinny(x, w, bias, positions, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads, head_dim,
                    write_kv=True, pack=0):
    """The decode step's q|k|v projection with its epilogue in one kernel: x [M <= 64, K] . w^T + bias, NeoX
    rotation of q and k, q returned as [M, nh*hd], k and v written into the paged cache at slot_mapping.
    x may be ScaledRows."""
    norm = None
    if isinstance(x, ScaledRows):
        norm = _SkinnyNorm()
        x = _norm_in(norm, x)
    _dev(x, w, bias, positions, cos, sin, slot_mapping, k_pages, v_pages)
    M, K = x.shape
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(w.shape == (width, K),
          "qkv weight must be [%d, %d], got %s",
          width, K, tuple(w.shape))
    _need(qkv_rope_skinny_supported(x, w, head_dim, 2 * cos.shape[1]),
          "the fused q|k|v kernel takes bfloat16, at most %d "
          "rows, head sizes that are multiples of 32 and a rotation of the whole head",
          SKINNY_MAX_ROWS)
    if bias is not None:
        _need(bias.dtype == torch.bfloat16 and bias.shape == (width,) and bias.is_contiguous(),
              "qkv bias must be bfloat16 [%d]",
              width)
    _need(positions.dtype == torch.int32 and positions.shape == (M,) and positions.is_contiguous(), "positions must be int32 [M]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape and cos.is_contiguous()
          and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, head_dim/2]")
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (M,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [M]")
        page_size = _check_pages(k_pages, v_pages, torch.bfloat16, num_kv_heads, head_dim)
    q = torch.empty((M, num_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    lib = build.load("gemm_skinny")
    _check(lib.ga_qkv_rope_skinny(_ptr(q), _ptr(x), _i64(x.stride(0)), _ptr(w), _ptr(bias), _ptr(positions), _ptr(cos),
                                  _ptr(sin), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), _i(M), _i(K), _i(num_heads),
                                  _i(num_kv_heads), _i(head_dim), _i(page_size), _i(1 if write_kv else 0), _i(pack),
                                  ctypes.byref(norm) if norm is not None else _vp(0), _stream()), "qkv_rope_skinny")
    return q


# ----------------------------------------------------------------------------- attention on the matrix cores

MFMA_HEAD_DIMS = tuple(range(16, 257, 16))


def attention_mfma_supported(dtype, head_dim, page_size):
    return (dtype == torch.bfloat16 and head_dim in MFMA_HEAD_DIMS and page_size >= 8
            and page_size & (page_size - 1) == 0)


def plan_rows(q_len, q_start, tile_rows):
    """How a step's rows go to the attention kernels: (rows, positions, entries of the single new tokens,
    tiles of the prompt portions as (entry, first row of the step, rows, first position), heaviest first)."""
    decode_rows, decode_pos, decode_entries, tiles = [], [], [], []
    o = 0
    for e, (n, start) in enumerate(zip(q_len, q_start)):
        if n == 1:
            decode_rows.append(o)
            decode_pos.append(start)
            decode_entries.append(e)
        else:
            for r in range(0, n, tile_rows):
                tiles.append((e, o + r, min(tile_rows, n - r), start + r))
        o += n
    tiles.sort(key=lambda t: -(t[3] + t[2]))      # the tiles with the most keys first
    return decode_rows, decode_pos, decode_entries, tiles


PLAN_TILE_ROWS = 16       # rows of a prompt portion per wavefront in steps of fewer than TUNING.prefill_wide_tiles_from tokens


def _attention_plan(step, tile_rows, device, split_for=None):
    """Which rows of the step are single new tokens and how the rows of prompt portions fall into tiles;
    made once per step and shared by all layers.  A recorded step brings its plan along (`static_plan` in the
    step's extra: device arrays of fixed size that the runner refills, counts that include padding).  split_for:
    (window, workgroups per tile, streams of a workgroup) where the kernel takes tiles whose keys are in parts."""
    key = ("attention_plan", tile_rows, split_for)
    plan = step.extra.get(key)
    if plan is not None:
        return plan
    static = step.extra.get("static_plan")
    if static is not None:
        _need(tile_rows == static["tile_rows"], "a recorded step was planned for tiles of %d rows, not %d",
              static["tile_rows"], tile_rows)
        plan = dict(n_decode=static["n_decode"], decode_pos=None, n_tiles=static["n_tiles"],
                    decode_span=step.extra.get("decode_span"), decode_info=step.extra.get("decode_info"),
                    tiles=static["tiles"], parts=None, part_rows=None, n_part_rows=0, num_parts=1)
        step.extra[key] = plan
        return plan
    import numpy as np
    decode_rows, decode_pos, entries, tiles = plan_rows(step.host_q_len, step.host_q_start, tile_rows)
    # (row, position, entry, -) of every single new token; the runner uploads it with the step's other inputs
    decode_info = step.extra.get("decode_info")
    if decode_info is None and decode_rows:
        decode_info = torch.tensor([[r, p, e, 0] for r, p, e in zip(decode_rows, decode_pos, entries)], dtype=torch.int32,
                                   device=device)
    plan = dict(n_decode=len(decode_rows), decode_pos=decode_pos, n_tiles=len(tiles), decode_span=step.extra.get("decode_span"),
                decode_info=decode_info, tiles=None, parts=None, part_rows=None, n_part_rows=0, num_parts=1)
    if tiles:
        split = key_parts(tiles, tile_rows, *split_for) if split_for is not None else None
        if split is None:
            plan["tiles"] = torch.tensor(np.asarray(tiles, dtype=np.int32).reshape(-1, 4), device=device)
        else:
            # the tiles, their parts and the rows that come in parts, in one transfer
            pieces, parts, rows, num_parts = split
            both = np.concatenate([np.asarray(pieces, dtype=np.int32).reshape(-1), np.asarray(parts, dtype=np.int32).reshape(-1),
                                   np.asarray(rows, dtype=np.int32).reshape(-1)])
            dev_all = torch.tensor(both, device=device)
            n, r = len(pieces), len(rows)
            plan.update(n_tiles=n, tiles=dev_all[:4 * n].view(n, 4), parts=dev_all[4 * n:8 * n].view(n, 4),
                        part_rows=dev_all[8 * n:].view(r, 4), n_part_rows=r, num_parts=num_parts)
    step.extra[key] = plan
    return plan


def key_parts(tiles, tile_rows, window, workgroups_per_tile, streams, compute_units=256):
    """Whether the keys of a step's heaviest tiles should be dealt to several workgroups, and how.  A short prompt alone
    in a step makes about as many workgroups as there are compute units, one round, so the kernel lasts as long as its
    heaviest tile's walk over the keys, twice the mean of a causal prompt's tiles.  tiles: (entry, first row, rows, first
    position), heaviest first.  None: leave the tiles whole.  Else (tiles with one entry per part, parts as the kernel takes
    them, the rows that come in parts as int32 x 4, number of parts): the tiles with more than the mean share of keys per
    compute unit fall into equal parts of at most that share.  Switched off in the table of thresholds
    (`prefill_split_imbalance` 0): measured on MI355X it does not pay (a 2,048-token prompt of 12 heads in 2 groups, head
    size 128: 40.8 us whole, 45.6 in parts: the workgroups beyond one round of the chip pay a workgroup's fixed part, some
    8 us, a second time, and the merge and 10 MB of partial results cost what the shorter walks save)."""
    def key_tiles(t):
        lo = max(0, t[3] - window + 1) if window else 0
        return (t[3] + t[2] - 1) // 32 + 1 - lo // 32, (lo // 32) * 32
    counts = [key_tiles(t)[0] for t in tiles]
    heaviest = max(counts)
    share = sum(counts) * workgroups_per_tile / float(compute_units)          # tiles of 32 keys per compute unit, on average
    if (TUNING.prefill_split_imbalance <= 0 or len(tiles) * workgroups_per_tile > TUNING.prefill_split_max_workgroups
            or heaviest < TUNING.prefill_split_min_key_tiles * streams or heaviest <= TUNING.prefill_split_imbalance * share):
        return None
    share = max(share, 1.0)
    num_parts = min(8, -(-heaviest // int(share)))
    if num_parts < 2:
        return None
    out, rows_in_parts = [], []
    for t, k in zip(tiles, counts):
        first = key_tiles(t)[1]
        if k <= 1.15 * share:
            out.append((k, t, (first, first + 32 * k, -1, 1 << 16)))
            continue
        at = len(rows_in_parts)
        rows_in_parts += [(t[1] + j, 0, 0, 0) for j in range(t[2])]
        per = -(-k // num_parts)
        per = -(-per // streams) * streams                    # whole rounds of the workgroup's streams
        for part in range(num_parts):
            b, e = min(part * per, k), min((part + 1) * per, k)
            # a part without keys still writes its rows' (empty) results, which the merge expects
            out.append((e - b, t, (first + 32 * b, first + 32 * e, at, part | (num_parts << 16))))
    out.sort(key=lambda x: -x[0])                             # the longest walks first
    return [x[1] for x in out], [x[2] for x in out], rows_in_parts, num_parts


def _decode_splits(plan, window, nkv, head_blocks):
    span = 0
    if plan.get("decode_span"):             # a recorded step: the split must fit every context of its bucket
        span = plan["decode_span"] if not window else min(plan["decode_span"], (window + 62) // 32 * 32)
    else:
        for pos in plan["decode_pos"]:
            lo = max(0, pos - window + 1) if window else 0
            span = max(span, pos + 1 - (lo // 32) * 32)
    per_split = plan["n_decode"] * nkv * head_blocks
    splits = max(1, min(TUNING.decode_target_workgroups // max(per_split, 1), -(-span // TUNING.decode_min_split_keys),
                        TUNING.decode_max_splits))
    split_keys = -(-(-(-span // splits)) // 32) * 32
    return split_keys, -(-span // split_keys)


def paged_attention_mfma(q, k_pages, v_pages, block_table, step, num_heads, num_kv_heads, head_dim, scale,
                         window=None, out=None):
    """bfloat16 attention of every token of the step on the matrix cores: single new tokens through the
    split-key kernel, rows of prompt portions through the tiled kernel."""
    T = _check_attention_operands(q, k_pages, v_pages, block_table, step.token_entry, step.positions, num_heads,
                                  num_kv_heads, head_dim)
    page_size = k_pages.shape[2]
    _need(attention_mfma_supported(q.dtype, head_dim, page_size),
          "the matrix-core attention kernels take bfloat16, head sizes in steps of 16 up to 256 and page sizes that "
          "are powers of two from 8; got %s, head %d, page %d",
          q.dtype, head_dim, page_size)
    _need(q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0, "q rows must be 16-byte aligned")
    _need(k_pages.shape[0] * num_kv_heads * max(page_size, head_dim) < 2 ** 31,
          "the matrix-core attention kernels count the rows of a layer's cache in 32 bits: %d pages x %d kv heads x "
          "%d is too many",
          k_pages.shape[0], num_kv_heads, max(page_size, head_dim))
    lib = build.load("attention_mfma", {"HEAD_DIM": head_dim})
    _need(lib.ga_attn_head_dim() == head_dim, "attention library was built for another head size")
    # rows of a prompt portion per wavefront: 32 where the kernel has it and the step is long, else 16
    wide = T >= TUNING.prefill_wide_tiles_from
    tile_rows = lib.ga_attn_prefill_max_tile_rows() if wide else 16
    plan = _attention_plan(step, tile_rows, q.device,
                           split_for=_prefill_workgroups(step, tile_rows, num_heads // num_kv_heads, num_kv_heads, head_dim,
                                                         int(window) if window else 0))
    _need(sum(step.host_q_len) == T, "the step's entries do not add up to its tokens")
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    _need(out.dtype == q.dtype and out.shape == (T, num_heads * head_dim) and out.is_contiguous(), "out must be [T, nh*hd]")
    w = int(window) if window else 0
    if plan["n_decode"]:
        group = num_heads // num_kv_heads
        split_keys, num_splits = _decode_splits(plan, w, num_kv_heads, -(-group // 16))
        n = plan["n_decode"] * num_heads * num_splits
        ws_o = torch.empty((n * head_dim,), dtype=torch.float32, device=q.device)
        ws_ml = torch.empty((n * 2,), dtype=torch.float32, device=q.device)
        _check(lib.ga_attn_decode(
            _ptr(out), _i64(out.stride(0)), _ptr(q), _i64(q.stride(0)), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            _i(block_table.shape[1]), _ptr(plan["decode_info"]), _i(plan["n_decode"]), _i(num_heads), _i(num_kv_heads), _i(page_size), _i(w), _f(scale), _i(split_keys),
            _i(num_splits), _ptr(ws_o), _ptr(ws_ml), _stream()), "attn_decode")
    if plan["n_tiles"]:
        part_o = part_ml = None
        if plan["n_part_rows"]:
            n = plan["n_part_rows"] * num_heads * plan["num_parts"]
            part_o = torch.empty((n * head_dim,), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((n * 2,), dtype=torch.float32, device=q.device)
        _check(lib.ga_attn_prefill(
            _ptr(out), _i64(out.stride(0)), _ptr(q), _i64(q.stride(0)), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            _i(block_table.shape[1]), _ptr(plan["tiles"]), _i(plan["n_tiles"]), _i(tile_rows), _i(num_heads), _i(num_kv_heads),
            _i(page_size), _i(w), _f(scale), _i(TUNING.prefill_fill_workgroups), _i(TUNING.prefill_prefer_workgroups),
            _ptr(plan["parts"]), _ptr(plan["part_rows"]),
            _i(plan["n_part_rows"]), _i(plan["num_parts"]), _ptr(part_o), _ptr(part_ml), _stream()), "attn_prefill")
    return out


def _prefill_workgroups(step, tile_rows, group, nkv, head_dim, window):
    """(window, workgroups per tile, streams of tiles in a workgroup) as the prefill launcher will choose them for this
    step, or None where the step brings its plan along (a recorded step) or has no prompt portion: what `key_parts`
    needs to know.  Follows ga_attn_prefill's choice of heads per workgroup (csrc/attention_mfma.hip)."""
    if "static_plan" in (step.extra or {}):
        return None
    n_tiles = sum(-(-n // tile_rows) for n in step.host_q_len if n > 1)
    if n_tiles == 0:
        return None
    fill, waves = TUNING.prefill_fill_workgroups, 8
    if head_dim in (64, 128, 256):
        heads = 1
        for d in range(waves - 1, 1, -1):
            if group % d == 0 and n_tiles * nkv * (group // d) >= fill:
                heads = d
                if n_tiles * nkv * (group // d) >= TUNING.prefill_prefer_workgroups:
                    break
        if heads >= 2:
            return window, nkv * (group // heads), max(1, waves // (heads + 1))
    hpw = 1
    for d in range(2, waves + 1):
        if group % d == 0 and n_tiles * nkv * (group // d) >= fill:
            hpw = d
    splits = waves // hpw
    if hpw > 1 and splits > 4:
        splits = 4
    return window, nkv * (group // hpw), splits


def paged_attention(q, k_pages, v_pages, block_table, step, num_heads, num_kv_heads, head_dim, scale, window=None):
    """Attention of every token of the step over its request's pages.  Chooses the kernel: the general
    one in 32-bit (fixed order of every sum: bit-identical however the work is cut); in bfloat16 the
    matrix-core kernels where they take the shape."""
    if attention_mfma_supported(q.dtype, head_dim, k_pages.shape[2]):
        return paged_attention_mfma(q, k_pages, v_pages, block_table, step, num_heads, num_kv_heads, head_dim, scale,
                                    window)
    if step.max_q_len == 1:
        grouping = 1
    elif "static_plan" not in (step.extra or {}) and min(step.host_q_len) >= 8:
        grouping = -1          # the step's own sizes are known here (a recorded step of padded sizes serves many)
    else:
        grouping = 0
    return paged_attention_generic(q, k_pages, v_pages, block_table, step.token_entry, step.positions, num_heads,
                                   num_kv_heads, head_dim, scale, window, tokens_per_workgroup=grouping)
