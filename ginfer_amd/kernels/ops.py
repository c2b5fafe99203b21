"""Python faces of the HIP kernels.

Every function checks on the host what its kernel and launch grid assume (devices, dtypes,
contiguity, matching sizes) and raises a clear error instead of launching with operands that do not
fit; a kernel never sees a shape it was not written for.  Tensors are torch tensors on the GPU;
kernels run on torch's current stream.
"""
import ctypes

import torch

from . import build

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_f = ctypes.c_float


class KernelError(RuntimeError):
    pass


def _ptr(t):
    return _vp(t.data_ptr()) if t is not None else _vp(0)


def _stream():
    return _vp(torch.cuda.current_stream().cuda_stream)


def _check(rc, name):
    if rc != 0:
        raise KernelError("kernel %s failed to launch (code %d)" % (name, rc))


def _need(cond, msg):
    if not cond:
        raise KernelError(msg)


def _dev(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        _need(t.is_cuda, "kernel operands must live on the GPU (got a %s tensor)" % t.device)
        dev = dev or t.device
        _need(t.device == dev, "kernel operands lie on different devices")


def _is_bf16(dtype):
    _need(dtype in (torch.float32, torch.bfloat16), "compute dtype must be float32 or bfloat16, got %s" % dtype)
    return 1 if dtype == torch.bfloat16 else 0


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
    `dtype` or None; gain [H] in `dtype` (or float32); rows int32 [R] or None -> normed [R or T, H]."""
    _dev(residual, delta, gain, rows, out)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    T, H = residual.shape
    if delta is not None:
        _need(delta.dtype == dtype and delta.shape == (T, H) and delta.is_contiguous(),
              "delta must be contiguous %s [%d, %d], got %s %s" % (dtype, T, H, delta.dtype, tuple(delta.shape)))
    _need(gain.shape == (H,) and gain.is_contiguous() and gain.dtype in (dtype, torch.float32),
          "gain must be contiguous [%d] in %s or float32" % (H, dtype))
    R = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be contiguous int32 [R]")
        R = rows.shape[0]
    if out is None:
        out = torch.empty((R, H), dtype=dtype, device=residual.device)
    _need(out.dtype == dtype and out.shape == (R, H) and out.is_contiguous(), "out must be contiguous [R, H]")
    lib = build.load("norm")
    _check(lib.ga_add_rmsnorm(_ptr(out), _ptr(residual), _ptr(delta), _ptr(gain), _ptr(rows), _i(R), _i(H),
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


def rope_kv_write(qkv, positions, cos, sin, slot_mapping, k_pages, v_pages, num_heads, num_kv_heads,
                  head_dim, write_kv=True):
    """Rotates q and k inside qkv [T, (nh + 2 nkv) hd] in place and writes k, v to the paged cache
    [pages, nkv, page_size, hd] at slot_mapping [T] int64 (-1: skip).  cos, sin: float32
    [positions, rotary_dim / 2]."""
    _dev(qkv, positions, cos, sin, slot_mapping, k_pages, v_pages)
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(qkv.dim() == 2 and qkv.shape[1] == width and qkv.is_contiguous(), "qkv must be contiguous [T, %d]" % width)
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(),
          "positions must be contiguous int32 [T]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape and cos.dim() == 2
          and cos.is_contiguous() and sin.is_contiguous(), "cos and sin must be contiguous float32 [P, rotary_dim/2]")
    rotary_dim = 2 * cos.shape[1]
    _need(0 < rotary_dim <= head_dim, "rotary_dim %d must lie in (0, head_dim %d]" % (rotary_dim, head_dim))
    page_size = 1
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.shape == (T,)
              and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int64 [T]")
        for p in (k_pages, v_pages):
            _need(p is not None and p.dtype == qkv.dtype and p.dim() == 4 and p.is_contiguous()
                  and p.shape[1] == num_kv_heads and p.shape[3] == head_dim,
                  "cache pages must be contiguous %s [pages, %d, page_size, %d]" % (qkv.dtype, num_kv_heads, head_dim))
        _need(k_pages.shape == v_pages.shape, "k and v pages differ in shape")
        page_size = k_pages.shape[2]
    lib = build.load("rope_kv")
    _check(lib.ga_rope_kv_write(_ptr(qkv), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
                                _ptr(k_pages), _ptr(v_pages), _i(T), _i(num_heads), _i(num_kv_heads),
                                _i(head_dim), _i(rotary_dim), _i(page_size), _i(1 if write_kv else 0),
                                _i(_is_bf16(qkv.dtype)), _stream()), "rope_kv_write")


def _check_attention_operands(q, k_pages, v_pages, block_table, token_entry, positions, nh, nkv, hd):
    _dev(q, k_pages, v_pages, block_table, token_entry, positions)
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd, "q must be [T, >= nh*hd] with unit inner stride")
    _need(nkv > 0 and nh % nkv == 0, "num_heads %d is not a multiple of num_kv_heads %d" % (nh, nkv))
    for p in (k_pages, v_pages):
        _need(p.dtype == q.dtype and p.dim() == 4 and p.is_contiguous() and p.shape[1] == nkv and p.shape[3] == hd,
              "cache pages must be contiguous %s [pages, %d, page_size, %d]" % (q.dtype, nkv, hd))
    _need(k_pages.shape == v_pages.shape, "k and v pages differ in shape")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [entries, width]")
    for name, x in (("token_entry", token_entry), ("positions", positions)):
        _need(x.dtype == torch.int32 and x.shape == (T,) and x.is_contiguous(), "%s must be contiguous int32 [T]" % name)
    return T


def paged_attention_generic(q, k_pages, v_pages, block_table, token_entry, positions, num_heads, num_kv_heads,
                            head_dim, scale, window=None, out=None):
    """q: rows of the fused projection ([T, >= nh*hd]; the first nh*hd columns are the queries).
    Token t attends to the keys of request token_entry[t] at positions
    [max(0, p - window + 1), p], p = positions[t].  Returns [T, nh*hd]."""
    T = _check_attention_operands(q, k_pages, v_pages, block_table, token_entry, positions, num_heads,
                                  num_kv_heads, head_dim)
    _need(head_dim % 8 == 0 and 0 < head_dim <= 256, "head_dim %d is not supported by the general attention kernel "
          "(multiples of 8 up to 256)" % head_dim)
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    _need(out.dtype == q.dtype and out.shape == (T, num_heads * head_dim) and out.stride(1) == 1, "out must be [T, nh*hd]")
    lib = build.load("attention_generic")
    _check(lib.ga_paged_attention_generic(
        _ptr(out), _i64(out.stride(0)), _ptr(q), _i64(q.stride(0)), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        _i(block_table.shape[1]), _ptr(token_entry), _ptr(positions), _i(T), _i(num_heads), _i(num_kv_heads),
        _i(head_dim), _i(k_pages.shape[2]), _i(int(window) if window else 0), _f(scale), _i(_is_bf16(q.dtype)),
        _stream()), "paged_attention_generic")
    return out


def gemm_nt(a, w, bias=None, out=None, out_dtype=None):
    """a [M, K] . w [N, K]^T (+ bias [N]) -> [M, N]; 32-bit accumulation, plain FMA.  a and w share a
    dtype (float32 or bfloat16); out is that dtype or float32."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_nt: a [M, K] and w [N, K] do not agree: %s, %s"
          % (tuple(a.shape), tuple(w.shape)))
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
            _need(x.dtype == torch.float32 and x.shape == (R,) and x.is_contiguous(), "%s must be contiguous float32 [R]" % name)
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out.dtype == torch.int32 and out.shape == (R,) and out.is_contiguous(), "out must be contiguous int32 [R]")
    lib = build.load("sampling")
    _check(lib.ga_sample_rows(_ptr(out), _ptr(logits), _i64(logits.stride(0)), _i(R), _i(V), _ptr(temperature),
                              _ptr(uniform), _stream()), "sample_rows")
    return out


def gemm_skinny_supported(a, w):
    """Whether the matrix-core kernel for few rows takes these operands."""
    return False


def paged_attention(q, k_pages, v_pages, block_table, step, num_heads, num_kv_heads, head_dim, scale, window=None):
    """Attention of every token of the step over its request's pages.  Chooses the kernel: the general
    one in 32-bit; in bfloat16 the matrix-core kernels where they take the shape."""
    return paged_attention_generic(q, k_pages, v_pages, block_table, step.token_entry, step.positions, num_heads,
                                   num_kv_heads, head_dim, scale, window)
