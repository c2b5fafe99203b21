"""y = x . W^T (+ b), W stored [out, in] as in the checkpoint (ginfer/core/layer/linear.cc:9-20).

32-bit: the package's own FMA kernel (no matrix unit, no reduced-precision mode).  bfloat16: the
package's matrix-core kernel for few rows (decode), the BLAS library for many rows (prefill), which
is where the reference calls its library (ginfer/core/op/kernels/cuda/gemm_kernel/gemm_kernel.cu:42-164);
both accumulate in 32-bit and add the bias before the one rounding."""
import torch

from ..kernels import ops


def linear(x, weight, bias=None, out_dtype=None):
    """x [M, K], weight [N, K], bias [N] | None -> [M, N] in x's dtype (or float32 on request)."""
    if x.dtype == torch.float32:
        return ops.gemm_nt(x, weight, bias)
    if ops.gemm_skinny_supported(x, weight):
        return ops.gemm_skinny(x, weight, bias, out_dtype=out_dtype)
    if out_dtype == torch.float32:
        y = torch.mm(x, weight.t(), out_dtype=torch.float32)
        if bias is not None:
            y += bias
        return y
    if bias is not None:
        return torch.addmm(bias, x, weight.t())
    return torch.mm(x, weight.t())
