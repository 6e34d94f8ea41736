"""Matrix products of the step: ``x @ weight.T`` for ``weight`` as a Linear stores it.

float32 runs through the hand-written FMA kernel (true 32-bit, fixed summation order).
bfloat16 with up to 64 rows (a decode step) runs through the hand-written matrix-core kernel, which
also folds the norm before a product, the residual add after it and the SwiGLU activation into
itself; with more rows the vendor library's product runs, which is also what the
reference's engine uses for its projections (reference src/qwen25vl_lite/text.py:61-66, 80-90).
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from . import kernels, skinny

__all__ = ["NormedRows", "linear", "linear_into", "gate_up_swiglu", "tune_library_products"]


class NormedRows:
    """``rmsnorm(h) * weight`` that has not been computed yet: a product that takes it may compute it
    on the way; anything else calls :meth:`materialize`."""

    def __init__(self, h: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype):
        self.h, self.weight, self.eps, self.dtype = h, weight, eps, dtype
        self.shape = h.shape

    def materialize(self) -> torch.Tensor:
        return kernels.add_rmsnorm(self.h, None, self.weight, self.eps, self.dtype)


def _library(x: torch.Tensor, weight: torch.Tensor, bias, out_dtype) -> torch.Tensor:
    if out_dtype == torch.float32:
        y = torch.mm(x, weight.t(), out_dtype=torch.float32)  # float32 accumulator written out unrounded
    else:
        y = torch.nn.functional.linear(x, weight)
    if bias is not None:
        y = y + bias.to(y.dtype)
    return y


def linear(x: Union[torch.Tensor, NormedRows], weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x [M, K] @ weight[N, K].T (+ bias)``.  ``out_dtype`` float32 is allowed for bfloat16
    operands (the products are accumulated in float32 either way).  ``x`` may be :class:`NormedRows`."""
    lazy = isinstance(x, NormedRows)
    m, k = x.shape
    if not weight.is_cuda:
        raise kernels.KernelError("linear has no CPU path: its tensors must be on the GPU")
    if weight.dtype == torch.bfloat16:
        few = m <= skinny.ONE_BLOCK_ROWS     # beyond, the library streams a plain product faster
        if lazy and few and skinny.takes_resident(m, k, weight, norm=True):
            return skinny.resident_product(weight, h=x.h, norm_weight=x.weight, eps=x.eps, bias=bias,
                                           out_dtype=out_dtype or torch.bfloat16)
        if lazy:
            x = x.materialize()
        if x.dtype != torch.bfloat16:
            raise kernels.KernelError(f"linear: operands {x.dtype}/{weight.dtype} are not built")
        if few and skinny.takes_resident(m, k, weight) and _aligned(x):
            return skinny.resident_product(weight, x=x, bias=bias, out_dtype=out_dtype or torch.bfloat16)
        return _library(x, weight, bias, out_dtype)
    if lazy:
        x = x.materialize()
    if not x.is_cuda:
        raise kernels.KernelError("linear has no CPU path: its tensors must be on the GPU")
    if x.dtype == torch.float32 and weight.dtype == torch.float32:
        return kernels.gemm_f32(x, weight, bias)
    raise kernels.KernelError(f"linear: operands {x.dtype}/{weight.dtype} are not built")


def _aligned(x: torch.Tensor) -> bool:
    return x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0


def linear_into(residual: Optional[torch.Tensor], x: torch.Tensor, weight: torch.Tensor) -> Optional[torch.Tensor]:
    """``residual += x @ weight.T`` inside the product's kernel where that exists (few bfloat16
    rows): then None is returned.  Otherwise what is to be added is returned and the caller hands
    it on to whoever adds it (the next norm's kernel): the product ``[M, N]``, or float32
    ``[slabs, M, N]`` whose slabs are added in order (the split kernel)."""
    m, k = x.shape
    fast = x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and _aligned(x)
    if fast and skinny.prefers_split(m, k, weight):
        return skinny.split_product(weight, x)
    if (fast and m <= skinny.ONE_BLOCK_ROWS and residual is not None and skinny.takes_resident(m, k, weight)
            and residual.dtype == torch.float32 and residual.shape == (m, weight.shape[0]) and residual.stride(1) == 1):
        skinny.resident_product(weight, x=x, epilogue=skinny.RESIDUAL, out=residual)
        return None
    # More rows: the library's product.  Its bfloat16 output is the form it is tuned for (float32
    # output costs a tenth of a 2,048-token prefill); the sum into the residual stays float32.
    return linear(x, weight, out_dtype=torch.float32 if m <= skinny.ONE_BLOCK_ROWS else None)


def tune_library_products(enable: bool = True, max_ms: int = 3000) -> None:
    """Let PyTorch's TunableOp pick the fastest library kernel for every product shape it meets
    (each new shape costs a few seconds once; its choices are kept in a per-user file under the
    temporary directory).  Meant for runs with few distinct shapes, such as a benchmark; off by
    default."""
    import os
    import tempfile

    import torch.cuda.tunable as tunable

    if enable:
        tunable.set_filename(os.path.join(tempfile.gettempdir(), f"qwen25vl_lite_amd-tunableop-{os.getuid()}.csv"))
        tunable.set_max_tuning_duration(int(max_ms))
    tunable.enable(enable)
    tunable.tuning_enable(enable)


def gate_up_swiglu(x: Union[torch.Tensor, NormedRows], weight: torch.Tensor, grouped: bool) -> torch.Tensor:
    """``silu(x Wg^T) * (x Wu^T)`` for ``weight`` holding gate and up rows: plain (gate rows, then up
    rows) or ``grouped`` (alternating groups of 8 gate rows and 8 up rows).  With few bfloat16 rows
    and grouped rows the activation is applied inside the product's kernel."""
    m, k = x.shape
    if (grouped and weight.dtype == torch.bfloat16 and weight.is_cuda and weight.shape[0] % 16 == 0
            and m <= skinny.ONE_BLOCK_ROWS):
        lazy = isinstance(x, NormedRows)
        if lazy and skinny.takes_resident(m, k, weight, norm=True):
            return skinny.resident_product(weight, h=x.h, norm_weight=x.weight, eps=x.eps, epilogue=skinny.SWIGLU)
        if not lazy and x.dtype == torch.bfloat16 and skinny.takes_resident(m, k, weight) and _aligned(x):
            return skinny.resident_product(weight, x=x, epilogue=skinny.SWIGLU)
    return kernels.swiglu(linear(x, weight), grouped=grouped)
