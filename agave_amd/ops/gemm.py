"""Choosing the matrix-product kernel for a linear layer."""
from __future__ import annotations

import torch

from . import gemm_mfma, kernels


def linear(x: torch.Tensor, lin, out: torch.Tensor) -> None:
    """out[N, out_features] = x[N, in_features] @ lin.weight^T."""
    if x.dim() != 2 or x.shape[1] != lin.in_features:
        raise ValueError(f"{lin.name}: input is {tuple(x.shape)}, weight takes {lin.in_features} columns")
    if out.shape != (x.shape[0], lin.out_features):
        raise ValueError(f"{lin.name}: output is {tuple(out.shape)}, needs {(x.shape[0], lin.out_features)}")
    if getattr(lin, "packed", None) is not None:
        if gemm_mfma.try_linear(x, lin, out):
            return
        raise ValueError(f"{lin.name}: the matrix-core product needs a 16-byte aligned bfloat16 input whose row "
                         f"stride is a multiple of 8, got {tuple(x.shape)} {x.dtype} strides {x.stride()}")
    kernels.gemm_plain(x, lin.weight, out)
