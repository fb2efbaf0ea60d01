"""Choosing the attention kernel for a step."""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels


def attention(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
              table: torch.Tensor, base: torch.Tensor, step, n_heads: int, n_kv: int, head_dim: int,
              scale: float, window: Optional[int], packed: bool = False) -> None:
    """Attention of the step's tokens over their sequences' cache pages (which already hold the
    step's own keys and values).  Pages in the matrix cores' tile order go to the MFMA kernels,
    pages stored row by row to the plain kernel."""
    if packed:
        from . import attention_mfma
        attention_mfma.attention(q, out, k_pages, v_pages, table, base, step, n_heads, n_kv, head_dim, scale, window)
        return
    kernels.attn_plain(q, out, k_pages, v_pages, table, base, step.tok_seq, step.tok_pos,
                       n_heads, n_kv, head_dim, scale, window)
