"""Choosing the attention kernel for a step."""
from __future__ import annotations

from typing import Optional

import torch

from . import attention_mfma, kernels


def attention(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
              table: torch.Tensor, base: torch.Tensor, step, n_heads: int, n_kv: int, head_dim: int,
              scale: float, window: Optional[int], packed: bool = False) -> None:
    """Attention of the step's tokens over their sequences' cache pages (which already hold the
    step's own keys and values).  Pages in the matrix cores' tile order go to the MFMA kernels,
    pages stored row by row to the plain kernel."""
    if packed:
        attention_mfma.attention(q, out, k_pages, v_pages, table, base, step, n_heads, n_kv, head_dim, scale, window)
        return
    kernels.attn_plain(q, out, k_pages, v_pages, table, base, step.tok_seq, step.tok_pos,
                       n_heads, n_kv, head_dim, scale, window)


def qk_attention(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], q_rot: torch.Tensor,
                 out: torch.Tensor, q_gain, k_gain, eps_q: float, eps_k: float, inv_freq, pos_scale: float,
                 k_pages: torch.Tensor, v_pages: torch.Tensor, table: torch.Tensor, base: torch.Tensor, step,
                 n_heads: int, n_kv: int, head_dim: int, scale: float, window: Optional[int], packed: bool,
                 partials_ok=None):
    """Head norm and rotation of q and k, k and v into the cache, and attention.  A decode step over
    pages in tile order does all of it in one kernel; otherwise the q/k kernel runs first (q into
    ``q_rot``) and the attention kernel after it.  ``partials_ok``: see
    :func:`agave_amd.ops.attention_mfma.decode_fused`; returns the partial results or None."""
    if packed and step.is_decode:
        if head_dim in attention_mfma.FUSED_HEAD_DIMS:
            return attention_mfma.decode_fused(q, k, v, out, q_gain, k_gain, eps_q, eps_k, inv_freq, pos_scale, k_pages,
                                               v_pages, table, base, step, n_heads, n_kv, head_dim, scale, window,
                                               partials_ok=partials_ok)
    kernels.qk_norm_rope_kv(q, k, v, q_rot, q_gain, k_gain, eps_q, eps_k, inv_freq, pos_scale, step.tok_seq,
                            step.tok_pos, k_pages, v_pages, table, base, n_heads, n_kv, head_dim, packed)
    attention(q_rot, out, k_pages, v_pages, table, base, step, n_heads, n_kv, head_dim, scale, window, packed)
    return None
