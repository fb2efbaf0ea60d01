"""Matrix-core (MFMA) attention for bfloat16.  Filled in after the plain path."""
from __future__ import annotations


def try_attention(q, out, k_pages, v_pages, table, base, step, n_heads, n_kv, head_dim, scale, window) -> bool:
    return False
