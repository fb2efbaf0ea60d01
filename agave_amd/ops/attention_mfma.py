"""Matrix-core (MFMA) attention over cache pages in tile order (bfloat16)."""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels, library
from .kernels import _F, _I, _L, _P

kernels.register_signatures("attention_mfma", {
    "agave_attn_decode_mfma": [_P, _L, _P, _L, _P, _P, _P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _F, _I, _I, _I, _I,
                               _I, _P],
    "agave_attn_decode_fused": [_P, _L, _P, _L, _P, _L, _P, _P, _F, _F, _P, _I, _F, _P, _L, _P, _P, _P, _P, _P, _I, _P, _I,
                                _P, _P, _I, _I, _I, _I, _F, _I, _I, _I, _I, _I, _I, _P],
    "agave_attn_prefill_mfma": [_P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "agave_attn_prefill_items_hw": [_I, _I],
    "agave_attn_prefill_items": [_P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P, _I, _I,
                                 _I, _P, _P, _P, _I, _P],
})

FUSED_HEAD_DIMS = (64, 128, 256)
MAX_SPLITS = 64              # what the merge inside the output product takes
SPLITS_AT_ONCE = 12          # and what it merges with one round trip to memory (at a batch of 1, 12 splits
                             # measured as fast as 16)
TARGET_WORKGROUPS = 256      # workgroups (of 4 waves) the general decode kernel aims for: one per compute unit
FAST_TARGET = 192            # the kernels that share half pages, 64 pages or more in reach: see split_plan
FAST_CAP = 240               # and with fewer pages in reach


def split_plan(page_span: int, units: int, head_dim: int = 0):
    """(splits, pages per split) for sequences spanning at most ``page_span`` pages when the launch
    has ``units`` (token, kv head) pairs.  The kernels for head sizes 64, 128 and 256 share a
    sequence's half pages evenly among the splits, four waves a split and a half page a wave at a
    time, so a split of n half pages takes ceil(n / 4) rounds.  The rules are fitted to whole
    decode steps of three model sizes at batches of 1 to 32.

    Fewer than 64 pages in reach (measured with 17): no more than 240 workgroups (256 are slower
    than 192 or 128; a second round of workgroups is far slower) and no more than 12 splits (what
    the output product merges with one round trip to memory).  Within that, the fewest rounds;
    among equals the fewest splits (each costs its partial results: 6 or 5 splits beat 7 and 8 at
    32 units, 3 beat 4 at 56 and 64), except that once every wave has at most one half page more
    splits still gain a little (12 beat 9 at a batch of 1 and of 4).

    64 pages or more: the keys outweigh the rest; as many splits as make 192 workgroups (6 beat 8
    at 32 units and 500 pages), but a launch that would leave half the compute units idle is split
    further (2 splits beat 1 at 128 units: by 1 % at 121 pages, by 4 % at 500).

    The general kernel gives each split a run of whole pages."""
    if head_dim in FUSED_HEAD_DIMS:
        u = max(units, 1)
        if page_span >= 64:
            splits = FAST_TARGET // u
            if splits * u <= TARGET_WORKGROUPS // 2:
                splits = TARGET_WORKGROUPS // u
            splits = max(1, min(splits, page_span, MAX_SPLITS))
        else:
            half_pages = 2 * page_span
            cap = max(1, min(FAST_CAP // u, page_span, SPLITS_AT_ONCE))

            def rounds(s):
                return -(-(-(-half_pages // s)) // 4)
            splits = min(range(1, cap + 1), key=lambda s: (rounds(s), s))
            if rounds(splits) == 1:
                splits = cap
        return splits, -(-page_span // splits)
    want = max(1, min(page_span, -(-TARGET_WORKGROUPS // max(units, 1))))
    per = -(-page_span // want)
    return -(-page_span // per), per


ITEM_PLACES = 192            # items are sized as if three quarters of the compute units' places were there: measured,
                             # fewer and larger pieces beat an even share (a piece more costs its partial results)
ITEM_MIN_PAGES = 4           # pages an item holds at least (what an item costs besides its pages is about a page)
ITEM_MAX_PIECES = 3
ITEM_MAX_PARTIAL_BYTES = 1 << 30


def plan_prefill_items(pos0, n_new, window: Optional[int], blk_len: int, heads_of_block: int, n_heads: int,
                       head_dim: int):
    """Cut a step of several tokens per sequence into items of about equal work for the item
    kernel.  A block is ``blk_len`` consecutive tokens of a sequence; it sees the pages from the
    window's edge of its first token to its last token.  With ``heads_of_block`` workgroups per
    item (kv heads times head chunks) and ITEM_PLACES workgroups running at a time, an item should
    hold about total / places pages; a block that sees more is cut into up to three pieces (whose
    partial results a second kernel merges), unless the partial results of the whole step would
    not fit a gigabyte.  Returns (items [n, 6] int32 sorted by falling size, pieces per token [N]
    int32, most pieces, most pages of an item)."""
    import numpy as np
    blocks = []                                   # (sequence, first token within the sequence, first page, pages)
    for b, (p0, n) in enumerate(zip(pos0, n_new)):
        for blk0 in range(0, n, blk_len):
            first, last = p0 + blk0, p0 + min(n, blk0 + blk_len) - 1
            lo = max(0, first - window + 1) if window else 0
            blocks.append((b, blk0, lo // 64, last // 64 - lo // 64 + 1))
    total = sum(blk[3] for blk in blocks) * heads_of_block
    per_item = max(ITEM_MIN_PAGES, -(-total // ITEM_PLACES))
    n_tokens = sum(n_new)
    may_cut = n_tokens * n_heads * ITEM_MAX_PIECES * (head_dim + 2) * 4 <= ITEM_MAX_PARTIAL_BYTES
    items = []
    tok_pieces = np.ones(n_tokens, dtype=np.int32)
    starts = np.concatenate([[0], np.cumsum(n_new)])
    max_pieces = 1
    for b, blk0, pg0, npg in blocks:
        pieces = min(ITEM_MAX_PIECES, -(-npg // per_item)) if may_cut else 1
        max_pieces = max(max_pieces, pieces)
        if pieces > 1:
            tok_pieces[starts[b] + blk0:starts[b] + min(n_new[b], blk0 + blk_len)] = pieces
        for k in range(pieces):
            lo, hi = k * npg // pieces, (k + 1) * npg // pieces
            items.append((b, blk0, pg0 + lo, hi - lo, k, pieces))
    items.sort(key=lambda it: -it[3])
    arr = np.asarray(items, dtype=np.int32).reshape(-1, 6)
    return arr, tok_pieces, max_pieces, int(arr[:, 3].max()) if len(items) else 1


def prefill_by_items(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                     table: torch.Tensor, base: torch.Tensor, step, n_heads: int, n_kv: int, head_dim: int,
                     scale: float, window: Optional[int], width: int, n_pages: int) -> None:
    """Attention of a step that brings several tokens per sequence, head sizes 64, 128 and 256."""
    import numpy as np
    lib = kernels.lib("attention_mfma")
    hw = int(lib.agave_attn_prefill_items_hw(n_heads, n_kv))
    # (the rows that pad a step to a fixed multiple are rows of its sequence like the others: every
    # step of that shape then has the same plan, whatever its real length)
    n_pad = getattr(step, "n_pad", 0)
    n_rows = list(step.n_new)
    n_rows[-1] += n_pad
    waves = 8 if max(n_rows) > 32 else 4           # eight waves once a sequence brings enough tokens for them
    blk_len = (waves // hw) * 16
    chunks = -(-(n_heads // n_kv) // hw)
    cache = step.__dict__.setdefault("_prefill_items", {})
    key = (window, blk_len, n_kv * chunks, n_heads, head_dim)
    plan = cache.get(key)
    if plan is None:
        items, tok_pieces, max_pieces, max_item_pages = plan_prefill_items(step.pos0, n_rows, window, blk_len,
                                                                           n_kv * chunks, n_heads, head_dim)
        both = torch.from_numpy(np.concatenate([items.reshape(-1), tok_pieces])).to(q.device)
        plan = cache[key] = (both[:items.size].view(-1, 6), both[items.size:], max_pieces, max_item_pages)
    items_dev, pieces_dev, max_pieces, max_item_pages = plan
    n = step.n_tokens
    part_o = part_ml = None
    if max_pieces > 1:
        ws = step.workspace
        part_o = ws.get("attn_part_o", n * n_heads * max_pieces, head_dim, torch.float32)
        part_ml = ws.get("attn_part_ml", n * n_heads * max_pieces, 2, torch.float32)
    library.call(lib, "agave_attn_prefill_items", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
                 k_pages.data_ptr(), v_pages.data_ptr(), table.data_ptr(), width, base.data_ptr(), n_pages,
                 step.tok_seq.data_ptr(), step.tok_pos.data_ptr(), step.cu_dev.data_ptr(), step.n_seqs, n, n_heads, n_kv,
                 head_dim, scale, int(window or 0), items_dev.data_ptr(), items_dev.shape[0], waves, max_item_pages,
                 pieces_dev.data_ptr(), kernels.ptr(part_o), kernels.ptr(part_ml), max_pieces, kernels.stream())


def check_table_reach(pos0, n_new, window: Optional[int], base, width: int) -> None:
    """Raise unless every sequence's table row covers what its tokens of this step reach: the row's
    first column (page index ``base[b]``) must not lie after the oldest page a query reaches, and
    the newest page written must lie inside the row's ``width`` columns.  The prefill kernel keeps
    a row's ids in an array of ``width`` entries and indexes it by page index minus the first
    page it needs; a table that is narrower than the reach would send it outside."""
    for b, (p0, n, b0) in enumerate(zip(pos0, n_new, base)):
        first = (max(0, p0 - window + 1) if window else 0) // 64
        last = (p0 + n - 1) // 64
        if b0 > first:
            raise ValueError(f"attention: sequence {b}'s table row starts at page {b0}, its queries reach back to page {first}")
        if last - b0 + 1 > width:
            raise ValueError(f"attention: sequence {b} reaches pages {b0}..{last}, the table has {width} columns")


def attention(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, table: torch.Tensor,
              base: torch.Tensor, step, n_heads: int, n_kv: int, head_dim: int, scale: float,
              window: Optional[int]) -> None:
    if not (q.is_cuda and out.is_cuda and k_pages.is_cuda):
        raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")
    n = step.n_tokens
    if q.dtype != torch.bfloat16 or q.shape != (n, n_heads * head_dim) or out.shape != q.shape or out.dtype != q.dtype:
        raise ValueError(f"attention: q and out must be bfloat16 [{n}, {n_heads * head_dim}]")
    if q.stride(1) != 1 or out.stride(1) != 1:
        raise ValueError("attention: q and out need contiguous rows")
    n_pages = kernels._check_pages(k_pages, v_pages, n_kv, head_dim, q.dtype, packed=True)
    width = kernels._check_table(table, base, step.tok_seq)
    base_host = getattr(step, "base_of", lambda t: None)(base)
    if base_host is not None:
        check_table_reach(step.pos0, step.n_new, window, base_host, width)
    lib = kernels.lib("attention_mfma")
    w = int(window or 0)
    if step.is_decode:
        span = step.page_span(window)
        chunks = -(-(n_heads // n_kv) // 16)
        splits, per = split_plan(span, n * n_kv * chunks, head_dim)
        part_o = part_ml = None
        if splits > 1:
            ws = step.workspace
            part_o = ws.get("attn_part_o", n * n_heads * splits, head_dim, torch.float32)
            part_ml = ws.get("attn_part_ml", n * n_heads * splits, 2, torch.float32)
        library.call(lib, "agave_attn_decode_mfma", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
                     kernels.ptr(part_o), kernels.ptr(part_ml), k_pages.data_ptr(), v_pages.data_ptr(),
                     table.data_ptr(), width, base.data_ptr(), n_pages, step.tok_seq.data_ptr(),
                     step.tok_pos.data_ptr(), n, n_heads, n_kv, head_dim, scale, w, splits, per,
                     1 if step.n_seqs == n else 0, 1 if getattr(step, "tables_start_at_reach", False) else 0,
                     kernels.stream())
    elif head_dim in FUSED_HEAD_DIMS:
        prefill_by_items(q, out, k_pages, v_pages, table, base, step, n_heads, n_kv, head_dim, scale, window, width, n_pages)
    else:
        library.call(lib, "agave_attn_prefill_mfma", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
                     k_pages.data_ptr(), v_pages.data_ptr(), table.data_ptr(), width, base.data_ptr(), n_pages,
                     step.tok_seq.data_ptr(), step.tok_pos.data_ptr(), step.cu_dev.data_ptr(), step.n_seqs,
                     step.max_new + getattr(step, "n_pad", 0), n, n_heads, n_kv, head_dim, scale, w, kernels.stream())


def decode_fused(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], out: torch.Tensor,
                 q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps_q: float, eps_k: float,
                 inv_freq: Optional[torch.Tensor], pos_scale: float, k_pages: torch.Tensor, v_pages: torch.Tensor,
                 table: torch.Tensor, base: torch.Tensor, step, n_heads: int, n_kv: int, head_dim: int, scale: float,
                 window: Optional[int], partials_ok=None):
    """A decode step's attention from the raw projections: the kernel normalises and rotates q and
    k, writes k and v into their pages (``k`` None: nothing is appended) and attends.
    ``partials_ok``: a function of the number of splits that says whether the caller's next kernel
    can merge the splits' partial results itself; if it says so and the step is split, they are returned as ``(part_o [n, heads, splits, head_dim], part_ml [n, heads,
    splits, 2])`` and ``out`` is left alone.  Otherwise None is returned and ``out`` is written."""
    n = step.n_tokens
    if not step.is_decode or head_dim not in FUSED_HEAD_DIMS:
        raise ValueError("decode_fused: needs a decode step and a head size of 64, 128 or 256")
    for name, t, cols in (("q", q, n_heads * head_dim), ("k", k, n_kv * head_dim), ("v", v, n_kv * head_dim),
                          ("out", out, n_heads * head_dim)):
        if t is None:
            continue
        if not t.is_cuda or t.dtype != torch.bfloat16 or t.shape != (n, cols) or t.stride(1) != 1:
            raise ValueError(f"decode_fused: {name} must be bfloat16 [{n}, {cols}] on the GPU with contiguous rows")
    if (k is None) != (v is None):
        raise ValueError("decode_fused: k and v come together")
    kernels._f32vec(q_gain, "q_gain", head_dim)
    kernels._f32vec(k_gain, "k_gain", head_dim)
    rot_half = 0
    if inv_freq is not None:
        rot_half = inv_freq.numel()
        kernels._f32vec(inv_freq, "inv_freq", rot_half)
    kernels._dev(q, k, v, out, q_gain, k_gain, inv_freq, k_pages, v_pages, table, base)
    n_pages = kernels._check_pages(k_pages, v_pages, n_kv, head_dim, q.dtype, packed=True)
    width = kernels._check_table(table, base, step.tok_seq)
    span = step.page_span(window)
    chunks = -(-(n_heads // n_kv) // 16)
    splits, per = split_plan(span, n * n_kv * chunks, head_dim)
    part_o = part_ml = None
    if splits > 1:
        ws = step.workspace
        part_o = ws.get("attn_part_o", n * n_heads * splits, head_dim, torch.float32)
        part_ml = ws.get("attn_part_ml", n * n_heads * splits, 2, torch.float32)
    leave = bool(splits > 1 and partials_ok is not None and partials_ok(splits))
    library.call(kernels.lib("attention_mfma"), "agave_attn_decode_fused", q.data_ptr(), q.stride(0),
                 kernels.ptr(k), k.stride(0) if k is not None else 0, kernels.ptr(v),
                 v.stride(0) if v is not None else 0, kernels.ptr(q_gain), kernels.ptr(k_gain), eps_q, eps_k,
                 kernels.ptr(inv_freq), rot_half, pos_scale, out.data_ptr(), out.stride(0), kernels.ptr(part_o),
                 kernels.ptr(part_ml), k_pages.data_ptr(), v_pages.data_ptr(), table.data_ptr(), width,
                 base.data_ptr(), n_pages, step.tok_seq.data_ptr(), step.tok_pos.data_ptr(), n, n_heads, n_kv,
                 head_dim, scale, int(window or 0), splits, per, 1 if step.n_seqs == n else 0,
                 1 if getattr(step, "tables_start_at_reach", False) else 0, 1 if leave else 0, kernels.stream())
    if leave:
        return part_o.view(n, n_heads, splits, head_dim), part_ml.view(n, n_heads, splits, 2)
    return None
