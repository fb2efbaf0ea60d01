"""Python faces of the HIP entry points.

Every function takes device tensors, checks on the host what the kernel and its grid
assume (device, dtype, contiguity, shapes), and launches on the current stream.  There is
no other implementation behind them: a tensor that is not on the GPU is an error.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import library

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

_SIGNATURES = {
    "elementwise": {
        "agave_embed_scale": [_I, _P, _P, _F, _P, _I, _I, _I, _P],
        "agave_residual_norm": [_I, _P, _P, _L, _I, _L, _P, _F, _P, _L, _P, _F, _P, _I, _I, _P, _P],
        "agave_qk_norm_rope_kv": [_I, _P, _L, _P, _L, _P, _L, _P, _L, _P, _P, _F, _F, _P, _I, _F,
                                  _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P],
        "agave_geglu": [_I, _P, _L, _P, _L, _P, _L, _I, _I, _P],
        "agave_gated_act": [_I, _I, _P, _L, _P, _L, _P, _L, _I, _I, _P],
        "agave_cast": [_I, _P, _I, _P, _L, _P],
        "agave_add_bias": [_I, _P, _L, _P, _I, _I, _P],
        "agave_scale_cap": [_P, _L, _F, _F, _P],
        "agave_gather_rows": [_I, _P, _P, _P, _L, _I, _I, _P],
    },
    "gemm": {
        "agave_gemm_plain": [_I, _P, _L, _I, _P, _L, _I, _P, _L, _I, _I, _I, _P],
    },
    "attention_plain": {
        "agave_attn_plain": [_I, _P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _F, _I, _P],
    },
}

_ready = {}


def register_signatures(library_name: str, signatures: dict) -> None:
    """Add entry points of a further library (used by the MFMA and sampling modules)."""
    _SIGNATURES.setdefault(library_name, {}).update(signatures)
    _ready.pop(library_name, None)


def lib(name: str):
    got = _ready.get(name)
    if got is not None:
        return got
    handle = library.load(name)
    for fn, argtypes in _SIGNATURES.get(name, {}).items():
        f = getattr(handle, fn)
        f.argtypes = argtypes
        f.restype = ctypes.c_int
    _ready[name] = handle
    return handle


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream() -> int:
    """The current HIP stream's handle.  Every launch asks for it, so it is read through torch's own
    raw accessor where there is one (a fraction of a microsecond; the stream object costs several)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}") from None


def ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride in elements of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{what}: expected a 2-D tensor with contiguous rows, got shape "
                         f"{tuple(t.shape)} strides {t.stride()}")
    return t.stride(0)


def _i32(t: Optional[torch.Tensor], what: str, n: Optional[int] = None) -> None:
    if t is None:
        return
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{what}: expected a contiguous int32 tensor")
    if n is not None and t.numel() < n:
        raise ValueError(f"{what}: holds {t.numel()} entries, needs {n}")


def _f32vec(t: Optional[torch.Tensor], what: str, n: int) -> None:
    if t is None:
        return
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
        raise TypeError(f"{what}: expected {n} contiguous float32 values, got {tuple(t.shape)} {t.dtype}")


# ---------------------------------------------------------------------------
def embed_scale(tokens: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor) -> None:
    """out[t] = table[tokens[t]] * scale, out in float32."""
    _dev(tokens, table, out)
    n = tokens.numel()
    _i32(tokens, "tokens")
    if table.dim() != 2 or not table.is_contiguous():
        raise ValueError("embedding table must be a contiguous [vocab, hidden] tensor")
    vocab, e = table.shape
    if out.dtype != torch.float32 or not out.is_contiguous() or out.shape != (n, e):
        raise ValueError(f"embed_scale: out must be float32 [{n}, {e}], got {tuple(out.shape)} {out.dtype}")
    h = lib("elementwise")
    library.call(h, "agave_embed_scale", dt(table), ptr(tokens), ptr(table), scale, ptr(out), n, e, vocab, stream())


def residual_norm(h: torch.Tensor, branch: Optional[torch.Tensor], post_gain: Optional[torch.Tensor],
                  post_eps: float, out: Optional[torch.Tensor], pre_gain: Optional[torch.Tensor],
                  pre_eps: float, rows: Optional[torch.Tensor] = None, src: Optional[torch.Tensor] = None) -> None:
    """If ``branch``: h += rmsnorm(branch) * post_gain.  If ``out``: out = rmsnorm(h) * pre_gain.
    ``rows`` (int32) picks the rows of ``h`` that ``out`` is computed for.  A three-dimensional
    float32 ``branch`` [slices, rows, hidden] stands for the sum of its slices (a product that was
    shared out along its columns).  ``src``: the residual rows are read from this tensor and
    written to ``h`` (a kernel that could not update the stream in place left it there)."""
    _dev(h, branch, post_gain, out, pre_gain, rows, src)
    if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
        raise ValueError("residual stream must be a contiguous float32 [rows, hidden] tensor")
    n_h, e = h.shape
    n = n_h if rows is None else rows.numel()
    _i32(rows, "rows")
    if src is not None:
        if src.dtype != torch.float32 or src.shape != h.shape or not src.is_contiguous() or src.data_ptr() == h.data_ptr():
            raise ValueError("the source of the residual rows must be another contiguous float32 tensor of h's shape")
        if rows is not None:
            raise ValueError("rows are gathered from the residual stream itself, not from another source")
    act = branch if branch is not None else out
    if act is None:
        if src is not None:
            h.copy_(src)
        return
    ldb = ldo = n_parts = part_stride = 0
    if branch is not None and branch.dim() == 3:
        if branch.dtype != torch.float32 or branch.shape[1:] != (n_h, e) or not branch.is_contiguous():
            raise ValueError(f"partial sums must be a contiguous float32 [slices, {n_h}, {e}] tensor")
        n_parts, part_stride, ldb = branch.shape[0], n_h * e, e
        _f32vec(post_gain, "post_gain", e)
        if out is not None:
            act = out
    elif branch is not None:
        ldb = _rows(branch, "branch")
        if branch.shape != (n_h, e):
            raise ValueError(f"branch must be [{n_h}, {e}], got {tuple(branch.shape)}")
        _f32vec(post_gain, "post_gain", e)
    if out is not None:
        ldo = _rows(out, "out")
        if out.shape != (n, e):
            raise ValueError(f"out must be [{n}, {e}], got {tuple(out.shape)}")
        _f32vec(pre_gain, "pre_gain", e)
        if branch is not None and n_parts == 0 and branch.dtype != out.dtype:
            raise TypeError("branch and out must have the same dtype")
    library.call(lib("elementwise"), "agave_residual_norm", dt(act), ptr(h), ptr(branch), ldb, n_parts, part_stride,
                 ptr(post_gain), post_eps, ptr(out), ldo, ptr(pre_gain), pre_eps, ptr(rows), n, e, ptr(src), stream())


def qk_norm_rope_kv(q: Optional[torch.Tensor], k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                    q_out: Optional[torch.Tensor], q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor],
                    eps_q: float, eps_k: float, inv_freq: Optional[torch.Tensor], pos_scale: float,
                    tok_seq: torch.Tensor, tok_pos: torch.Tensor, k_pages: Optional[torch.Tensor],
                    v_pages: Optional[torch.Tensor], table: Optional[torch.Tensor], base: Optional[torch.Tensor],
                    n_heads: int, n_kv: int, head_dim: int, packed: bool = False) -> None:
    """Per-head RMSNorm of q and k, rotation, q to ``q_out`` and k, v into their cache pages.
    ``k`` None: only q is processed (a layer that reads another layer's cache).  ``packed``:
    the pages are in the matrix cores' tile order."""
    _dev(q, k, v, q_out, q_gain, k_gain, inv_freq, tok_seq, tok_pos, k_pages, v_pages, table, base)
    n = tok_pos.numel()
    _i32(tok_pos, "tok_pos")
    _i32(tok_seq, "tok_seq", n)
    ref = q if q is not None else k
    d = dt(ref)
    ldq = ldqo = ldk = ldv = 0
    nh = nkv = 0
    if q is not None:
        nh = n_heads
        ldq, ldqo = _rows(q, "q"), _rows(q_out, "q_out")
        if q.shape != (n, nh * head_dim) or q_out.shape != (n, nh * head_dim) or q_out.dtype != q.dtype:
            raise ValueError(f"q and q_out must be [{n}, {nh * head_dim}] of one dtype")
        _f32vec(q_gain, "q_gain", head_dim)
    width = n_pages = 0
    if k is not None:
        nkv = n_kv
        ldk, ldv = _rows(k, "k"), _rows(v, "v")
        if k.shape != (n, nkv * head_dim) or v.shape != (n, nkv * head_dim) or k.dtype != ref.dtype or v.dtype != ref.dtype:
            raise ValueError(f"k and v must be [{n}, {nkv * head_dim}] of the activations' dtype")
        _f32vec(k_gain, "k_gain", head_dim)
        n_pages = _check_pages(k_pages, v_pages, nkv, head_dim, ref.dtype, packed)
        width = _check_table(table, base, tok_seq)
    rot_half = 0
    if inv_freq is not None:
        rot_half = inv_freq.numel()
        _f32vec(inv_freq, "inv_freq", rot_half)
    library.call(lib("elementwise"), "agave_qk_norm_rope_kv", d, ptr(q), ldq, ptr(k), ldk, ptr(v), ldv, ptr(q_out),
                 ldqo, ptr(q_gain), ptr(k_gain), eps_q, eps_k, ptr(inv_freq), rot_half, pos_scale, ptr(tok_seq),
                 ptr(tok_pos), ptr(k_pages), ptr(v_pages), ptr(table), width, ptr(base), n_pages, n, nh, nkv,
                 head_dim, 1 if (packed and k is not None) else 0, stream())


def _check_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, nkv: int, hd: int, dtype: torch.dtype,
                 packed: bool = False) -> int:
    hd_k = (hd + 31) // 32 * 32 if packed else hd       # packed K rows are padded to whole tiles
    if packed and (dtype != torch.bfloat16 or hd % 16):
        raise ValueError("packed cache pages need bfloat16 and a head size that is a multiple of 16")
    if k_pages.dim() != 4 or tuple(k_pages.shape[1:]) != (nkv, 64, hd_k) or not k_pages.is_contiguous():
        raise ValueError(f"K pages must be contiguous [pages, {nkv}, 64, {hd_k}], got {tuple(k_pages.shape)}")
    if v_pages.dim() != 4 or tuple(v_pages.shape[1:]) != (nkv, hd, 64) or not v_pages.is_contiguous():
        raise ValueError(f"V pages must be contiguous [pages, {nkv}, {hd}, 64], got {tuple(v_pages.shape)}")
    if k_pages.shape[0] != v_pages.shape[0] or k_pages.dtype != dtype or v_pages.dtype != dtype:
        raise ValueError("K and V pages must agree in page count and dtype with the activations")
    return k_pages.shape[0]


def _check_table(table: torch.Tensor, base: torch.Tensor, tok_seq: Optional[torch.Tensor]) -> int:
    if table.dtype != torch.int32 or table.dim() != 2 or not table.is_contiguous():
        raise TypeError("page table must be a contiguous int32 [sequences, width] tensor")
    _i32(base, "page base", table.shape[0])
    return table.shape[1]


# The activations of a gated feed-forward that the elementwise kernel knows, by the number it knows them by.
GATE_ACTIVATIONS = {"gelu_tanh": 0, "silu": 1, "gelu": 2, "relu": 3}


def gated_act(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor, activation: str = "gelu_tanh") -> None:
    """out = act(gate) * up, row by row; ``activation`` is one of ``GATE_ACTIVATIONS``."""
    _dev(gate, up, out)
    try:
        act = GATE_ACTIVATIONS[activation]
    except KeyError:
        raise ValueError(f"gated_act: unknown activation {activation!r}; known: {sorted(GATE_ACTIVATIONS)}") from None
    ldg, ldu, ldo = _rows(gate, "gate"), _rows(up, "up"), _rows(out, "out")
    if gate.shape != up.shape or gate.shape != out.shape or not (gate.dtype == up.dtype == out.dtype):
        raise ValueError("gated_act: gate, up and out must agree in shape and dtype")
    n, ff = gate.shape
    library.call(lib("elementwise"), "agave_gated_act", dt(gate), act, ptr(gate), ldg, ptr(up), ldu, ptr(out), ldo, n, ff,
                 stream())


def geglu(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor) -> None:
    """out = gelu_tanh(gate) * up, row by row."""
    gated_act(gate, up, out, "gelu_tanh")


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """y[r] += bias for every row of y (float32 or bfloat16, rows contiguous); the bias is float32."""
    _dev(y, bias)
    ldy = _rows(y, "y")
    _f32vec(bias, "bias", y.shape[1])
    library.call(lib("elementwise"), "agave_add_bias", dt(y), ptr(y), ldy, ptr(bias), y.shape[0], y.shape[1], stream())


def scale_cap(logits: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> None:
    """logits <- cap * tanh(scale * logits / cap) if ``cap`` > 0, scale * logits otherwise, in place
    (soft-capping as ``src/models/gemma4.zig:2365-2385`` states it)."""
    _dev(logits)
    if logits.dtype != torch.float32 or not logits.is_contiguous():
        raise ValueError("scale_cap: logits must be a contiguous float32 tensor")
    if cap < 0:
        raise ValueError("scale_cap: a cap cannot be negative")
    library.call(lib("elementwise"), "agave_scale_cap", ptr(logits), logits.numel(), float(scale), float(cap), stream())


def gather_rows(h: torch.Tensor, rows: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """out[i] = h[rows[i]] (all rows in order if ``rows`` is None), rounded to out's element type;
    ``h`` is the 32-bit residual stream.  The caller vouches that the row numbers lie inside ``h``."""
    _dev(h, rows, out)
    if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
        raise ValueError("gather_rows: the source must be a contiguous float32 [rows, hidden] tensor")
    n = h.shape[0] if rows is None else rows.numel()
    _i32(rows, "rows")
    ldo = _rows(out, "out")
    if out.shape != (n, h.shape[1]):
        raise ValueError(f"gather_rows: out must be [{n}, {h.shape[1]}], got {tuple(out.shape)}")
    library.call(lib("elementwise"), "agave_gather_rows", dt(out), ptr(h), ptr(rows), ptr(out), ldo, n, h.shape[1], stream())


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _dev(src, dst)
    if not (src.is_contiguous() and dst.is_contiguous()) or src.numel() != dst.numel():
        raise ValueError("cast: tensors must be contiguous and of equal size")
    library.call(lib("elementwise"), "agave_cast", dt(src), ptr(src), dt(dst), ptr(dst), src.numel(), stream())


def gemm_plain(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor) -> None:
    """c[M,N] = a[M,K] @ w[N,K]^T with 32-bit accumulation (ordinary multiply-adds)."""
    _dev(a, w, c)
    lda, ldw, ldc = _rows(a, "a"), _rows(w, "w"), _rows(c, "c")
    m, k = a.shape
    n, k2 = w.shape
    if k != k2 or c.shape != (m, n):
        raise ValueError(f"gemm: shapes do not fit: a {tuple(a.shape)}, w {tuple(w.shape)}, c {tuple(c.shape)}")
    library.call(lib("gemm"), "agave_gemm_plain", dt(a), ptr(a), lda, dt(w), ptr(w), ldw, dt(c), ptr(c), ldc,
                 m, n, k, stream())


def attn_plain(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
               table: torch.Tensor, base: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor,
               n_heads: int, n_kv: int, head_dim: int, scale: float, window: Optional[int]) -> None:
    """Attention of every token over its sequence's cache pages (keys up to its own position,
    and not older than ``window`` - 1 positions back if a window is given)."""
    _dev(q, out, k_pages, v_pages, table, base, tok_seq, tok_pos)
    n = tok_pos.numel()
    _i32(tok_pos, "tok_pos")
    _i32(tok_seq, "tok_seq", n)
    ldq, ldo = _rows(q, "q"), _rows(out, "out")
    if q.shape != (n, n_heads * head_dim) or out.shape != q.shape or out.dtype != q.dtype:
        raise ValueError(f"attention: q and out must be [{n}, {n_heads * head_dim}] of one dtype")
    n_pages = _check_pages(k_pages, v_pages, n_kv, head_dim, q.dtype)
    width = _check_table(table, base, tok_seq)
    library.call(lib("attention_plain"), "agave_attn_plain", dt(q), ptr(q), ldq, ptr(out), ldo, ptr(k_pages),
                 ptr(v_pages), ptr(table), width, ptr(base), n_pages, ptr(tok_seq), ptr(tok_pos), n, n_heads, n_kv,
                 head_dim, scale, int(window or 0), stream())
