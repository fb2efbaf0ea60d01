"""Matrix-core (MFMA) matrix products for bfloat16 weights in the packed layout."""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels, library
from .kernels import _F, _I, _L, _P

kernels.register_signatures("gemm_mfma", {
    "agave_pack_w16": [_P, _L, _P, _I, _I, _I, _I, _P],
    "agave_embed_scale_packed": [_P, _P, _F, _P, _I, _I, _I, _P],
    "agave_gemm_skinny": [_P, _L, _P, _I, _P, _L, _I, _I, _I, _I, _I, _P],
    "agave_gemm_skinny_slices": [_I, _I, _I],
    "agave_gemm_row_normed_ok": [_I, _I, _I, _I],
    "agave_gemm_row_normed": [_P, _P, _P, _I, _I, _L, _P, _F, _P, _F, _P, _P, _I, _I, _I, _P],
    "agave_gemm_tiled_slices": [_I, _I, _I],
    "agave_gemm_tiled_in_slices": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
    "agave_gemm_tiled": [_P, _L, _P, _I, _P, _L, _I, _I, _I, _I, _P, _L, _P],
    "agave_gemm_tiled_as": [_P, _L, _P, _I, _P, _L, _I, _I, _I, _I, _I, _P],
    "agave_gemm_tiled_in_slices_as": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
    "agave_oproj_combine_heads_per_run": [_I, _I, _I, _I],
    "agave_gemm_oproj_combine": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _P],
})

SKINNY_MAX_M = 64


def pack_weight(weight: torch.Tensor, interleave_ff: int = 0) -> torch.Tensor:
    """Row-major bfloat16 W[N, K] -> packed tiles of 16 rows by 32 columns (a flat bfloat16
    tensor).  ``interleave_ff`` > 0: W is a stacked [gate; up] matrix of 2*ff rows whose rows are
    interleaved for the GeGLU epilogue."""
    if not weight.is_cuda or weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.stride(1) != 1:
        raise TypeError("pack_weight takes a bfloat16 GPU matrix with contiguous rows")
    n, k = weight.shape
    nb = (interleave_ff + 7) // 8 if interleave_ff else (n + 15) // 16
    kb = (k + 31) // 32
    packed = torch.empty(nb * kb * 512, dtype=torch.bfloat16, device=weight.device)
    library.call(kernels.lib("gemm_mfma"), "agave_pack_w16", weight.data_ptr(), weight.stride(0), packed.data_ptr(),
                 n, k, 1 if interleave_ff else 0, interleave_ff, kernels.stream())
    return packed


def _x_ok(x: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1 and x.shape[1] % 8 == 0
            and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0)


def product(x: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, n_out: int, epilogue: int = 0) -> None:
    """out[M, n_out] = x[M, K] @ W^T (epilogue 0) or gelu_tanh(gate) * up (epilogue 1), any M: the
    skinny kernel up to 64 rows, the tiled one above."""
    if x.shape[0] <= SKINNY_MAX_M:
        skinny(x, packed, out, n_out, epilogue)
    else:
        _launch("agave_gemm_tiled", x, packed, out, n_out, epilogue)


def skinny(x: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, n_out: int, epilogue: int = 0) -> None:
    """out[M, n_out] = x[M, K] @ W^T (epilogue 0) or gelu_tanh(gate) * up (epilogue 1) for M <= 64."""
    _launch("agave_gemm_skinny", x, packed, out, n_out, epilogue)


_normed_ok = {}


def normed_ok(m: int, n_out: int, k: int, epilogue: int = 0) -> bool:
    """Whether :func:`row_normed` takes a product of these sizes (the kernel library decides)."""
    key = (m, n_out, k, epilogue)
    got = _normed_ok.get(key)
    if got is None:
        got = _normed_ok[key] = bool(kernels.lib("gemm_mfma").agave_gemm_row_normed_ok(m, n_out, k, epilogue))
    return got


def row_normed(h_in: torch.Tensor, h_out: Optional[torch.Tensor], branch: Optional[torch.Tensor],
                  post_gain: Optional[torch.Tensor], post_eps: float, pre_gain: torch.Tensor, pre_eps: float,
                  packed: torch.Tensor, out: torch.Tensor, n_out: int, epilogue: int = 0) -> None:
    """out = rmsnorm(h') * pre_gain @ W^T (or its GeGLU) with h' = h_in + post(branch), for one row:
    the product's workgroups make the normalised row themselves, and h' goes to ``h_out``, which
    must be other memory than ``h_in``.  ``branch``: [1, K] in bfloat16 or float32, or float32
    slices [slices, 1, K] that add up to it, or None (then h' is h_in and nothing but ``out`` is
    written); ``post_gain`` None: the branch is added as it is."""
    for t in (h_in, h_out, branch, post_gain, pre_gain, packed, out):
        if t is not None and not t.is_cuda:
            raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")
    if h_in.dtype != torch.float32 or h_in.dim() != 2 or not h_in.is_contiguous():
        raise ValueError("row_normed: the residual row must be a contiguous float32 [1, K] tensor")
    m, k = h_in.shape
    if not normed_ok(m, n_out, k, epilogue):
        raise ValueError(f"row_normed: no kernel for {m} rows, {n_out} outputs and {k} columns")
    if out.dtype != torch.bfloat16 or out.dim() != 2 or out.shape != (m, n_out) or out.stride(1) != 1:
        raise ValueError(f"row_normed: out must be bfloat16 [{m}, {n_out}] with contiguous rows")
    if branch is not None and branch.dim() == 2 and branch.stride(0) < k:
        raise ValueError("row_normed: the branch's row is too short")
    nb = (n_out + 7) // 8 if epilogue else (n_out + 15) // 16
    if packed.numel() != nb * ((k + 31) // 32) * 512:
        raise ValueError("row_normed: the packed weight does not fit these sizes")
    for g, what in ((pre_gain, "pre_gain"), (post_gain, "post_gain")):
        if g is not None and (g.dtype != torch.float32 or not g.is_contiguous() or g.numel() != k):
            raise TypeError(f"row_normed: {what} must hold {k} contiguous float32 values")
    n_parts = part_stride = 0
    if branch is not None:
        if h_out is None or h_out.dtype != torch.float32 or h_out.shape != h_in.shape or not h_out.is_contiguous() \
                or h_out.data_ptr() == h_in.data_ptr():
            raise ValueError("row_normed: the sum needs a float32 tensor of its own, shaped like the residual row")
        if branch.dim() == 3:
            if branch.dtype != torch.float32 or branch.shape[1:] != (m, k) or not branch.is_contiguous():
                raise ValueError(f"row_normed: slices must be a contiguous float32 [slices, {m}, {k}] tensor")
            n_parts, part_stride = branch.shape[0], m * k
        elif branch.dtype not in (torch.float32, torch.bfloat16) or branch.shape != (m, k) or branch.stride(1) != 1:
            raise ValueError(f"row_normed: the branch must be [{m}, {k}] in float32 or bfloat16 with contiguous rows")
    library.call(kernels.lib("gemm_mfma"), "agave_gemm_row_normed", h_in.data_ptr(), kernels.ptr(h_out), kernels.ptr(branch),
                 1 if (branch is not None and branch.dtype == torch.float32) else 0, n_parts, part_stride,
                 kernels.ptr(post_gain), post_eps, pre_gain.data_ptr(), pre_eps, packed.data_ptr(), out.data_ptr(),
                 n_out, k, epilogue, kernels.stream())


_slices = {}


def slices_for(m: int, n_out: int, k: int) -> int:
    """How many 32-bit slices a product of few tokens is worth to a caller that can add them up
    (the kernel library decides: it knows how it cuts a product into workgroups)."""
    key = (m, n_out, k)
    got = _slices.get(key)
    if got is None:
        got = 1
        if 0 < m <= SKINNY_MAX_M:
            fn = kernels.lib("gemm_mfma").agave_gemm_skinny_slices
            got = _slices[key] = int(fn(m, n_out, k))
    return got


def tiled_slices_for(m: int, n_out: int, k: int) -> int:
    """The same for a product of many tokens: more than one where the tiles would leave many
    compute units idle and the columns are many."""
    key = (m, n_out, k)
    got = _slices.get(key)
    if got is None:
        got = 1
        if m > SKINNY_MAX_M and m * n_out * 4 * 8 <= TILED_SLICES_MAX_BYTES:       # (at most eight slices)
            got = int(kernels.lib("gemm_mfma").agave_gemm_tiled_slices(m, n_out, k))
        _slices[key] = got
    return got


TILED_SLICES_MAX_BYTES = 512 << 20       # what the slices of one product may take


def tiled_slices(x: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, n_out: int) -> None:
    """out[s] = the sums over the s-th run of columns of x[M, K] @ W^T for M > 64; out is float32
    [tiled_slices_for(M, n_out, K), M, n_out] and its slices add up to the product."""
    if not (x.is_cuda and packed.is_cuda and out.is_cuda):
        raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")
    if not _x_ok(x):
        raise ValueError("packed product: input must be 16-byte aligned bfloat16 rows with K and the row stride multiples of 8")
    m, k = x.shape
    if out.dtype != torch.float32 or out.dim() != 3 or out.shape[1:] != (m, n_out) or not out.is_contiguous():
        raise ValueError(f"partial sums must be a contiguous float32 [slices, {m}, {n_out}] tensor")
    if packed.numel() != ((n_out + 15) // 16) * ((k + 31) // 32) * 512:
        raise ValueError("packed product: the packed weight does not fit these sizes")
    library.call(kernels.lib("gemm_mfma"), "agave_gemm_tiled_in_slices", x.data_ptr(), x.stride(0), packed.data_ptr(),
                 out.data_ptr(), m, n_out, k, out.shape[0], kernels.stream())


TILE_SHAPES = ((256, 256), (128, 256), (128, 128), (64, 128))       # weight rows x tokens a workgroup


def tiled_as(x: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, n_out: int, tile: int, epilogue: int = 0) -> None:
    """:func:`product` in tiles of ``TILE_SHAPES[tile]`` whatever the library would choose (tests of
    every tile shape, measurements)."""
    if not (x.is_cuda and packed.is_cuda and out.is_cuda) or not _x_ok(x):
        raise ValueError("packed product: bfloat16 GPU rows, 16-byte aligned, K and the row stride multiples of 8")
    m, k = x.shape
    if out.dim() != 2 or out.shape != (m, n_out) or out.stride(1) != 1:
        raise ValueError(f"packed product: out must be [{m}, {n_out}] with contiguous rows")
    nb = (n_out + 7) // 8 if epilogue else (n_out + 15) // 16
    if packed.numel() != nb * ((k + 31) // 32) * 512:
        raise ValueError("packed product: the packed weight does not fit these sizes")
    library.call(kernels.lib("gemm_mfma"), "agave_gemm_tiled_as", x.data_ptr(), x.stride(0), packed.data_ptr(),
                 kernels.dt(out), out.data_ptr(), out.stride(0), m, n_out, k, epilogue, tile, kernels.stream())


def tiled_slices_as(x: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, n_out: int, tile: int) -> None:
    """:func:`tiled_slices` with the tile shape and the number of slices (``out.shape[0]``) given."""
    if not (x.is_cuda and packed.is_cuda and out.is_cuda) or not _x_ok(x):
        raise ValueError("packed product: bfloat16 GPU rows, 16-byte aligned, K and the row stride multiples of 8")
    m, k = x.shape
    if out.dtype != torch.float32 or out.dim() != 3 or out.shape[1:] != (m, n_out) or not out.is_contiguous():
        raise ValueError(f"partial sums must be a contiguous float32 [slices, {m}, {n_out}] tensor")
    if packed.numel() != ((n_out + 15) // 16) * ((k + 31) // 32) * 512:
        raise ValueError("packed product: the packed weight does not fit these sizes")
    library.call(kernels.lib("gemm_mfma"), "agave_gemm_tiled_in_slices_as", x.data_ptr(), x.stride(0), packed.data_ptr(),
                 out.data_ptr(), m, n_out, k, tile, out.shape[0], kernels.stream())


def skinny_slices(x: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, n_out: int) -> None:
    """out[s] = the sums over the s-th run of columns of x[M, K] @ W^T; out is float32 [slices, M, n_out]
    and its slices add up to the product (M <= 64)."""
    if not (x.is_cuda and packed.is_cuda and out.is_cuda):
        raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")
    if not _x_ok(x):
        raise ValueError("packed product: input must be 16-byte aligned bfloat16 rows with K and the row stride multiples of 8")
    m, k = x.shape
    if out.dtype != torch.float32 or out.dim() != 3 or out.shape[1:] != (m, n_out) or not out.is_contiguous():
        raise ValueError(f"partial sums must be a contiguous float32 [slices, {m}, {n_out}] tensor")
    if packed.numel() != ((n_out + 15) // 16) * ((k + 31) // 32) * 512:
        raise ValueError("packed product: the packed weight does not fit these sizes")
    library.call(kernels.lib("gemm_mfma"), "agave_gemm_skinny", x.data_ptr(), x.stride(0), packed.data_ptr(),
                 kernels.dt(out), out.data_ptr(), n_out, m, n_out, k, 0, out.shape[0], kernels.stream())


# The tiled kernel shares a product out along its columns only when it has fewer than 160 tiles of
# 64 x 128, and among at most 8 workgroups a tile: the partial sums never need more than this.
PARTS_ELEMS = 8 * 160 * 64 * 128
_parts = {}


def _partial_sums(x: torch.Tensor, epilogue: int):
    """The buffer of 32-bit partial sums that the tiled kernel may use for a product with few tiles
    and many columns.  One per device, of a fixed size, so that its address can be recorded in a
    graph."""
    if epilogue:
        return None
    buf = _parts.get(x.device)
    if buf is None:
        buf = _parts[x.device] = torch.empty(PARTS_ELEMS, dtype=torch.float32, device=x.device)
    return buf


def _launch(fn: str, x: torch.Tensor, packed: torch.Tensor, out: torch.Tensor, n_out: int, epilogue: int) -> None:
    if not (x.is_cuda and packed.is_cuda and out.is_cuda):
        raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")
    m, k = x.shape
    if not _x_ok(x):
        raise ValueError("packed product: x must be bfloat16, 16-byte aligned, K and row stride multiples of 8")
    if out.dim() != 2 or out.shape != (m, n_out) or out.stride(1) != 1:
        raise ValueError(f"packed product: out must be [{m}, {n_out}] with contiguous rows")
    nb = (n_out + 7) // 8 if epilogue else (n_out + 15) // 16
    if packed.numel() != nb * ((k + 31) // 32) * 512:
        raise ValueError("packed product: the packed weight does not fit these sizes")
    if fn == "agave_gemm_tiled":
        part = _partial_sums(x, epilogue)
        library.call(kernels.lib("gemm_mfma"), fn, x.data_ptr(), x.stride(0), packed.data_ptr(),
                     kernels.dt(out), out.data_ptr(), out.stride(0), m, n_out, k, epilogue,
                     kernels.ptr(part), part.numel() if part is not None else 0, kernels.stream())
        return
    library.call(kernels.lib("gemm_mfma"), fn, x.data_ptr(), x.stride(0), packed.data_ptr(),
                 kernels.dt(out), out.data_ptr(), out.stride(0), m, n_out, k, epilogue, 1, kernels.stream())


def try_linear(x: torch.Tensor, lin, out: torch.Tensor) -> bool:
    """Run the product on the matrix cores if a kernel takes these sizes; False otherwise."""
    packed = getattr(lin, "packed", None)
    if packed is None or not _x_ok(x):
        return False
    product(x, packed, out, lin.out_features, 0)
    return True


def partials_runs(m: int, n_heads: int, head_dim: int, splits: int) -> int:
    """How many 32-bit slices :func:`product_of_partials` leaves for these sizes (runs of heads that a
    workgroup takes together); 0 if it does not take them."""
    if splits < 2:
        return 0
    key = ("runs", m, n_heads, head_dim, splits)
    got = _slices.get(key)
    if got is None:
        hps = int(kernels.lib("gemm_mfma").agave_oproj_combine_heads_per_run(m, n_heads, head_dim, splits))
        got = _slices[key] = n_heads // hps if hps > 0 else 0
    return got


def product_of_partials(part_o: torch.Tensor, part_ml: torch.Tensor, packed: torch.Tensor, out: torch.Tensor,
                        n_out: int) -> None:
    """The product of the decode attention's merged output rows with W^T, from the splits' partial
    results: out[r] (float32 [runs, M, n_out]) are slices that add up to it.  part_o is [M, heads,
    splits, head_dim], part_ml [M, heads, splits, 2] (reference in natural logarithms, sum)."""
    if not (part_o.is_cuda and part_ml.is_cuda and packed.is_cuda and out.is_cuda):
        raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")
    if part_o.dim() != 4 or part_o.dtype != torch.float32 or not part_o.is_contiguous():
        raise ValueError("product_of_partials: part_o must be a contiguous float32 [M, heads, splits, head_dim] tensor")
    m, nh, splits, hd = part_o.shape
    if part_ml.shape != (m, nh, splits, 2) or part_ml.dtype != torch.float32 or not part_ml.is_contiguous():
        raise ValueError(f"product_of_partials: part_ml must be a contiguous float32 [{m}, {nh}, {splits}, 2] tensor")
    runs = partials_runs(m, nh, hd, splits)
    if runs == 0:
        raise ValueError(f"product_of_partials: no kernel for {m} tokens, {nh} heads of {hd}, {splits} splits")
    if out.dtype != torch.float32 or out.shape != (runs, m, n_out) or not out.is_contiguous():
        raise ValueError(f"product_of_partials: out must be a contiguous float32 [{runs}, {m}, {n_out}] tensor")
    if packed.dtype != torch.bfloat16 or packed.numel() != ((n_out + 15) // 16) * ((nh * hd + 31) // 32) * 512:
        raise ValueError("product_of_partials: the packed weight does not fit these sizes")
    library.call(kernels.lib("gemm_mfma"), "agave_gemm_oproj_combine", part_o.data_ptr(), part_ml.data_ptr(),
                 packed.data_ptr(), out.data_ptr(), m, n_out, nh, hd, splits, kernels.stream())


def embed_scale_packed(tokens: torch.Tensor, packed: torch.Tensor, scale: float, out: torch.Tensor, vocab: int) -> None:
    """out[t] = table[tokens[t]] * scale, the table being a packed [vocab, hidden] weight."""
    if not (tokens.is_cuda and packed.is_cuda and out.is_cuda):
        raise RuntimeError("agave_amd kernels run on the GPU only; got a CPU tensor")
    n, e = out.shape
    if tokens.dtype != torch.int32 or tokens.numel() != n or out.dtype != torch.float32 or not out.is_contiguous():
        raise TypeError("embed_scale_packed: int32 tokens and a contiguous float32 [tokens, hidden] output")
    if packed.numel() != ((vocab + 15) // 16) * ((e + 31) // 32) * 512:
        raise ValueError("embed_scale_packed: the packed table does not fit these sizes")
    library.call(kernels.lib("gemm_mfma"), "agave_embed_scale_packed", tokens.data_ptr(), packed.data_ptr(), scale,
                 out.data_ptr(), n, e, vocab, kernels.stream())
