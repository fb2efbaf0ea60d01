"""Faces of the sampling kernels."""
from __future__ import annotations

import ctypes

import torch

from . import kernels, library
from .kernels import _I, _L, _P

kernels.register_signatures("sampling", {
    "agave_sample": [_P, _L, _P, _L, _P, _P, _I, _I, _P, _I, _P],
    "agave_repeat_penalty": [_P, _L, _P, _P, _P, _I, _I, _P],
    "agave_gather_tokens": [_P, _P, _P, _I, _I, _P],
    "agave_token_logprob": [_P, _L, _P, _P, _I, _I, _P],
})


def _logits(logits: torch.Tensor) -> int:
    if not logits.is_cuda:
        raise RuntimeError("sampling runs on the GPU only; got CPU logits")
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise TypeError("logits must be float32 [rows, vocab] with contiguous rows")
    return logits.stride(0)


KIND_TEMPERATURE = 1     # some row draws with a temperature
KIND_FILTER = 2          # some row has top-k or top-p
KIND_ALL = 3


def scratch_words() -> int:
    """float32 words of scratch per row that let rows of a large vocabulary be shared among workgroups."""
    lib = kernels.lib("sampling")
    lib.agave_sample_scratch_words.restype = ctypes.c_int
    lib.agave_sample_scratch_words.argtypes = []
    return int(lib.agave_sample_scratch_words())


def kinds_of(rows, vocab: int) -> int:
    """What a batch's rows (objects with temperature, top_k, top_p) need of the sampler."""
    kinds = 0
    for r in rows:
        if r.temperature > 0:
            kinds |= KIND_TEMPERATURE
            if 0 < min(r.top_k, 1 << 20) < vocab or 0.0 < r.top_p < 1.0:     # (top_k travels capped at 2^20)
                kinds |= KIND_FILTER
    return kinds


def sample(logits: torch.Tensor, work: torch.Tensor, params: torch.Tensor, out: torch.Tensor,
           scratch: torch.Tensor = None, kinds: int = KIND_ALL) -> None:
    """out[b] = a token drawn from row b.  ``params`` float32 [rows, 4] = temperature, top_k,
    top_p, u; temperature 0 takes the argmax (first index on ties).  ``work``: float32 scratch
    of the logits' shape.  ``scratch`` (``scratch_words()`` float32 per row) lets rows of a large
    vocabulary be shared among 64 workgroups each; ``kinds`` then says what the rows need
    (``kinds_of``), so that kernels no row needs are not launched."""
    ld = _logits(logits)
    b, v = logits.shape
    if work.dtype != torch.float32 or work.shape != logits.shape or work.stride(1) != 1 or not work.is_cuda:
        raise TypeError("sample: work must be a float32 GPU tensor of the logits' shape")
    if params.dtype != torch.float32 or params.shape != (b, 4) or not params.is_contiguous() or not params.is_cuda:
        raise TypeError(f"sample: params must be contiguous float32 [{b}, 4] on the GPU")
    if out.dtype != torch.int32 or out.numel() != b or not out.is_contiguous() or not out.is_cuda:
        raise TypeError(f"sample: out must be {b} contiguous int32 on the GPU")
    if scratch is not None:
        need = scratch_words() * b
        if (scratch.dtype != torch.float32 or scratch.numel() < need or not scratch.is_cuda
                or not scratch.is_contiguous() or scratch.data_ptr() % 16 != 0):
            raise TypeError(f"sample: scratch must be {need} contiguous float32 on the GPU, 16-byte aligned")
    if kinds not in (0, 1, 2, 3):
        raise ValueError("sample: kinds is a mask of KIND_TEMPERATURE and KIND_FILTER")
    library.call(kernels.lib("sampling"), "agave_sample", logits.data_ptr(), ld, work.data_ptr(), work.stride(0),
                 params.data_ptr(), out.data_ptr(), b, v, kernels.ptr(scratch), int(kinds), kernels.stream())


def repeat_penalty(logits: torch.Tensor, ids: torch.Tensor, cu: torch.Tensor, penalty: torch.Tensor) -> None:
    """In place: for every id in ids[cu[b]:cu[b+1]], once per occurrence, row b's logit is divided
    by penalty[b] if positive, else multiplied."""
    ld = _logits(logits)
    b, v = logits.shape
    for t, n, what in ((ids, 0, "ids"), (cu, b + 1, "cu")):
        if t.dtype != torch.int32 or not t.is_contiguous() or not t.is_cuda or t.numel() < n:
            raise TypeError(f"repeat_penalty: {what} must be contiguous int32 on the GPU")
    if penalty.dtype != torch.float32 or penalty.numel() != b or not penalty.is_cuda:
        raise TypeError(f"repeat_penalty: penalty must be {b} float32 on the GPU")
    library.call(kernels.lib("sampling"), "agave_repeat_penalty", logits.data_ptr(), ld, ids.data_ptr(),
                 cu.data_ptr(), penalty.data_ptr(), b, v, kernels.stream())


def gather_tokens(src: torch.Tensor, index: torch.Tensor, dst: torch.Tensor) -> None:
    """dst[i] = src[index[i]] (int32, on the GPU): what a step sampled becomes the next step's tokens."""
    for t, what in ((src, "src"), (index, "index"), (dst, "dst")):
        if t.dtype != torch.int32 or not t.is_contiguous() or not t.is_cuda:
            raise TypeError(f"gather_tokens: {what} must be contiguous int32 on the GPU")
    if index.numel() != dst.numel():
        raise ValueError("gather_tokens: one index per destination")
    library.call(kernels.lib("sampling"), "agave_gather_tokens", src.data_ptr(), index.data_ptr(), dst.data_ptr(),
                 dst.numel(), src.numel(), kernels.stream())


def token_logprob(logits: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> None:
    """out[b] = log softmax(logits[b])[tokens[b]] (natural logarithm, float32)."""
    ld = _logits(logits)
    b, v = logits.shape
    if tokens.dtype != torch.int32 or tokens.numel() != b or not tokens.is_contiguous() or not tokens.is_cuda:
        raise TypeError(f"token_logprob: tokens must be {b} contiguous int32 on the GPU")
    if out.dtype != torch.float32 or out.numel() != b or not out.is_contiguous() or not out.is_cuda:
        raise TypeError(f"token_logprob: out must be {b} contiguous float32 on the GPU")
    library.call(kernels.lib("sampling"), "agave_token_logprob", logits.data_ptr(), ld, tokens.data_ptr(),
                 out.data_ptr(), b, v, kernels.stream())
