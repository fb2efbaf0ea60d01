"""A linear map y = W x with W stored row-major [out, in] (``src/backend/backend.zig:474, 481``).

The weight's element type is the build environment's choice (``BuildEnv.weight_dtype``): a
32-bit engine widens everything (exactly); a bfloat16 engine keeps bfloat16, casts half
precision to bfloat16, and keeps a matrix that was stored in 32-bit as it is unless told to cast
it.  The kernel is chosen by the types: 32-bit anything goes through the plain multiply-add
kernel; bfloat16 activations with bfloat16 weights go through the matrix-core kernels, which
fall back to the plain kernel for shapes they refuse.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..ops import gemm, gemm_mfma, kernels, library
from .base import BuildEnv
from .norm import NormedRows


class Linear:
    def __init__(self, weights: Sequence[torch.Tensor], env: BuildEnv, name: str = "linear", pack: bool = True,
                 interleave_ff: int = 0, biases: Optional[Sequence[Optional[torch.Tensor]]] = None):
        """``weights``: one or more [out_i, in] matrices that are stacked along ``out``.
        ``interleave_ff``: the stack is [gate; up] of that many rows each; if the weight is packed
        its rows are interleaved for the product that ends in GeGLU (see ``forward_geglu``).
        ``biases``: one vector [out_i] or None per matrix; y = W x + b then (the sum is made in
        32-bit by a kernel of its own after the product: a model without biases pays nothing)."""
        ws = []
        for w in weights:
            if w.dim() != 2:
                raise ValueError(f"{name}: weight must be a matrix, got {tuple(w.shape)}")
            keep = env.weight_dtype(w.dtype)
            if w.dtype != keep:
                w = w.to(keep)
            ws.append(w)
        if len({w.shape[1] for w in ws}) != 1:
            raise ValueError(f"{name}: stacked weights must agree in input size")
        if len({w.dtype for w in ws}) != 1:
            # a stack of matrices stored in different widths is held in 32-bit (what is stored in
            # 32-bit stays so; widening the others loses nothing)
            ws = [w.to(torch.float32) for w in ws]
        dev = [w.to(env.device) for w in ws]
        self.weight = dev[0].contiguous() if len(dev) == 1 else torch.cat(dev, dim=0).contiguous()
        self.out_features, self.in_features = self.weight.shape
        self.env = env
        self.name = name
        self.packed = None          # the weight in the matrix cores' tile layout (bfloat16 engines)
        if pack and env.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and self.in_features % 8 == 0:
            self.packed = gemm_mfma.pack_weight(self.weight, interleave_ff=interleave_ff)
            self.weight = None      # only the packed copy is kept
        elif env.dtype == torch.bfloat16 and self.weight.dtype == torch.float32:
            env.kept_32bit.append(name)
        self.interleave_ff = interleave_ff if self.packed is not None else 0
        self.bias: Optional[torch.Tensor] = None
        if biases is not None and any(b is not None for b in biases):
            if len(biases) != len(ws):
                raise ValueError(f"{name}: {len(biases)} biases for {len(ws)} matrices")
            if interleave_ff:
                raise ValueError(f"{name}: a product that ends in GeGLU takes no bias")
            pieces = []
            for w, b in zip(ws, biases):
                if b is None:
                    b = torch.zeros(w.shape[0])
                if tuple(b.shape) != (w.shape[0],):
                    raise ValueError(f"{name}: a bias of shape {tuple(b.shape)} for a matrix of {w.shape[0]} rows")
                pieces.append(b.to(device=env.device, dtype=torch.float32))
            self.bias = torch.cat(pieces).contiguous()

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, tag: Optional[str] = None,
                slices_ok: bool = False) -> torch.Tensor:
        """``slices_ok``: the caller also takes a float32 [slices, n, out] tensor whose slices add
        up to the product (a norm that adds a branch to the residual stream does); a product
        with few rows of W and many columns is then shared out along the columns."""
        if isinstance(x, NormedRows):
            plain = not self.interleave_ff and out_dtype in (None, torch.bfloat16)
            made = self._forward_normed(x, out, tag, 0) if plain else None
            if made is not None:
                return made
            x = x.rows()
        n = x.shape[0]
        if slices_ok and out is None and self.packed is not None and not self.interleave_ff:
            many = n > gemm_mfma.SKINNY_MAX_M
            slices = (gemm_mfma.tiled_slices_for if many else gemm_mfma.slices_for)(n, self.out_features, self.in_features)
            if slices > 1 and gemm_mfma._x_ok(x):
                out = self.env.workspace.get3((tag or self.name) + "_slices", slices, n, self.out_features, torch.float32)
                library.profile.label = self.name
                (gemm_mfma.tiled_slices if many else gemm_mfma.skinny_slices)(x, self.packed, out, self.out_features)
                if self.bias is not None:
                    kernels.add_bias(out[0], self.bias)
                library.profile.label = None
                return out
        if out is None:
            out = self.env.workspace.get(tag or self.name, n, self.out_features, out_dtype or x.dtype)
        if self.interleave_ff:
            raise RuntimeError(f"{self.name}: a weight packed for GeGLU only serves forward_geglu")
        library.profile.label = self.name
        gemm.linear(x, self, out)
        if self.bias is not None:
            kernels.add_bias(out, self.bias)
        library.profile.label = None
        return out

    def takes_partials(self, n: int, n_heads: int, head_dim: int, splits: int) -> bool:
        """Whether :meth:`forward_partials` can take the decode attention's partial results for
        ``n`` tokens in ``splits`` splits (the kernel library has the last word on the sizes)."""
        if self.packed is None or self.interleave_ff or self.in_features != n_heads * head_dim:
            return False
        return gemm_mfma.partials_runs(n, n_heads, head_dim, splits) > 0

    def forward_partials(self, part_o: torch.Tensor, part_ml: torch.Tensor, tag: Optional[str] = None) -> torch.Tensor:
        """The product of the attention rows that the splits' partial results stand for: they are
        merged inside the product's kernel.  Returns float32 slices [runs, n, out] that add up."""
        n, nh, splits, hd = part_o.shape
        runs = gemm_mfma.partials_runs(n, nh, hd, splits)
        out = self.env.workspace.get3((tag or self.name) + "_runs", runs, n, self.out_features, torch.float32)
        library.profile.label = self.name
        gemm_mfma.product_of_partials(part_o, part_ml, self.packed, out, self.out_features)
        if self.bias is not None:
            kernels.add_bias(out[0], self.bias)
        library.profile.label = None
        return out

    def _forward_normed(self, x: NormedRows, out: Optional[torch.Tensor], tag: Optional[str], epilogue: int):
        """The product of rows that are still a promise, made inside the product's kernel if the
        kernel library has one for these sizes and both norms are RMS norms; None otherwise."""
        n, k = x.shape
        n_out = self.interleave_ff if epilogue else self.out_features
        if self.packed is None or x.dtype != torch.bfloat16 or k != self.in_features or (out is not None and out.dtype != torch.bfloat16):
            return None
        if not gemm_mfma.normed_ok(n, n_out, k, epilogue):
            return None
        args = x.rms_arguments()
        if args is None:
            return None
        h_in, h_out, branch, post_gain, post_eps, pre_gain, pre_eps = args
        if out is None:
            out = self.env.workspace.get(tag or self.name, n, n_out, torch.bfloat16)
        library.profile.label = self.name
        gemm_mfma.row_normed(h_in, h_out, branch, post_gain, post_eps, pre_gain, pre_eps, self.packed, out, n_out, epilogue)
        x.made_by_consumer(h_in, h_out)
        if self.bias is not None:
            kernels.add_bias(out, self.bias)
        library.profile.label = None
        return out

    def forward_geglu(self, x, out: torch.Tensor) -> bool:
        """out = gelu_tanh(gate x) * (up x) in one kernel, if the weight was packed for it."""
        if not self.interleave_ff:
            return False
        if isinstance(x, NormedRows):
            if self._forward_normed(x, out, None, 1) is not None:
                return True
            x = x.rows()
        library.profile.label = self.name
        gemm_mfma.product(x, self.packed, out, self.interleave_ff, epilogue=1)
        library.profile.label = None
        return True
