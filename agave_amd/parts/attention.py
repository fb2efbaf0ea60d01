"""Attention as a mixer: grouped-query attention over the paged cache, with optional per-head
q/k norm, a position encoding, and an optional sliding window.

Order of operations as the reference (``src/models/gemma3.zig:701-828``): q, k, v projections;
RMSNorm of every q and k head with one gain vector per tensor, before the rotation
(``:722-729``); rotation (``:732-749``); k and v appended to the cache, then attention over it
with ``scale`` on the scores (``:795-813``); output projection (``:819-820``).  A query at
position p sees keys ``max(0, p-W+1) .. p`` on a windowed layer, ``0 .. p`` otherwise.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import AttentionSpec
from ..ops import attention as attn_ops
from ..ops import kernels
from ..weights.loader import TensorNeed
from .base import BuildEnv, lookup, register
from .linear import Linear


class Attention:
    prompt_steps_can_be_recorded = True        # a multi-token step is the same launches whatever its tokens are
    takes_rows_to_be_normed = True             # its first product may make the normalised rows itself (NormedRows)

    def __init__(self, spec: AttentionSpec, weights, env: BuildEnv):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        self.spec = spec
        self.env = env
        self.qd = spec.n_heads * spec.head_dim
        self.kvd = spec.n_kv_heads * spec.head_dim
        self._qkv_bounds = (0, self.qd, self.qd + self.kvd, self.qd + 2 * self.kvd)
        def bias(name):
            return weights.get(name) if name else None

        # q, k and v in one product: rows of the three matrices stacked
        self.qkv = Linear([weights.get(spec.q_proj), weights.get(spec.k_proj), weights.get(spec.v_proj)], env, "qkv",
                          biases=[bias(spec.q_bias), bias(spec.k_bias), bias(spec.v_bias)])
        self.o = Linear([weights.get(spec.o_proj)], env, "attn_o", biases=[bias(spec.o_bias)])
        self.q_norm = lookup("norm", spec.q_norm.kind)(spec.q_norm, weights, env) if spec.q_norm else None
        self.k_norm = lookup("norm", spec.k_norm.kind)(spec.k_norm, weights, env) if spec.k_norm else None
        self.position = lookup("position", spec.position.kind)(spec.position, env)
        # the per-head norms are computed inside the q/k kernel, which knows the RMS kind (a gain and an eps)
        for name, part in (("q_norm", self.q_norm), ("k_norm", self.k_norm)):
            if part is not None and not (hasattr(part, "gain") and hasattr(part, "eps")):
                raise ValueError(f"attention: {name} of kind {getattr(spec, name).kind!r} has no gain and eps; the q/k "
                                 f"kernel computes the per-head norm itself and takes those of an RMS norm")

    @staticmethod
    def tensor_needs(spec: AttentionSpec) -> List[TensorNeed]:
        qd, kvd = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim
        needs = [TensorNeed(spec.q_proj, (qd, spec.hidden)), TensorNeed(spec.k_proj, (kvd, spec.hidden)),
                 TensorNeed(spec.v_proj, (kvd, spec.hidden)), TensorNeed(spec.o_proj, (spec.hidden, qd))]
        for name, size in ((spec.q_bias, qd), (spec.k_bias, kvd), (spec.v_bias, kvd), (spec.o_bias, spec.hidden)):
            if name:
                needs.append(TensorNeed(name, (size,)))
        for n in (spec.q_norm, spec.k_norm):
            if n is not None:
                needs += lookup("norm", n.kind).tensor_needs(n)
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        return GroupKey(self.spec.window, self.spec.n_kv_heads, self.spec.head_dim)

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        s, ws = self.spec, self.env.workspace
        n = x.shape[0]
        k_pages, v_pages, packed = step.cache.pages_of(memory)
        table, base = step.tables[step.cache.group_of_memory[memory]]
        fused = getattr(self.position, "fused_rotation", None)
        qkv = self.qkv.forward(x, tag="qkv")
        q, k, v = ws.columns(qkv, self._qkv_bounds)
        if not writes:
            k = v = None            # a run that reads another run's cache appends nothing
        q_out = ws.get("q_rot", n, self.qd, x.dtype)
        qg, kg = (self.q_norm.gain if self.q_norm else None), (self.k_norm.gain if self.k_norm else None)
        qe, ke = (self.q_norm.eps if self.q_norm else 0.0), (self.k_norm.eps if self.k_norm else 0.0)
        ctx_out = ws.get("attn_ctx", n, self.qd, x.dtype)
        if fused is not None:
            inv_freq, pos_scale = fused()
            # a decode step whose keys are shared among workgroups leaves partial results, which the
            # output product merges itself if it can (one kernel less a layer)
            partials_ok = (lambda splits: self.o.takes_partials(n, s.n_heads, s.head_dim, splits)) if step.is_decode else None
            parts = attn_ops.qk_attention(q, k, v, q_out, ctx_out, qg, kg, qe, ke, inv_freq, pos_scale, k_pages, v_pages,
                                          table, base, step, s.n_heads, s.n_kv_heads, s.head_dim, s.scale, s.window,
                                          packed, partials_ok=partials_ok)
            if parts is not None:
                return self.o.forward_partials(parts[0], parts[1], tag="attn_o")
            return self.o.forward(ctx_out, tag="attn_o", slices_ok=True)       # the block adds it to the residual stream
        else:
            # a position encoding the q/k kernel does not know: the norms, then the part's own
            # ``apply`` on the normalised rows, then the cache write
            kernels.qk_norm_rope_kv(q, None, None, q_out, qg, None, qe, 0.0, None, 1.0, step.tok_seq, step.tok_pos,
                                    None, None, None, None, s.n_heads, 0, s.head_dim)
            k_n = None
            if k is not None:
                k_n = ws.get("k_normed", n, self.kvd, x.dtype)
                kernels.qk_norm_rope_kv(k, None, None, k_n, kg, None, ke, 0.0, None, 1.0, step.tok_seq, step.tok_pos,
                                        None, None, None, None, s.n_kv_heads, 0, s.head_dim)
            self.position.apply(q_out, k_n, step)
            if k is not None:
                kernels.qk_norm_rope_kv(None, k_n, v, None, None, None, 0.0, 0.0, None, 1.0, step.tok_seq,
                                        step.tok_pos, k_pages, v_pages, table, base, 0, s.n_kv_heads, s.head_dim,
                                        packed)
        attn_ops.attention(q_out, ctx_out, k_pages, v_pages, table, base, step, s.n_heads, s.n_kv_heads,
                           s.head_dim, s.scale, s.window, packed)
        return self.o.forward(ctx_out, tag="attn_o", slices_ok=True)       # the block adds it to the residual stream


register("mixer", "attention", Attention)
