"""The model: embedding, the layers in their run order, final norm, output matrix.

It is built from a :class:`ModelSpec` alone, out of registered parts; the same class serves
every architecture.  Reference for the overall order: embedding scaled by ``embed_scale``
(``src/models/gemma3.zig:338, 1017-1046``), ``for i in 0..L: attention(i); feedForward(i)``
(``:341-348``), final norm and output product on the rows whose logits are wanted
(``:352-359``), the output matrix being the embedding table when none is stored (``:357-358``).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import ModelSpec
from ..ops import gemm_mfma, kernels
from ..parts import BuildEnv, Linear, add_pending_and_norm, lookup, part_tensors
from ..weights.loader import TensorNeed


def tensor_needs(spec: ModelSpec) -> List[TensorNeed]:
    """Every tensor the model reads, in a fixed order (embedding, layers, final norm, head)."""
    needs = [TensorNeed(spec.embed_weight, (spec.vocab_size, spec.hidden))]
    for layer in spec.layers:
        needs += lookup("block", layer.kind).tensor_needs(layer)
    if spec.final_norm is not None:
        needs += lookup("norm", spec.final_norm.kind).tensor_needs(spec.final_norm)
    if spec.head_weight is not None:
        needs.append(TensorNeed(spec.head_weight, (spec.vocab_size, spec.hidden)))
    return needs


class Model:
    def __init__(self, spec: ModelSpec, weights, env: BuildEnv):
        self.spec = spec
        self.env = env
        table = weights.get(spec.embed_weight)
        keep = env.weight_dtype(table.dtype)
        if table.dtype != keep:
            table = table.to(keep)
        self.embed_table: Optional[torch.Tensor] = table.to(env.device).contiguous()
        self.blocks = [lookup("block", layer.kind)(layer, weights, env) for layer in spec.layers]
        self.final_norm = (lookup("norm", spec.final_norm.kind)(spec.final_norm, weights, env)
                           if spec.final_norm is not None else None)
        if spec.head_weight is not None:
            self.head = Linear([weights.get(spec.head_weight)], env, "lm_head")
        else:
            self.head = Linear([self.embed_table], env, "lm_head")      # tied: the same device tensor
            if self.head.packed is not None:
                self.embed_table = None                                  # rows are gathered from the packed copy
        for entry in spec.order:
            if not (0 <= entry.layer < len(self.blocks)):
                raise ValueError(f"run order names layer {entry.layer}, the model has {len(self.blocks)}")
        writers = {e.memory for e in spec.order if e.writes}
        for e in spec.order:
            if not e.writes and e.memory not in writers:
                raise ValueError(f"run order: memory {e.memory} is read but never written")

    # ------------------------------------------------------------------ what the cache must hold
    def kv_needs(self) -> Dict[int, GroupKey]:
        needs: Dict[int, GroupKey] = {}
        for e in self.spec.order:
            need = self.blocks[e.layer].mixer.kv_need()
            if need is None:
                continue
            if e.memory in needs and needs[e.memory] != need:
                raise ValueError(f"memory {e.memory} is shared by mixers with different needs: "
                                 f"{needs[e.memory]} and {need}")
            needs[e.memory] = need
        return needs

    def state_needs(self) -> Dict[int, StateNeed]:
        needs: Dict[int, StateNeed] = {}
        for e in self.spec.order:
            need = self.blocks[e.layer].mixer.state_need()
            if need is None:
                continue
            if e.memory in needs and needs[e.memory] != need:
                raise ValueError(f"memory {e.memory} is shared by mixers with different state")
            needs[e.memory] = need
        return needs

    def weight_bytes(self) -> int:
        """Bytes of all weights on the device, shared tensors counted once."""
        parts = [self.embed_table, self.blocks, self.final_norm, self.head]
        return sum(t.numel() * t.element_size() for t in part_tensors(parts))

    # ------------------------------------------------------------------ one step
    def forward(self, step) -> Optional[torch.Tensor]:
        """Run the step's tokens through the model; float32 logits [wanted, vocab] or None."""
        ws = self.env.workspace
        n = step.n_tokens
        h = ws.get("residual", n, self.spec.hidden, torch.float32)
        if self.embed_table is not None:
            kernels.embed_scale(step.tokens, self.embed_table, self.spec.embed_scale, h)
        else:
            gemm_mfma.embed_scale_packed(step.tokens, self.head.packed, self.spec.embed_scale, h, self.spec.vocab_size)
        pending = None
        for entry in self.spec.order:
            pending = self.blocks[entry.layer].forward(h, pending, step, entry.memory, entry.writes)
        if step.n_want == 0:
            return None
        x = ws.get("final_normed", step.n_want, self.spec.hidden, self.env.dtype)
        # (a decode step wants every row, in order: no gather, and the last branch is added in the norm's kernel)
        rows = None if (step.is_decode and step.n_want == n) else step.want_rows
        add_pending_and_norm(h, pending, self.final_norm, x, rows=rows)   # no final norm: the rows as they are
        logits = ws.get("logits", step.n_want, self.spec.vocab_size, torch.float32)
        self.head.forward(x, out=logits)
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap > 0.0:
            kernels.scale_cap(logits, self.spec.logit_scale, self.spec.logit_softcap)
        return logits
