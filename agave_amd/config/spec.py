"""Architecture-neutral description of a decoder: what the engine builds from.

An architecture's typed configuration (for instance :class:`Gemma3Config`) turns
itself into a :class:`ModelSpec`: a list of layers, each naming its mixer, its
feed-forward, its norms and its position encoding *by kind* with their sizes and
constants as plain data, plus the order in which the layers run.  The engine
looks every ``kind`` up in the part registries (``agave_amd.parts``); no part
knows which model it is in, and no size lives anywhere but here.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """A normalisation over the last axis.  ``weight`` is the tensor's full name."""
    kind: str                      # "rmsnorm"
    size: int
    eps: float
    weight: str
    add_one: bool = False          # gain = 1 + w instead of w


@dataclass(frozen=True)
class PositionSpec:
    """A position encoding applied to queries and keys inside a mixer."""
    kind: str                      # "rope" | "none"
    rotary_dim: int = 0
    theta: float = 0.0
    factor: float = 1.0            # linear scaling: positions are divided by it


@dataclass(frozen=True)
class MixerSpec:
    """Base of the token mixers.  ``kind`` selects the implementation."""
    kind: str


@dataclass(frozen=True)
class AttentionSpec(MixerSpec):
    hidden: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0             # multiplies q.k
    window: Optional[int] = None   # None: all earlier keys; W: keys p-W+1 .. p
    position: PositionSpec = PositionSpec("none")
    q_norm: Optional[NormSpec] = None
    k_norm: Optional[NormSpec] = None
    q_proj: str = ""
    k_proj: str = ""
    v_proj: str = ""
    o_proj: str = ""
    q_bias: str = ""               # names of the projections' bias vectors; "": none
    k_bias: str = ""
    v_bias: str = ""
    o_bias: str = ""


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str


@dataclass(frozen=True)
class GatedFfnSpec(FeedForwardSpec):
    hidden: int = 0
    intermediate: int = 0
    activation: str = "gelu_tanh"
    gate_proj: str = ""
    up_proj: str = ""
    down_proj: str = ""
    gate_bias: str = ""            # names of the products' bias vectors; "": none
    up_bias: str = ""
    down_bias: str = ""


@dataclass(frozen=True)
class LayerSpec:
    """One block.  ``kind`` selects the arrangement of the parts:

    ``"sandwich"``: h += post_mixer_norm(mixer(pre_mixer_norm(h)));
                    h += post_ffn_norm(ffn(pre_ffn_norm(h)))
    ``"prenorm"``:  the same without the two post norms.
    """
    kind: str
    mixer: MixerSpec
    ffn: Optional[FeedForwardSpec]
    pre_mixer_norm: Optional[NormSpec] = None
    post_mixer_norm: Optional[NormSpec] = None
    pre_ffn_norm: Optional[NormSpec] = None
    post_ffn_norm: Optional[NormSpec] = None


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers``;
    ``memory`` names the cache (and fixed-size state) this run of the layer uses;
    two entries with the same ``memory`` share it, and only entries with
    ``writes`` append to it."""
    layer: int
    memory: int
    writes: bool = True


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    embed_weight: str
    embed_scale: float
    layers: List[LayerSpec]
    order: List[RunEntry]
    final_norm: Optional[NormSpec]
    head_weight: Optional[str]           # None: tied to the embedding
    max_context: int
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()
    # Name prefixes of the tensors that are this model's own.  A checkpoint's tensor that no
    # part asked for is an error under one of them and is passed over elsewhere (a vision
    # tower beside a text decoder).  None: every name in the checkpoint is the model's.
    tensor_scope: Optional[Tuple[str, ...]] = None
    # what is done to the logits after the output product: multiplied by ``logit_scale``, then
    # soft-capped to +-``logit_softcap`` (cap * tanh(x / cap)) if that is above zero
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    extra: Dict[str, object] = field(default_factory=dict)

    def default_order(self) -> List[RunEntry]:
        return [RunEntry(i, i, True) for i in range(len(self.layers))]
