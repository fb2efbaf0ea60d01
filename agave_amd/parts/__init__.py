"""The parts a layer is put together from, and their registries."""
from .base import BuildEnv, Workspace, lookup, part_tensors, register, registered
from . import norm, position, attention, ffn, block  # noqa: F401  (registers the built-in kinds)
from .attention import Attention
from .block import PreNormBlock, SandwichBlock, add_pending_and_norm
from .ffn import GatedFfn
from .linear import Linear
from .norm import Norm, NormedRows, RmsNorm, add_branch
from .position import NoPosition, RotaryPosition

__all__ = ["BuildEnv", "Workspace", "lookup", "part_tensors", "register", "registered", "Attention", "GatedFfn",
           "Linear", "Norm", "NormedRows", "RmsNorm", "add_branch", "RotaryPosition", "NoPosition", "SandwichBlock", "PreNormBlock",
           "add_pending_and_norm"]
