"""Model, step function, engine and generation."""
from .engine import Engine, parse_dtype, require_gpu
from .model import Model, tensor_needs
from .step import Step, StepError, StepPlanner

__all__ = ["Engine", "Model", "Step", "StepError", "StepPlanner", "tensor_needs", "parse_dtype", "require_gpu"]
