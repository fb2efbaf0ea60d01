"""Sampling options and results; the kernels are in ``agave_amd.ops.sampling``."""
from .params import GenerationResult, SamplingParams

__all__ = ["SamplingParams", "GenerationResult"]
