"""Searchers of this path.

``HIPSearcher`` is the MI355X searcher; ``CUDASearcher`` is the name the reference's callers
import (searcher/__init__.py:1-10; PyTorch-ROCm calls the device "cuda").  ``DecodePlan`` and
``StreamingStep`` are the low-overhead ways to run decode steps: a plan resolved once per
index, and a whole token step captured as one HIP graph.
"""
from .base import BaseSearcher
from .hip import DecodePlan, HIPSearcher, StreamingStep

CUDASearcher = HIPSearcher

__all__ = ["BaseSearcher", "HIPSearcher", "CUDASearcher", "DecodePlan", "StreamingStep"]
