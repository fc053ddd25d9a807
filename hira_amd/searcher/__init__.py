from .base import BaseSearcher
from .hip import DecodePlan, HIPSearcher, StreamingStep

CUDASearcher = HIPSearcher  # searcher/__init__.py:1-10 of the reference

__all__ = ["BaseSearcher", "HIPSearcher", "CUDASearcher", "DecodePlan", "StreamingStep"]
