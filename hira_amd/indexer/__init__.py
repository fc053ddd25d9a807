from .base import BaseIndexer
from .hip import HIPIndexer

# the name the reference's callers import (indexer/__init__.py:1-9); on ROCm the device
# PyTorch calls "cuda" is the MI355X
CUDAIndexer = HIPIndexer

__all__ = ["BaseIndexer", "HIPIndexer", "CUDAIndexer"]
