"""Indexers of this path.

``HIPIndexer`` builds and grows the ball trees on the MI355X; ``CUDAIndexer`` is the name the
reference's callers import (indexer/__init__.py:1-9; PyTorch-ROCm calls the device "cuda").
"""
from .base import BaseIndexer
from .hip import HIPIndexer

CUDAIndexer = HIPIndexer

__all__ = ["BaseIndexer", "HIPIndexer", "CUDAIndexer"]
