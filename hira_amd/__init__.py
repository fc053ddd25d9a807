"""hira_amd: the HIRA range-search sparse-attention hot path on MI355X (gfx950).

Mirrors the reference's module layout for this path (indexer / searcher / cache /
attention); the kernels live in csrc/ behind the C ABI declared in include/hira_hip.h.
"""
__version__ = "0.1.0"
__all__ = []
