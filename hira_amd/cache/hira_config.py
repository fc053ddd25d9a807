"""Settings of the cache and its index (the reference's cache/hira_config.py:5-46, same field
names and defaults apart from the device mode, which is the GPU here), with validation and with
the two loaders the reference leaves unimplemented (``from_dict`` / ``from_yaml``, :27-33).
"""
from __future__ import annotations

import dataclasses
import warnings
from typing import Any, Dict


class DeviceMode:
    """Where index and search run.  Only ``CUDA_ONLY`` is served by this package: PyTorch-ROCm
    names the MI355X "cuda", and the string is what configurations of the reference carry."""

    CPU_ONLY = "cpu_only"
    CUDA_ONLY = "cuda_only"
    CPU_CUDA = "cpu-cuda"
    ALL = (CPU_ONLY, CUDA_ONLY, CPU_CUDA)


_THRESHOLD_METHODS = ("sample_max", "sample_mean_topk", "exact_topk", "none")
# sections a configuration file may group its settings under
_SECTIONS = {"indexing": ("num_levels", "max_iterations", "branching_factor"),
             "thresholds": ("threshold_method", "sample_size", "threshold_topk")}


@dataclasses.dataclass
class HiraConfig:
    device_mode: str = DeviceMode.CUDA_ONLY   # cache: which backend a layer's index lives on
    update_every: int = 1                     # cache: queued tokens that trigger an index update
    num_levels: int = 5                       # index: levels of the tree, keys included
    max_iterations: int = 1                   # index: Lloyd rounds per level at build
    branching_factor: int = 10                # index: children per node
    threshold_method: str = "sample_mean_topk"  # thresholds: one of _THRESHOLD_METHODS
    sample_size: int = 1000                   # thresholds: keys sampled per KV head
    threshold_topk: int = 10                  # thresholds: k of "sample_mean_topk" (not in the
    #                                           reference, whose stub takes k at the call)
    chunk_size = 8 * 1024                     # host searcher only (a class attribute, as in the
    #                                           reference: not a dataclass field)

    def __post_init__(self):
        if self.device_mode not in DeviceMode.ALL:
            raise ValueError(f"device_mode {self.device_mode!r}: one of {DeviceMode.ALL}")
        for name in ("update_every", "num_levels", "branching_factor", "sample_size",
                     "threshold_topk"):
            if int(getattr(self, name)) < 1:
                raise ValueError(f"{name} must be at least 1, got {getattr(self, name)}")
        if int(self.max_iterations) < 0:
            raise ValueError(f"max_iterations must not be negative, got {self.max_iterations}")
        if self.threshold_method not in _THRESHOLD_METHODS:
            raise ValueError(f"threshold_method {self.threshold_method!r}: one of {_THRESHOLD_METHODS}")

    # ------------------------------------------------------------------ loaders
    @classmethod
    def from_dict(cls, config_dict: Dict[str, Any]) -> "HiraConfig":
        """Settings from a mapping: the field names flat, or grouped the way the reference's
        sample file groups them (examples/configs/1_example_config.yml:1-8: the index's three
        settings under ``indexing:``; likewise ``thresholds:``).  ``cuda_memory_limit`` (the
        sample file's budget for the reference's unbuilt "cpu-cuda" mode, which nothing reads
        there either) is accepted and ignored with a warning.  Any other unknown key, a key in
        the wrong section or a key given twice is a ``ValueError``."""
        names = {f.name for f in dataclasses.fields(cls)}
        flat: Dict[str, Any] = {}

        def take(key, value, where):
            if key not in names and key != "chunk_size":
                raise ValueError(f"unknown HiraConfig key {where}{key!r}")
            if key in flat:
                raise ValueError(f"HiraConfig key {key!r} is given twice")
            flat[key] = value

        for key, value in config_dict.items():
            if key in _SECTIONS:
                if not isinstance(value, dict):
                    raise ValueError(f"section {key!r} must be a mapping, got {type(value).__name__}")
                for sub, sub_value in value.items():
                    if sub not in _SECTIONS[key]:
                        raise ValueError(f"{sub!r} is not a setting of section {key!r} "
                                         f"(which holds {_SECTIONS[key]})")
                    take(sub, sub_value, f"{key}.")
            elif key == "cuda_memory_limit":
                warnings.warn("HiraConfig: 'cuda_memory_limit' only concerns a mixed host/GPU "
                              "mode that does not exist here; ignored", stacklevel=2)
            else:
                take(key, value, "")
        chunk_size = flat.pop("chunk_size", None)
        cfg = cls(**flat)
        if chunk_size is not None:
            cfg.chunk_size = int(chunk_size)
        return cfg

    @classmethod
    def from_yaml(cls, config_path: str) -> "HiraConfig":
        import yaml

        with open(config_path, "r", encoding="utf-8") as handle:
            return cls.from_dict(yaml.safe_load(handle) or {})

    # ------------------------------------------------------------------ what each part is built from
    def get_indexer_kwargs(self) -> Dict[str, int]:
        return {name: int(getattr(self, name))
                for name in ("num_levels", "max_iterations", "branching_factor")}

    def get_searcher_kwargs(self) -> Dict[str, int]:
        on_gpu = self.device_mode == DeviceMode.CUDA_ONLY
        return {"block_c": self.branching_factor} if on_gpu else {"chunk_size": self.chunk_size}

    def get_threshold_kwargs(self) -> Dict[str, Any]:
        """What the cache layer needs to keep a key sample and turn it into thresholds."""
        return {"method": self.threshold_method, "sample_size": int(self.sample_size),
                "topk": int(self.threshold_topk)}
