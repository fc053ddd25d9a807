"""HiraConfig / DeviceMode: the reference's cache/hira_config.py:5-46, with the two
loaders it leaves unimplemented (from_dict / from_yaml, :27-33) filled in."""
from __future__ import annotations

from dataclasses import dataclass, fields


@dataclass
class DeviceMode:
    CPU_ONLY = "cpu_only"
    CUDA_ONLY = "cuda_only"  # the HIP backend: PyTorch-ROCm names the MI355X "cuda"
    CPU_CUDA = "cpu-cuda"


@dataclass
class HiraConfig:
    # cache
    device_mode: str = DeviceMode.CUDA_ONLY
    update_every: int = 1
    # indexers
    num_levels: int = 5
    max_iterations: int = 1
    branching_factor: int = 10
    # threshold
    threshold_method: str = "sample_mean_topk"  # "sample_max" | "sample_mean_topk" | "exact_topk"
    sample_size: int = 1000
    threshold_topk: int = 10  # k of "sample_mean_topk" (the reference passes k at the call)
    # searcher
    chunk_size = 8 * 1024

    @classmethod
    def from_dict(cls, config_dict: dict) -> "HiraConfig":
        known = {f.name for f in fields(cls)}
        unknown = set(config_dict) - known - {"chunk_size"}
        if unknown:
            raise ValueError(f"unknown HiraConfig keys: {sorted(unknown)}")
        cfg = cls(**{k: v for k, v in config_dict.items() if k in known})
        if "chunk_size" in config_dict:
            cfg.chunk_size = int(config_dict["chunk_size"])
        return cfg

    @classmethod
    def from_yaml(cls, config_path: str) -> "HiraConfig":
        import yaml

        with open(config_path, "r") as f:
            return cls.from_dict(yaml.safe_load(f) or {})

    def get_indexer_kwargs(self) -> dict:
        return {
            "num_levels": self.num_levels,
            "max_iterations": self.max_iterations,
            "branching_factor": self.branching_factor,
        }

    def get_threshold_kwargs(self) -> dict:
        """What the cache layer needs to keep a key sample and turn it into thresholds."""
        return {"method": self.threshold_method, "sample_size": self.sample_size,
                "topk": self.threshold_topk}

    def get_searcher_kwargs(self) -> dict:
        if self.device_mode == DeviceMode.CUDA_ONLY:
            return {"block_c": self.branching_factor}
        return {"chunk_size": self.chunk_size}
