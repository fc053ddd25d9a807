from .hira_config import DeviceMode, HiraConfig
from .threshold_finder import THRESHOLD_METHODS, exact_topk, sample_max, sample_mean_topk

__all__ = ["DeviceMode", "HiraConfig", "THRESHOLD_METHODS", "exact_topk", "sample_max",
           "sample_mean_topk"]
