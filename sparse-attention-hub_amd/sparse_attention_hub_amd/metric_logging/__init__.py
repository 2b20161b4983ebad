"""Micro-metric logging (reference: sparse_attention_hub/metric_logging/)."""
from .logger import LogEvent, MicroMetricLogger

__all__ = ["LogEvent", "MicroMetricLogger"]
