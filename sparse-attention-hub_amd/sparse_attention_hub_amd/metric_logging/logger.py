"""Process-wide logger of small per-call metrics, JSON-lines on disk.

Behavioural mirror of the reference's `MicroMetricLogger`
(sparse_attention_hub/metric_logging/logger.py:12-282) so that code written against it - the
density and output-error hooks of ResearchAttention (research_attention/base.py:121-126,
:150-168) and any external reader of `micro_metrics.jsonl` - keeps working:

* one instance per process; the constructor arguments of the first construction win;
* metrics are registered on the class (`register_metric(name, type)`), enabled per instance
  (`enable_metrics(list | "all")`, unregistered names are dropped with a warning);
* `log(name, value, metadata)` queues an event when a log path is configured and the metric is
  enabled (a warning is printed otherwise), subject to `max_records` and `sampling_factor`;
* `flush()` appends the queued events to `<log_path>/micro_metrics.jsonl`, one JSON object per
  line with the keys `timestamp` (ISO 8601), `metric`, `value`, `metadata`, `location`
  (`module[.Class].function` of the caller of `log`).
"""
from __future__ import annotations

import json
import os
import random
import sys
import time
from collections import deque
from dataclasses import dataclass
from datetime import datetime
from typing import Any, Deque, Dict, Iterable, Optional, Set, Union

_LOG_FILE = "micro_metrics.jsonl"
_QUEUE_LIMIT = 10000


@dataclass
class LogEvent:
    timestamp: datetime
    metric: str
    value: Any
    metadata: Dict[str, Any]
    location: str

    def as_record(self) -> Dict[str, Any]:
        return {
            "timestamp": self.timestamp.isoformat(),
            "metric": self.metric,
            "value": self.value,
            "metadata": self.metadata,
            "location": self.location,
        }


def _caller_name(depth: int) -> str:
    """`module[.Class].function` of the frame `depth` levels above the caller of this helper."""
    try:
        frame = sys._getframe(depth + 1)
    except ValueError:
        return "unknown"
    module = frame.f_globals.get("__name__", "unknown")
    owner = frame.f_locals.get("self")
    parts = [module]
    if owner is not None:
        parts.append(type(owner).__name__)
    parts.append(frame.f_code.co_name)
    return ".".join(parts)


class MicroMetricLogger:
    _instance: Optional["MicroMetricLogger"] = None
    _initialized: bool = False
    _registered_metrics: Dict[str, type] = {}

    def __new__(cls, *args: Any, **kwargs: Any) -> "MicroMetricLogger":
        if cls._instance is None:
            cls._instance = super().__new__(cls)
        return cls._instance

    def __init__(
        self,
        log_path: Optional[str] = None,
        flush_every: int = 1000,
        flush_interval: float = 60.0,
        enabled_metrics: Union[Iterable[str], str, None] = None,
        max_records: Optional[int] = None,
        sampling_factor: float = 1.0,
    ) -> None:
        if MicroMetricLogger._initialized:
            if self.log_path and log_path and self.log_path != log_path:
                print(f"Warning: MicroMetricLogger already initialized with log_path: {self.log_path}")
            return
        self.log_path = log_path
        self.flush_every = flush_every
        self.flush_interval = flush_interval
        self.max_records = max_records
        self.sampling_factor = min(1.0, max(0.0, sampling_factor))
        self.log_queue: Deque[LogEvent] = deque(maxlen=_QUEUE_LIMIT)
        self.enabled_metrics: Set[str] = set()
        self.last_flush_time = time.time()
        self._total_records_logged = 0
        if log_path is not None:
            os.makedirs(log_path, exist_ok=True)
            self.enable_metrics(enabled_metrics)
        MicroMetricLogger._initialized = True

    # ----------------------------------------------------------- registration
    @classmethod
    def register_metric(cls, identifier: str, dtype: type) -> None:
        if identifier in cls._registered_metrics:
            print(f"Warning: Metric '{identifier}' is being re-registered")
        cls._registered_metrics[identifier] = dtype

    @classmethod
    def get_registered_metrics(cls) -> Dict[str, type]:
        return dict(cls._registered_metrics)

    # ---------------------------------------------------------- configuration
    def enable_metrics(self, metrics: Union[Iterable[str], str, None] = None) -> None:
        known = set(self._registered_metrics)
        if metrics == "all":
            self.enabled_metrics = known
        elif isinstance(metrics, (list, set, tuple)):
            wanted = set(metrics)
            unknown = wanted - known
            if unknown:
                print(f"Warning: Attempting to enable unregistered metrics: {unknown}")
            self.enabled_metrics = wanted & known
        else:
            self.enabled_metrics = set()

    def configure_logging(
        self,
        log_path: str,
        enabled_metrics: Union[Iterable[str], str, None] = None,
        max_records: Optional[int] = None,
        sampling_factor: float = 1.0,
    ) -> None:
        self.log_path = log_path
        os.makedirs(log_path, exist_ok=True)
        self.enable_metrics(enabled_metrics)
        self.max_records = max_records
        self.sampling_factor = min(1.0, max(0.0, sampling_factor))
        self._total_records_logged = 0

    # ---------------------------------------------------------------- logging
    def log(self, identifier: str, value: Any, metadata: Optional[Dict[str, Any]] = None) -> None:
        if self.log_path is None:
            print(f"Warning: Cannot log metric '{identifier}' - log_path not defined. Use configure_logging() first.")
            return
        if identifier not in self.enabled_metrics:
            print(f"Warning: Attempting to log metric '{identifier}' which is not enabled")
            return
        if self.max_records is not None and self._total_records_logged >= self.max_records:
            return
        if self.sampling_factor < 1.0 and random.random() > self.sampling_factor:
            return
        self.log_queue.append(LogEvent(datetime.now(), identifier, value, metadata or {}, _caller_name(1)))
        self._total_records_logged += 1
        if len(self.log_queue) >= self.flush_every:
            self.flush()

    def flush(self) -> None:
        if self.log_path is None or not self.log_queue:
            return
        with open(os.path.join(self.log_path, _LOG_FILE), "a", encoding="utf-8") as out:
            while self.log_queue:
                out.write(json.dumps(self.log_queue.popleft().as_record()) + "\n")
        self.last_flush_time = time.time()

    def __del__(self) -> None:
        try:
            self.flush()
        except Exception:
            pass  # interpreter shutdown: the file system may already be gone

    # ---------------------------------------------------------------- queries
    def is_metric_enabled(self, identifier: str) -> bool:
        return identifier in self.enabled_metrics

    def get_enabled_metrics(self) -> Set[str]:
        return set(self.enabled_metrics)

    def is_logging_configured(self) -> bool:
        return self.log_path is not None

    def get_total_records_logged(self) -> int:
        return getattr(self, "_total_records_logged", 0)

    def is_max_records_reached(self) -> bool:
        return self.max_records is not None and self.get_total_records_logged() >= self.max_records

    def get_records_remaining(self) -> Optional[int]:
        if self.max_records is None:
            return None
        return max(0, self.max_records - self.get_total_records_logged())

    def get_sampling_factor(self) -> float:
        return getattr(self, "sampling_factor", 1.0)

    def get_max_records(self) -> Optional[int]:
        return self.max_records
