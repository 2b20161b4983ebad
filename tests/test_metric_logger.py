"""MicroMetricLogger: the behaviours the reference's own unit tests check
(tests/unit/metric_logging/test_micro_metric_logger.py) - singleton, class-level registration,
enabling, warnings, queue / flush, JSON-lines record layout, record limit and sampling."""
import json
from datetime import datetime

import pytest

from sparse_attention_hub_amd.metric_logging import LogEvent, MicroMetricLogger


@pytest.fixture()
def fresh_logger():
    """Each test starts from an unconstructed singleton with no registered metrics; the process-wide
    state (ResearchAttention registers two metrics at import) is restored afterwards."""
    saved = (MicroMetricLogger._instance, MicroMetricLogger._initialized, dict(MicroMetricLogger._registered_metrics))
    MicroMetricLogger._instance = None
    MicroMetricLogger._initialized = False
    MicroMetricLogger._registered_metrics = {}
    yield MicroMetricLogger
    MicroMetricLogger._instance, MicroMetricLogger._initialized, MicroMetricLogger._registered_metrics = saved


def test_log_event_fields():
    t = datetime.now()
    e = LogEvent(timestamp=t, metric="m", value=42.0, metadata={"layer": 1, "head": 2}, location="a.b.c")
    assert (e.timestamp, e.metric, e.value, e.metadata, e.location) == (t, "m", 42.0, {"layer": 1, "head": 2}, "a.b.c")
    assert LogEvent(t, "m", None, {}, "x").value is None


def test_singleton_and_first_construction_wins(fresh_logger, tmp_path):
    a = fresh_logger(log_path=str(tmp_path / "one"))
    b = fresh_logger(log_path=str(tmp_path / "two"))
    assert a is b and b.log_path == str(tmp_path / "one")
    assert (tmp_path / "one").is_dir() and not (tmp_path / "two").exists()


def test_defaults(fresh_logger):
    lg = fresh_logger()
    assert lg.log_path is None and lg.flush_every == 1000 and lg.flush_interval == 60.0
    assert lg.enabled_metrics == set() and len(lg.log_queue) == 0 and lg.log_queue.maxlen == 10000
    assert lg.is_logging_configured() is False
    custom = None
    MicroMetricLogger._instance, MicroMetricLogger._initialized = None, False
    custom = fresh_logger(log_path=None, flush_every=500, flush_interval=30.0)
    assert custom.flush_every == 500 and custom.flush_interval == 30.0


def test_registration_is_class_level(fresh_logger, capsys):
    fresh_logger.register_metric("attention_score", float)
    fresh_logger.register_metric("sparsity_ratio", float)
    reg = fresh_logger.get_registered_metrics()
    assert reg == {"attention_score": float, "sparsity_ratio": float}
    reg["new_metric"] = int
    assert "new_metric" not in fresh_logger.get_registered_metrics()
    fresh_logger.register_metric("attention_score", float)
    assert "Warning: Metric 'attention_score' is being re-registered" in capsys.readouterr().out


def test_enable_metrics(fresh_logger, tmp_path, capsys):
    for name in ("metric1", "metric2", "metric3"):
        fresh_logger.register_metric(name, float)
    lg = fresh_logger(log_path=str(tmp_path), enabled_metrics="all")
    assert lg.enabled_metrics == {"metric1", "metric2", "metric3"}
    lg.enable_metrics(["metric1", "metric3"])
    assert lg.enabled_metrics == {"metric1", "metric3"}
    assert lg.is_metric_enabled("metric1") is True and lg.is_metric_enabled("metric2") is False
    lg.enable_metrics(["metric1", "nope"])
    assert "Warning: Attempting to enable unregistered metrics" in capsys.readouterr().out
    assert lg.enabled_metrics == {"metric1"}
    got = lg.get_enabled_metrics()
    got.add("metric3")
    assert "metric3" not in lg.enabled_metrics
    lg.enable_metrics(None)
    assert lg.enabled_metrics == set()
    lg.enable_metrics([])
    assert lg.enabled_metrics == set()


def test_log_needs_a_path_and_an_enabled_metric(fresh_logger, tmp_path, capsys):
    fresh_logger.register_metric("test_metric", float)
    lg = fresh_logger()
    lg.log("test_metric", 1.0)
    assert "Cannot log metric 'test_metric' - log_path not defined" in capsys.readouterr().out
    lg.configure_logging(str(tmp_path), enabled_metrics=[])
    assert lg.is_logging_configured() is True
    lg.log("test_metric", 1.0)
    assert "Attempting to log metric 'test_metric' which is not enabled" in capsys.readouterr().out
    assert len(lg.log_queue) == 0


def test_log_queue_flush_and_record_layout(fresh_logger, tmp_path):
    fresh_logger.register_metric("test_metric", float)
    lg = fresh_logger(log_path=str(tmp_path), enabled_metrics=["test_metric"])
    lg.flush()
    assert not (tmp_path / "micro_metrics.jsonl").exists()        # nothing queued: no file
    lg.log("test_metric", 42.0, {"layer": 1})
    lg.log("test_metric", 43.0)
    assert len(lg.log_queue) == 2
    first = lg.log_queue[0]
    assert first.metric == "test_metric" and first.value == 42.0 and first.metadata == {"layer": 1}
    assert isinstance(first.timestamp, datetime) and lg.log_queue[1].metadata == {}
    assert first.location.endswith("test_metric_logger.test_log_queue_flush_and_record_layout")
    before = lg.last_flush_time
    lg.flush()
    assert len(lg.log_queue) == 0 and lg.last_flush_time >= before
    lines = (tmp_path / "micro_metrics.jsonl").read_text().splitlines()
    assert len(lines) == 2
    rec = json.loads(lines[0])
    assert set(rec) == {"timestamp", "metric", "value", "metadata", "location"}
    assert rec["metric"] == "test_metric" and rec["value"] == 42.0 and rec["metadata"] == {"layer": 1}
    datetime.fromisoformat(rec["timestamp"])
    lg.log("test_metric", 1.0)
    lg.flush()                                                      # appends
    assert len((tmp_path / "micro_metrics.jsonl").read_text().splitlines()) == 3


def test_auto_flush_record_limit_and_sampling(fresh_logger, tmp_path):
    fresh_logger.register_metric("m", float)
    lg = fresh_logger(log_path=str(tmp_path), flush_every=3, enabled_metrics=["m"])
    for i in range(3):
        lg.log("m", float(i))
    assert len(lg.log_queue) == 0                                   # third event triggered the flush
    lg.configure_logging(str(tmp_path), enabled_metrics=["m"], max_records=2)
    assert lg.get_total_records_logged() == 0 and lg.get_records_remaining() == 2 and lg.get_max_records() == 2
    for i in range(5):
        lg.log("m", float(i))
    assert lg.get_total_records_logged() == 2 and lg.is_max_records_reached() and lg.get_records_remaining() == 0
    lg.configure_logging(str(tmp_path), enabled_metrics=["m"], sampling_factor=0.0)
    for i in range(20):
        lg.log("m", float(i))
    assert lg.get_total_records_logged() == 0 and lg.get_sampling_factor() == 0.0
    lg.configure_logging(str(tmp_path), enabled_metrics=["m"], sampling_factor=7.0)
    assert lg.get_sampling_factor() == 1.0 and lg.get_records_remaining() is None
