"""Counters, gauges and histograms of the engine, and its log.

The reference registers counters (``llm.prompt_recv``), gauges (``llm.alive_prompt``) and histograms
(sampler timings) with a recorder that writes all of them to the log once a minute, histograms as the
quantiles 0, 0.8, 0.9, 0.99, 0.999 and 1 over a window of the last summaries
(common/src/metrics.rs:35-110, :136-195; core/src/engine/llm_engine.rs:794-795), and sets up a log
that goes to stderr or to a daily file ``lmsf.log`` in ``--log-dir`` (common/src/tracing.rs:1-22).
The same here, without a background thread: the engine calls ``maybe_report`` at the end of a step,
and a report is written when the interval has passed. Histograms keep the last ``window`` values.
"""
import collections
import logging
import logging.handlers
import os
import sys
import time
from typing import Deque, Dict, List, Optional

QUANTILES = ((0.0, "min"), (0.8, "p80"), (0.9, "p90"), (0.99, "p99"), (0.999, "p999"), (1.0, "max"))
LOGGER_NAME = "lmsf_amd"


def init_logging(log_dir: Optional[str] = None, alsologtostderr: bool = False) -> logging.Logger:
    """The engine's logger: to ``log_dir``/lmsf.log (a new file every day) if a folder is given, to
    stderr if none is given or ``alsologtostderr`` is set. Calling it again replaces the handlers."""
    log = logging.getLogger(LOGGER_NAME)
    for h in list(log.handlers):
        log.removeHandler(h)
        h.close()
    fmt = logging.Formatter("%(asctime)s %(levelname)s %(filename)s:%(lineno)d %(message)s")
    if log_dir:
        os.makedirs(log_dir, exist_ok=True)
        fh = logging.handlers.TimedRotatingFileHandler(os.path.join(log_dir, "lmsf.log"), when="midnight", backupCount=0,
                                                       delay=True)
        fh.setFormatter(fmt)
        log.addHandler(fh)
    if not log_dir or alsologtostderr:
        sh = logging.StreamHandler(sys.stderr)
        sh.setFormatter(fmt)
        log.addHandler(sh)
    log.setLevel(logging.INFO)
    log.propagate = False
    return log


class Histogram:
    def __init__(self, window: int):
        self.values: Deque[float] = collections.deque(maxlen=window)
        self.count = 0

    def record(self, v: float) -> None:
        self.values.append(float(v))
        self.count += 1

    def quantiles(self) -> Dict[str, float]:
        """The value at each of QUANTILES (nearest rank over the window); empty if nothing was recorded."""
        if not self.values:
            return {}
        xs = sorted(self.values)
        n = len(xs)
        return {label: xs[min(n - 1, max(0, int(q * n + 0.5) - 1 if q > 0 else 0))] for q, label in QUANTILES}


class Metrics:
    """``counter(name, n)``, ``gauge(name, v)``, ``histogram(name, v)``; ``snapshot()`` gives all of them."""

    def __init__(self, report_interval_s: float = 60.0, window: int = 4096, logger: Optional[logging.Logger] = None):
        self.counters: Dict[str, int] = collections.defaultdict(int)
        self.gauges: Dict[str, float] = {}
        self.histograms: Dict[str, Histogram] = {}
        self.report_interval_s = report_interval_s
        self.window = window
        self.logger = logger
        self._last_report = time.monotonic()

    def counter(self, name: str, n: int = 1) -> None:
        self.counters[name] += n

    def gauge(self, name: str, v: float) -> None:
        self.gauges[name] = v

    def histogram(self, name: str, v: float) -> None:
        h = self.histograms.get(name)
        if h is None:
            h = self.histograms[name] = Histogram(self.window)
        h.record(v)

    def snapshot(self) -> Dict[str, Dict]:
        return {"counters": dict(self.counters), "gauges": dict(self.gauges),
                "histograms": {k: h.quantiles() for k, h in self.histograms.items()}}

    def report_lines(self) -> List[str]:
        snap = self.snapshot()
        lines = ["Gauges:"] + ["%s:%g" % kv for kv in sorted(snap["gauges"].items())]
        lines += ["Counters:"] + ["%s:%d" % kv for kv in sorted(snap["counters"].items())]
        lines += ["Histograms:"]
        for name, qs in sorted(snap["histograms"].items()):
            lines += ["%s_%s:%.6g" % (name, label, qs[label]) for _, label in QUANTILES if label in qs]
        return lines

    def maybe_report(self, now: Optional[float] = None) -> bool:
        """Write a report to the log if the interval has passed since the last one."""
        now = time.monotonic() if now is None else now
        if self.logger is None or now - self._last_report < self.report_interval_s:
            return False
        self._last_report = now
        self.logger.info("\n".join(["======== metrics ========"] + self.report_lines()))
        return True
