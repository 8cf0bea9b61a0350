"""The engine's counters, gauges and histograms and its log (CPU, torch stand-ins for the kernels)."""
import logging
import os

from helpers import TINY, make_model_folder, random_tokens
from torch_ops import TorchOps

from lmsf_amd.engine import EngineArgs, LLMEngine
from lmsf_amd.engine.metrics import QUANTILES, Histogram, Metrics, init_logging
from lmsf_amd.sampling import SamplingParams


def test_histogram_quantiles_over_the_window():
    h = Histogram(window=1000)
    assert h.quantiles() == {}
    for v in range(1, 1001):
        h.record(v)
    q = h.quantiles()
    assert [label for _, label in QUANTILES] == list(q)
    assert (q["min"], q["p80"], q["p90"], q["p99"], q["p999"], q["max"]) == (1, 800, 900, 990, 999, 1000)
    h.record(5000)                       # the window moves on: 1 has left it
    assert h.quantiles()["min"] == 2 and h.quantiles()["max"] == 5000 and h.count == 1001
    one = Histogram(window=4)
    one.record(3.5)
    assert set(one.quantiles().values()) == {3.5}


def test_report_goes_to_the_log_when_the_interval_has_passed(tmp_path):
    log = init_logging(str(tmp_path / "logs"))
    m = Metrics(report_interval_s=60.0, logger=log)
    m.counter("c", 2)
    m.counter("c")
    m.gauge("g", 1.5)
    m.histogram("h", 0.25)
    assert not m.maybe_report(now=m._last_report + 59.0)
    assert m.maybe_report(now=m._last_report + 61.0)
    for h in log.handlers:
        h.flush()
    text = open(os.path.join(str(tmp_path / "logs"), "lmsf.log")).read()
    assert "c:3" in text and "g:1.5" in text and "h_p99:0.25" in text and "h_max:0.25" in text
    assert Metrics(logger=None).maybe_report(now=1e12) is False
    init_logging(None, False)            # back to stderr only: the file is closed
    assert all(not isinstance(h, logging.FileHandler) for h in logging.getLogger("lmsf_amd").handlers)


def test_engine_counts_what_it_does(tmp_path):
    folder, cfg = make_model_folder(tmp_path, "A")
    args = EngineArgs(model=folder, dtype="float32", block_size=TINY["A"][2], device="cpu", num_gpu_blocks_override=64,
                      max_num_seqs=8, prefill_chunk_size=16, log_dir=str(tmp_path / "logs"))
    engine = LLMEngine(args, ops=TorchOps())
    engine.metrics.report_interval_s = 0.0           # a report after every step
    for i, n in enumerate((5, 40)):
        engine.add_request(i, random_tokens(n, cfg.vocab_size, i), SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    first = None
    while engine.has_unfinished_requests():
        engine.step()
        first = first or dict(engine.last_step)
    snap = engine.metrics.snapshot()
    c, g, h = snap["counters"], snap["gauges"], snap["histograms"]
    assert c["llm.prompt_recv"] == 2 and c["llm.generated_tokens"] == 8 and c["llm.steps"] == engine.stats["steps"]
    assert c["llm.tokens"] == engine.stats["tokens"] == 5 + 40 + 2 * 3
    assert g["llm.alive_prompt"] == 0 and g["llm.free_pages"] == 64
    assert set(h) >= {"llm.step_ms", "llm.step_tokens", "llm.request_s", "llm.first_token_s"}
    assert h["llm.step_tokens"]["max"] == first["tokens"] == 5 + 16      # the short prompt whole, a portion of the long one
    assert first["prefill_tokens"] == 21 and first["decode_tokens"] == 0 and first["sequences"] == 2 and first["ms"] > 0
    assert engine.last_step["decode_tokens"] >= 1
    for hd in engine.logger.handlers:
        hd.flush()
    assert "llm.generated_tokens:8" in open(os.path.join(str(tmp_path / "logs"), "lmsf.log")).read()
    init_logging(None, False)
