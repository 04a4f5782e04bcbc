"""The level-controlled messages (reference: include/pulse/logging.hpp:13-130)."""
import pytest

from pulse_infer_amd import log


def test_levels_filter_and_everything_goes_to_standard_error(capsys):
    log.set_level("info")
    log.debug("not shown")
    log.info("shown %d", 1)
    log.warn("careful")
    out = capsys.readouterr()
    assert out.out == "" and out.err.splitlines() == ["[pulse_infer_amd] shown 1", "[pulse_infer_amd] careful"]
    log.set_level("trace")
    log.trace("fine detail")
    assert log.enabled("debug") and "fine detail" in capsys.readouterr().err
    log.set_level("error")
    log.warn("dropped")
    log.error("kept")
    log.fatal("kept too")
    assert capsys.readouterr().err.splitlines() == ["[pulse_infer_amd] kept", "[pulse_infer_amd] kept too"]
    log.set_level("off")
    log.fatal("silence")
    assert capsys.readouterr().err == "" and not log.enabled("critical")
    log.set_pattern("%(levelname)s|%(message)s")
    log.set_level("debug")
    log.debug("x")
    assert capsys.readouterr().err == "DEBUG|x\n"
    log.set_pattern(log.DEFAULT_PATTERN)
    log.set_level("info")
    with pytest.raises(ValueError, match="unknown log level"):
        log.set_level("loud")


def test_the_serving_loop_reports_at_debug_level(capsys):
    from test_engine_loop import LoopOnly, draw

    log.set_level("debug")
    try:
        engine = LoopOnly(draw, pages=3, page_size=4, batch=2, chunk=4)
        engine.runner = type("R", (), {"graph_records": 0, "graph_replays": 0})()
        for n in (6, 5):
            engine.add_request([3] * n, 5)
        engine.run_until_complete()
        err = capsys.readouterr().err
        assert "step 0: 0 requests running, 2 waiting" in err and "2 of 2 requests finished" in err
        assert "gives its pages back" in err        # a pool of three pages: one of the two was preempted
    finally:
        log.set_level("info")
