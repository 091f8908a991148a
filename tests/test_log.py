"""The leveled logger (the reference's static Logger, src/log/Logger.h:17-36)."""
import io

import pytest

from tffinfer_amd import log


@pytest.fixture
def captured():
    buf = io.StringIO()
    level, app, stream = log.get_level(), log._State.app, log._State.stream
    log.init("unit", "info", buf)
    yield buf
    log.init(app, level, stream)


def test_levels_and_printf_formats(captured):
    log.debug("hidden %d", 1)
    log.info("loaded %s in %.1f s", "m", 2.25)
    log.warning("pages short: %d", 3)
    log.error("no %s", "gpu")
    lines = captured.getvalue().splitlines()
    assert [ln[0] for ln in lines] == ["I", "W", "E"]
    assert lines[0].endswith("unit] loaded m in 2.2 s") or lines[0].endswith("unit] loaded m in 2.3 s")
    assert all(" unit] " in ln for ln in lines)
    log.set_level("error")
    log.warning("dropped")
    assert len(captured.getvalue().splitlines()) == 3
    log.set_level("debug")
    log.debug("now %s", "shown")
    assert captured.getvalue().splitlines()[-1].startswith("D")


def test_fatal_logs_and_raises(captured):
    with pytest.raises(log.FatalError, match="cache of 3 pages"):
        log.fatal("cache of %d pages", 3)
    assert captured.getvalue().splitlines()[-1].startswith("F")


def test_a_bad_format_never_loses_the_message(captured):
    log.info("count %d", "seven")
    assert "count %d" in captured.getvalue() and "seven" in captured.getvalue()


def test_off_and_unknown_level(captured):
    log.set_level("off")
    log.error("nothing")
    assert captured.getvalue() == ""
    with pytest.raises(ValueError):
        log.set_level("loud")
