"""The command lines' logging options: the reference's names, levels and defaults
(reference: include/utils/logging_cli.hpp:11-63, include/utils/logging.hpp:56-84)."""
import argparse
import logging

import pytest

from zedinfer_amd.cli.logging_options import VERBOSE, add_logging_arguments, init_logger, parse_level


def parser():
    p = argparse.ArgumentParser()
    add_logging_arguments(p, "logs/ping.log")
    return p


def test_names_defaults_and_levels():
    a = parser().parse_args([])
    assert a.log_level == "info" and a.log_file == "logs/ping.log" and a.log_to_console and not a.no_log_to_console
    assert not a.log_append and not a.log_overwrite
    assert parse_level("WARN") == logging.WARNING and parse_level("err") == logging.ERROR
    assert parse_level("trace") == VERBOSE and parse_level("off") > logging.CRITICAL
    with pytest.raises(ValueError, match="unknown log level"):
        parse_level("loud")


def test_file_console_append_and_overwrite(tmp_path, capsys):
    f = tmp_path / "sub" / "x.log"
    log = init_logger(parser().parse_args(["--log-file", str(f), "--log-level", "debug"]))
    log.debug("first")
    assert "first" in f.read_text() and "first" in capsys.readouterr().err
    log = init_logger(parser().parse_args(["--log-file", str(f), "--log-append", "--no-log-to-console"]))
    log.info("second")
    log.debug("hidden")                      # below the level
    for h in log.handlers:
        h.flush()
    text = f.read_text()
    assert "first" in text and "second" in text and "hidden" not in text and capsys.readouterr().err == ""
    log = init_logger(parser().parse_args(["--log-file", str(f)]))       # replaced on startup
    log.warning("third")
    assert "first" not in f.read_text() and "third" in f.read_text()
    with pytest.raises(ValueError, match="mutually exclusive"):
        init_logger(parser().parse_args(["--log-append", "--log-overwrite"]))
    quiet = init_logger(parser().parse_args(["--log-file", str(tmp_path / "none.log"), "--log-level", "none"]))
    quiet.critical("nothing")
    assert not (tmp_path / "none.log").exists()
