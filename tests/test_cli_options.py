"""The command lines' logging options (the reference's names, levels and defaults) and text prompts through a supplied tokenizer
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


def test_text_prompts_through_a_supplied_tokenizer(tmp_path):
    """``ping --prompt`` encodes with a tokenizer.json beside the model (the engine itself is ids in, ids out)."""
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    from zedinfer_amd.cli.main import load_tokenizer
    tok = tokenizers.Tokenizer(WordLevel({"[UNK]": 0, "a": 1, "token": 2, "in": 3, "out": 4}, unk_token="[UNK]"))
    tok.pre_tokenizer = Whitespace()
    tok.save(str(tmp_path / "tokenizer.json"))
    loaded = load_tokenizer(str(tmp_path / "tokenizer.json"))
    assert loaded.encode("a token in a token out").ids == [1, 2, 3, 1, 2, 4]
    assert loaded.decode([2, 4]) == "token out"
    with pytest.raises(OSError, match="no tokenizer file"):
        load_tokenizer(str(tmp_path / "none.json"))
