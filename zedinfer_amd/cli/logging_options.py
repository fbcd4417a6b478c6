"""The logging options of the command lines, with the reference's names and meanings
(reference: include/utils/logging_cli.hpp:11-63, include/utils/logging.hpp:56-84): ``--log-level``
(none, fatal, error, warning, info, debug, verbose), ``--log-file``, ``--log-to-console`` /
``--no-log-to-console``, ``--log-append`` / ``--log-overwrite`` (the default; the two exclude each other).
The messages go through Python's ``logging`` under the name ``zedinfer_amd``."""
from __future__ import annotations

import argparse
import logging
import os
import sys

VERBOSE = 5
LEVELS = {"none": logging.CRITICAL + 50, "off": logging.CRITICAL + 50, "fatal": logging.CRITICAL,
          "error": logging.ERROR, "err": logging.ERROR, "warning": logging.WARNING, "warn": logging.WARNING,
          "info": logging.INFO, "debug": logging.DEBUG, "verbose": VERBOSE, "verb": VERBOSE, "trace": VERBOSE}
LOGGER = "zedinfer_amd"


def parse_level(text: str) -> int:
    try:
        return LEVELS[text.strip().lower()]
    except KeyError:
        raise ValueError(f"unknown log level {text!r}: one of none, fatal, error, warning, info, debug, verbose")


def add_logging_arguments(p: argparse.ArgumentParser, default_log_file: str, default_level: str = "info",
                          default_to_console: bool = True) -> None:
    p.add_argument("--log-level", default=default_level,
                   help="Log level: none, fatal, error, warning, info, debug, verbose")
    p.add_argument("--log-file", default=default_log_file, help="Path to the log file")
    p.add_argument("--log-to-console", action="store_true", default=default_to_console,
                   help="Mirror logs to stderr")
    p.add_argument("--no-log-to-console", action="store_true", help="Disable stderr log mirroring")
    p.add_argument("--log-append", action="store_true", help="Append to --log-file instead of replacing it")
    p.add_argument("--log-overwrite", action="store_true", help="Replace --log-file on startup (default)")


def init_logger(args: argparse.Namespace) -> logging.Logger:
    """Configure the ``zedinfer_amd`` logger from parsed options.  A log file that cannot be opened is
    reported on the console and left out; the program goes on."""
    if args.log_append and args.log_overwrite:
        raise ValueError("--log-append and --log-overwrite are mutually exclusive")
    level = parse_level(args.log_level)
    logging.addLevelName(VERBOSE, "VERBOSE")
    log = logging.getLogger(LOGGER)
    for h in list(log.handlers):
        log.removeHandler(h)
    log.setLevel(level)
    log.propagate = False
    fmt = logging.Formatter("%(asctime)s %(levelname)s %(message)s")
    to_console = args.log_to_console and not args.no_log_to_console
    if to_console:
        console = logging.StreamHandler(sys.stderr)
        console.setFormatter(fmt)
        log.addHandler(console)
    if args.log_file and level <= logging.CRITICAL:
        try:
            folder = os.path.dirname(os.path.abspath(args.log_file))
            os.makedirs(folder, exist_ok=True)
            fh = logging.FileHandler(args.log_file, mode="a" if args.log_append else "w")
            fh.setFormatter(fmt)
            log.addHandler(fh)
        except OSError as e:
            print(f"cannot write the log file {args.log_file}: {e}", file=sys.stderr)
    if not log.handlers:
        log.addHandler(logging.NullHandler())
    return log
