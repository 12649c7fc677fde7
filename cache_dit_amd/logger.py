"""Logging helper: `init_logger(__name__)` returns a child of the package
logger with `warning_once` / `info_once` (the reference's logger offers the same
two helpers, src/cache_dit/logger.py:31-160). Level from CACHE_DIT_LOG_LEVEL."""
from __future__ import annotations

import logging
import os
import sys

_ROOT_NAME = "CACHE_DIT_AMD"
_seen: set = set()
_configured = False


class _OnceLogger(logging.LoggerAdapter):

  def process(self, msg, kwargs):
    return msg, kwargs

  def _once(self, level: int, msg: str, *args) -> None:
    key = (self.logger.name, level, msg % args if args else msg)
    if key in _seen:
      return
    _seen.add(key)
    self.logger.log(level, msg, *args)

  def warning_once(self, msg, *args) -> None:
    self._once(logging.WARNING, msg, *args)

  def info_once(self, msg, *args) -> None:
    self._once(logging.INFO, msg, *args)

  def isEnabledFor(self, level):  # noqa: N802
    return self.logger.isEnabledFor(level)


def _configure() -> None:
  global _configured
  if _configured:
    return
  root = logging.getLogger(_ROOT_NAME)
  if not root.handlers:
    h = logging.StreamHandler(sys.stderr)
    h.setFormatter(logging.Formatter("%(levelname)s %(asctime)s [%(name)s:%(lineno)d] %(message)s",
                                     "%m-%d %H:%M:%S"))
    root.addHandler(h)
  root.setLevel(os.environ.get("CACHE_DIT_LOG_LEVEL", "INFO").upper())
  root.propagate = False
  _configured = True


def init_logger(name: str) -> _OnceLogger:
  _configure()
  short = name.split(".", 1)[1] if "." in name else name
  return _OnceLogger(logging.getLogger(f"{_ROOT_NAME}.{short}"), {})
