"""Leveled logging to standard error, text or one JSON object a line.

In the manner of the reference's logger (server/logging/logger.h:13-47): levels DEBUG, INFO, WARN,
ERROR; a component name per entry; plain text "[LEVEL] component: message key=value" or, with
INFERFLUX_LOG_FORMAT=json, a JSON object.  The level comes from INFERFLUX_LOG_LEVEL (default WARN,
so that tools which print results on standard output stay quiet).
"""
from __future__ import annotations

import json
import os
import sys
import time

LEVELS = {"DEBUG": 10, "INFO": 20, "WARN": 30, "ERROR": 40}
_level = LEVELS.get(os.environ.get("INFERFLUX_LOG_LEVEL", "WARN").upper(), 30)
_json = os.environ.get("INFERFLUX_LOG_FORMAT", "").lower() == "json"


def set_level(name: str) -> None:
    global _level
    _level = LEVELS[name.upper()]


def set_json_mode(enabled: bool) -> None:
    global _json
    _json = bool(enabled)


def log(level: str, component: str, message: str, **extra) -> None:
    if LEVELS[level] < _level:
        return
    if _json:
        rec = {"ts": round(time.time(), 3), "level": level, "component": component, "message": message, **extra}
        line = json.dumps(rec, default=str)
    else:
        tail = "".join(f" {k}={v}" for k, v in extra.items())
        line = f"[{level}] {component}: {message}{tail}"
    print(line, file=sys.stderr, flush=True)


def debug(component: str, message: str, **extra) -> None: log("DEBUG", component, message, **extra)
def info(component: str, message: str, **extra) -> None: log("INFO", component, message, **extra)
def warn(component: str, message: str, **extra) -> None: log("WARN", component, message, **extra)
def error(component: str, message: str, **extra) -> None: log("ERROR", component, message, **extra)
