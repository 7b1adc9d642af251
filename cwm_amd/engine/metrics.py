"""A log of the scheduler's events as JSON lines, switched on by the environment.

With `FG_METRICS=path` in the environment every event is appended to that file as one
JSON object with its kind, a timestamp and the event's own fields; without it nothing
is recorded.  The variable's name and the kinds `nactive` (the number of running
requests has changed; with the free pages), `yield` (a request is finished and handed
back) and `unpark` (a preempted request is admitted again) are the reference's
(cwm/fastgen/utils/metrics.py:13-38; call sites cwm/fastgen/generate.py:471-478,513,
637); `preempt` is added here.
"""

from __future__ import annotations

import json
import os
import time
from typing import Any, Optional, TextIO


class MetricsLog:
    def __init__(self, path: Optional[str] = None) -> None:
        """`path` None: taken from FG_METRICS when the first event arrives."""
        self._path = path
        self._file: Optional[TextIO] = None
        self._resolved = path is not None

    def enabled(self) -> bool:
        if not self._resolved:
            self._path = os.environ.get("FG_METRICS") or None
            self._resolved = True
        return self._path is not None

    def record(self, kind: str, **fields: Any) -> None:
        if not self.enabled():
            return
        if self._file is None:
            self._file = open(self._path, "a", encoding="utf-8")
        self._file.write(json.dumps({"kind": kind, "timestamp": time.time(), **fields}) + "\n")
        self._file.flush()

    def close(self) -> None:
        if self._file is not None:
            self._file.close()
            self._file = None
