"""JSONL event log of the scheduler.

Behaviour as the reference's audit trace (flow_engine/trace.py:9-28): one JSON
object per line with wall and monotonic time and the event kind; events carry
counts and timings, never prompts, text or token ids; the file is bounded
(20 MiB, four older files kept); without a path every call does nothing.
"""
from __future__ import annotations

import json
import os
import threading
import time

MAX_BYTES = 20 * 1024 * 1024
KEPT_FILES = 4


class Trace:
    def __init__(self, path=None, max_bytes=MAX_BYTES, kept_files=KEPT_FILES):
        self._path = os.fspath(path) if path else None
        self._max_bytes, self._kept = int(max_bytes), int(kept_files)
        self._guard = threading.Lock()
        self._file = None
        self._written = 0
        if self._path:
            folder = os.path.dirname(self._path)
            if folder:
                os.makedirs(folder, exist_ok=True)
            self._open()

    def _open(self):
        self._file = open(self._path, "a", encoding="utf-8")
        self._written = self._file.tell()

    def _rotate(self):
        self._file.close()
        for n in range(self._kept, 0, -1):
            older = f"{self._path}.{n}"
            newer = self._path if n == 1 else f"{self._path}.{n - 1}"
            if os.path.exists(newer):
                os.replace(newer, older)
        self._open()

    def emit(self, kind, **data):
        if self._file is None:
            return
        line = json.dumps({"time": time.time(), "monotonic": time.monotonic(), "event": kind, **data},
                          allow_nan=False, ensure_ascii=False) + "\n"
        with self._guard:
            if self._file is None:
                return
            if self._written and self._written + len(line) > self._max_bytes:
                self._rotate()
            self._file.write(line)
            self._file.flush()
            self._written += len(line)

    def close(self):
        with self._guard:
            if self._file is not None:
                self._file.close()
                self._file = None


def read_events(path, kinds=("step", "admit", "finish", "first_token", "fatal")):
    """The events of a trace file whose kind is in KINDS (what `replay` prints, flow_engine/cli.py:94-98)."""
    with open(path, encoding="utf-8") as f:
        for line in f:
            line = line.strip()
            if line:
                event = json.loads(line)
                if event.get("event") in kinds:
                    yield event
