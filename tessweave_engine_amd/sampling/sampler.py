"""Next-token choice on the device: greedy and temperature sampling.

The reference takes argmax on the device for temperature 0 and otherwise moves
the whole logits row to the CPU and draws with torch.multinomial from a
per-request CPU generator (flow_engine/engine.py:154-158). It samples with
nothing else (no top-p, top-k or penalties). Here both cases are one kernel
over all rows of a step; only the chosen ids come back to the host. The draw
for a request's n-th output token depends on (its seed, n) alone, so a
request's tokens do not depend on what else is in a batch
(tests/test_engine.py:251-260 of the reference). The random stream is this
engine's own, not torch.multinomial's.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops


def validate_temperature(temperature):
    """flow_engine/engine.py:79-80: finite and within [0, 2]."""
    if not isinstance(temperature, (int, float)) or not math.isfinite(temperature) or not 0 <= temperature <= 2:
        raise ValueError("temperature must be finite and between 0 and 2")
    return float(temperature)


class PendingTokens:
    """Token ids that a sampling kernel is still producing; `result()` waits for them."""

    def __init__(self, event, host, rows):
        self.event, self.host, self.rows = event, host, rows

    def result(self):
        self.event.synchronize()
        return self.host[:self.rows].tolist()


class DeviceSampler:
    RING = 4          # pinned staging sets; a set is reused only after its own copies have completed

    def __init__(self, device, capacity=64):
        self.device = device
        self._alloc(capacity)

    def _alloc(self, capacity):
        self.capacity = capacity
        self._temps = torch.zeros(capacity, dtype=torch.float32, device=self.device)
        self._seeds = torch.zeros(capacity, dtype=torch.int64, device=self.device)
        self._counters = torch.zeros(capacity, dtype=torch.int32, device=self.device)
        self._out = torch.zeros(capacity, dtype=torch.int32, device=self.device)
        self._scratch = torch.empty(ops.sample_workspace_bytes(capacity), dtype=torch.uint8, device=self.device)
        self._ring = [dict(temps=torch.zeros(capacity, dtype=torch.float32, pin_memory=True),
                           seeds=torch.zeros(capacity, dtype=torch.int64, pin_memory=True),
                           counters=torch.zeros(capacity, dtype=torch.int32, pin_memory=True),
                           out=torch.zeros(capacity, dtype=torch.int32, pin_memory=True), event=None)
                      for _ in range(self.RING)]
        self._next = 0

    @property
    def out_buffer(self):
        """The device tensor the sampled ids of the latest call are in (row r of the call at index r)."""
        return self._out

    def sample(self, logits, temperatures, seeds, counters):
        """One token id per row of LOGITS (float32 [rows, vocab]); returns a list of ints.

        temperatures[r] == 0 is greedy: the lowest index among the largest logits.
        """
        pending = self.sample_async(logits, temperatures, seeds, counters)
        return pending.result() if pending is not None else []

    def sample_async(self, logits, temperatures, seeds, counters):
        """Start sampling on the current stream; returns PendingTokens (None for no rows).

        Nothing here waits for the device: parameters go up and ids come down through pinned memory.
        """
        rows = logits.shape[0]
        if rows == 0:
            return None
        if rows > self.capacity:
            torch.cuda.current_stream(self.device).synchronize()
            self._alloc(max(rows, 2 * self.capacity))
        slot = self._ring[self._next]
        self._next = (self._next + 1) % self.RING
        if slot["event"] is not None:
            slot["event"].synchronize()
        out = self._out[:rows]
        if all(t == 0 for t in temperatures):
            ops.sample_rows(logits, out, workspace=self._scratch)
        else:
            slot["temps"][:rows] = torch.tensor(temperatures, dtype=torch.float32)
            slot["seeds"][:rows] = torch.tensor([s & (2 ** 63 - 1) for s in seeds], dtype=torch.int64)
            slot["counters"][:rows] = torch.tensor(counters, dtype=torch.int32)
            self._temps[:rows].copy_(slot["temps"][:rows], non_blocking=True)
            self._seeds[:rows].copy_(slot["seeds"][:rows], non_blocking=True)
            self._counters[:rows].copy_(slot["counters"][:rows], non_blocking=True)
            ops.sample_rows(logits, out, temperature=self._temps[:rows], seeds=self._seeds[:rows],
                            counters=self._counters[:rows], workspace=self._scratch)
        slot["out"][:rows].copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self.device))
        slot["event"] = event
        return PendingTokens(event, slot["out"], rows)
