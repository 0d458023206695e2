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


class DeviceSampler:
    def __init__(self, device, capacity=64):
        self.device = device
        self._alloc(capacity)

    def _alloc(self, capacity):
        self.capacity = capacity
        self._host = torch.zeros(capacity, 4, dtype=torch.int64, pin_memory=True)    # temp bits, seed, counter
        self._temps = torch.zeros(capacity, dtype=torch.float32, device=self.device)
        self._seeds = torch.zeros(capacity, dtype=torch.int64, device=self.device)
        self._counters = torch.zeros(capacity, dtype=torch.int32, device=self.device)
        self._out = torch.zeros(capacity, dtype=torch.int32, device=self.device)

    def sample(self, logits, temperatures, seeds, counters):
        """One token id per row of LOGITS (float32 [rows, vocab]); returns a list of ints.

        temperatures[r] == 0 is greedy: the lowest index among the largest logits.
        """
        rows = logits.shape[0]
        if rows == 0:
            return []
        if rows > self.capacity:
            self._alloc(max(rows, 2 * self.capacity))
        out = self._out[:rows]
        if all(t == 0 for t in temperatures):
            ops.sample_rows(logits, out)
        else:
            self._temps[:rows].copy_(torch.tensor(temperatures, dtype=torch.float32), non_blocking=False)
            self._seeds[:rows].copy_(torch.tensor([s & (2 ** 63 - 1) for s in seeds], dtype=torch.int64))
            self._counters[:rows].copy_(torch.tensor(counters, dtype=torch.int32))
            ops.sample_rows(logits, out, temperature=self._temps[:rows], seeds=self._seeds[:rows],
                            counters=self._counters[:rows])
        return out.tolist()
