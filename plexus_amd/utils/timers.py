"""Named device-event timers under the reference's timer keys.

The reference wraps every product of the layer in AxoNN timers (``ax.get_timers().start/stop``,
plexus/gcn_conv.py:173-280, plexus/cross_entropy.py:20,103,110,113).  This is the one-GPU counterpart:
HIP events on the current stream, resolved lazily so that timing does not synchronise the stream
while an epoch is in flight.
"""
from __future__ import annotations

from collections import defaultdict
from typing import Dict, List, Tuple

import torch


class Timers:
    def __init__(self):
        self.enabled = False
        self._open: Dict[str, torch.cuda.Event] = {}
        self._pairs: Dict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]] = defaultdict(list)

    def start(self, name: str) -> None:
        if not self.enabled:
            return
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self._open[name] = ev

    def stop(self, name: str) -> None:
        if not self.enabled:
            return
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self._pairs[name].append((self._open.pop(name), ev))

    def get_times(self) -> Dict[str, float]:
        """Total milliseconds per name (synchronises the device)."""
        torch.cuda.synchronize()
        return {k: sum(a.elapsed_time(b) for a, b in v) for k, v in self._pairs.items()}

    def get_counts(self) -> Dict[str, int]:
        return {k: len(v) for k, v in self._pairs.items()}

    def reset(self) -> None:
        self._open.clear()
        self._pairs.clear()


_TIMERS = Timers()


def get_timers() -> Timers:
    return _TIMERS
