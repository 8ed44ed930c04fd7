"""Per-step timers and the Tokens/second summary, with the keys the reference's stats module uses
(recurrent_drafting/stats.py): `step_record.time(key)`, `step_record.set({...})`, `summarize`.

Records are kept in memory (the reference writes JSON lines to a temporary directory); a timed
block is bracketed by device synchronisation exactly when `Ledger(sync=True)`, the default.
"""

from __future__ import annotations

import contextlib
import dataclasses
import time
from typing import Any, Dict, Generator, List

import torch


class TextGeneration:
    """Stats of one call to RecurrentDrafting.generate."""

    def __init__(self, sync: bool = True) -> None:
        self.n_steps = 0
        self.sync = sync
        self.wall_times: Dict[str, List[float]] = {}
        self.stats: Dict[str, Any] = {"step": [], "wall_times": self.wall_times}

    @contextlib.contextmanager
    def step(self) -> Generator["TextGeneration.Step", None, None]:
        record = TextGeneration.Step(self)
        yield record
        self.stats["step"].append(self.n_steps)
        self.n_steps += 1

    class Step:
        def __init__(self, owner: "TextGeneration") -> None:
            self._owner = owner

        @contextlib.contextmanager
        def time(self, key: str) -> Generator[None, None, None]:
            sync = self._owner.sync and torch.cuda.is_available()
            with torch.profiler.record_function(key):
                if sync:
                    torch.cuda.synchronize()
                start = time.perf_counter()
                try:
                    yield
                finally:
                    if sync:
                        torch.cuda.synchronize()
                    self._owner.wall_times.setdefault(key, []).append(time.perf_counter() - start)

        def set(self, values: Dict[str, Any]) -> None:
            for key, value in values.items():
                self._owner.stats.setdefault(key, []).append(value)


class Ledger:
    """Collects the stats of every generate call."""

    def __init__(self, sync: bool = True) -> None:
        self.sync = sync
        self.records: List[Dict[str, Any]] = []


@contextlib.contextmanager
def text_generation(ledger: Ledger) -> Generator[TextGeneration, None, None]:
    r = TextGeneration(sync=ledger.sync)
    try:
        yield r
    finally:
        ledger.records.append(r.stats)


@dataclasses.dataclass
class TableStats:
    avg_token_per_step: float  # per sequence
    acceptance_rate: float
    avg_generate_candidates: float
    avg_verify_candidates: float
    avg_accept_candidate_tokens: float
    avg_step_time: float

    @property
    def tokens_per_second(self) -> float:
        """Per-sequence tokens per step over the summed three stage times (stats.py:235)."""
        return self.avg_token_per_step / self.avg_step_time


def summarize(ledger: Ledger, batch_size: int, candidate_len: int) -> TableStats:
    """Means over all recorded steps (stats.py:158-215)."""
    n_steps, tokens = 0, 0.0
    times = {"generate_candidates": [], "verify_candidates": [], "accept_candidate_tokens": []}
    for rec in ledger.records:
        for accepted in rec.get("avg_num_accepted", []):
            n_steps += 1
            tokens += batch_size * (float(accepted) + 1)
        for key in times:
            times[key] += rec["wall_times"].get(key, [])
    per_step = tokens / max(n_steps, 1)
    mean = {k: (sum(v) / len(v) if v else 0.0) for k, v in times.items()}
    return TableStats(
        per_step / batch_size,
        100.0 * (per_step - batch_size) / batch_size / candidate_len,
        mean["generate_candidates"], mean["verify_candidates"], mean["accept_candidate_tokens"],
        sum(mean.values()),
    )
