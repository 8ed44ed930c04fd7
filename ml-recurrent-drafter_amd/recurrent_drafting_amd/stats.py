"""Per-step timers and the Tokens/second summary, with the keys the reference's stats module uses
(recurrent_drafting/stats.py): `step_record.time(key)`, `step_record.set({...})`, `summarize`.

Records are kept in memory (the reference writes JSON lines to a temporary directory); a timed
block is bracketed by device synchronisation exactly when `Ledger(sync=True)`, the default.
"""

from __future__ import annotations

import contextlib
import dataclasses
import time
from typing import Any, Dict, Generator, List, Tuple

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


@dataclasses.dataclass
class PlotStats:
    sorted_steps: List[int]
    sorted_num_tokens_step: List[float]  # batch tokens per step index, averaged over the generations
    sorted_input_lengths: List[int]
    sorted_num_tokens_input_length: List[float]  # the same, grouped by the step's input length
    acceptance_rate: float


def summarize(ledger: Ledger, batch_size: int, candidate_len: int) -> Tuple[TableStats, PlotStats]:
    """(TableStats, PlotStats) over every recorded step of every generation (stats.py:158-215).

    A step that accepted `a` drafted tokens per sequence on average produced batch_size * (a + 1)
    tokens; the acceptance rate is the share of the candidate_len drafted tokens that were kept."""
    per_step: Dict[int, List[float]] = {}
    per_length: Dict[int, List[float]] = {}
    times = {"generate_candidates": [], "verify_candidates": [], "accept_candidate_tokens": []}
    for rec in ledger.records:
        accepted = rec.get("avg_num_accepted", [])
        for step, a in zip(rec.get("step", []), accepted):
            per_step.setdefault(step, []).append(batch_size * (float(a) + 1))
        for length, a in zip(rec.get("input_id_length", []), accepted):
            per_length.setdefault(length, []).append(batch_size * (float(a) + 1))
        for key in times:
            times[key] += rec["wall_times"].get(key, [])
    steps = sorted(per_step)
    lengths = sorted(per_length)
    n_steps = sum(len(per_step[i]) for i in steps)
    tokens = sum(sum(per_step[i]) for i in steps)
    per_step_tokens = tokens / max(n_steps, 1)
    rate = 100.0 * (per_step_tokens - batch_size) / batch_size / candidate_len
    mean = {k: (sum(v) / len(v) if v else 0.0) for k, v in times.items()}
    table = TableStats(
        per_step_tokens / batch_size, rate,
        mean["generate_candidates"], mean["verify_candidates"], mean["accept_candidate_tokens"],
        sum(mean.values()),
    )
    plot = PlotStats(
        steps, [sum(per_step[i]) / len(per_step[i]) for i in steps],
        lengths, [sum(per_length[i]) / len(per_length[i]) for i in lengths], rate,
    )
    return table, plot


def draw_table(title: str, ts: TableStats) -> None:
    """Prints the summary with the reference's row labels (stats.py:218-241)."""
    rows = [
        ("Average number of tokens per step:", f"{ts.avg_token_per_step:.4f}"),
        ("Average draft head acceptance rate (%):", f"{ts.acceptance_rate:.4f}"),
        ("generate_candidates:", f"{ts.avg_generate_candidates:.4f}"),
        ("verify_candidates:", f"{ts.avg_verify_candidates:.4f}"),
        ("accept_candidate_tokens:", f"{ts.avg_accept_candidate_tokens:.4f}"),
        ("Tokens/second", f"{ts.tokens_per_second:.4f}"),
    ]
    width = max(len(label) for label, _ in rows)
    print(f"Title: {title}")
    for label, value in rows:
        print(f"{label:<{width}}  {value:>12}")
