"""Kernel selection for the dense layers' GEMMs.

The GEMMs of the Llama layers and of the drafter head stay with the vendor libraries (torch ->
hipBLASLt / rocBLAS), but which of a library's kernels runs a given problem is a choice: the
default heuristic is up to 11 % off the best kernel for the row counts of a decode step (700-900
rows) when the weights come from HBM, as they do in the model.  `gemm_tuning_gfx950.csv` holds the
winners of a search over every kernel both libraries offer (torch's TunableOp, timed with rotating
buffers so that no weight is served from a cache) for the problem sizes of the 7B-shaped model of
the benchmark; `load()` hands it to torch.  A problem that is not in the table, or a table written
for other library versions (torch checks the versions recorded in the file), leaves the default
heuristic in charge.

Opt-in: nothing in the package calls `load()`.  It switches torch's TunableOp on for the whole
process (look-up only), so every later GEMM of the process goes through
the table; a caller that wants it says so (`recurrent_drafting_amd.gemm_tuning.load()`, as the
benchmark does).
"""

from __future__ import annotations

import os

import torch

TABLE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_tuning_gfx950.csv")
_loaded = None


def load(path: str = TABLE) -> int:
    """Makes torch use the table (once per process).  Returns the number of entries in effect;
    0 when switched off (RD_GEMM_TUNING=0), when there is no GPU or no table, or when torch
    refuses the file."""
    global _loaded
    if _loaded is not None:
        return _loaded
    _loaded = 0
    if os.environ.get("RD_GEMM_TUNING", "1") == "0" or not torch.cuda.is_available() or not os.path.exists(path):
        return 0
    import torch.cuda.tunable as tunable

    tunable.enable(True)
    tunable.tuning_enable(False)  # look up only: never search inside a decode step
    if hasattr(tunable, "write_file_on_exit"):
        tunable.write_file_on_exit(False)  # leave no results file in the working directory
    if tunable.read_file(path):
        _loaded = len(tunable.get_results())
    if _loaded == 0:
        tunable.enable(False)
    return _loaded
