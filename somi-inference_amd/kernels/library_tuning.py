"""Autotuning of the library matrix products (the ones ``kernels.linear`` leaves to hipBLASLt/rocBLAS).

The library picks a GEMM solution for a shape by a heuristic; at 7B layer sizes and 2,048 rows the
heuristic's pick for the feed-forward products runs at 0.8 to 1.0 PFLOP/s where the best solution
it ships reaches 1.05 to 1.3.  torch's TunableOp times the shipped solutions once per shape and
remembers the fastest.  Timing costs seconds per shape, so it is switched on only inside
:func:`tuning` (a warm-up run of the shapes that matter); afterwards shapes that were tuned use
their recorded solution and every other shape the library's heuristic, with no timing at run time.
Results are kept in a file under the temporary folder, keyed by the library versions, so the next
process starts from them.
"""

from __future__ import annotations

import contextlib
import os
import stat
import tempfile

import torch


def _results_file() -> str:
    """A file in a folder of the user's own under the temporary folder (a folder of that name that someone else
    made, or that others may write, is not used: a fresh one is made instead)."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    folder = os.path.join(tempfile.gettempdir(), f"somi_inference_amd_tuning_{uid}")
    try:
        os.makedirs(folder, mode=0o700, exist_ok=True)
        info = os.lstat(folder)
        if not stat.S_ISDIR(info.st_mode) or (hasattr(os, "getuid") and info.st_uid != uid) or info.st_mode & 0o022:
            raise OSError("not a private folder")
    except OSError:
        folder = tempfile.mkdtemp(prefix="somi_inference_amd_tuning_")
    return os.path.join(folder, "library_products.csv")


_prepared = False


def _prepare() -> None:
    global _prepared
    if _prepared:
        return
    tunable = torch.cuda.tunable
    tunable.set_filename(_results_file())            # never the working directory
    tunable.set_max_tuning_duration(30)              # ms per candidate
    tunable.set_max_tuning_iterations(20)
    _prepared = True


@contextlib.contextmanager
def tuning():
    """Library products called inside time their candidate solutions once per new shape."""
    tunable = torch.cuda.tunable
    _prepare()
    tunable.enable(True)
    tunable.tuning_enable(True)
    try:
        yield
    finally:
        tunable.tuning_enable(False)                 # recorded shapes keep their solution; nothing new is timed


def tuned_shapes() -> int:
    return len(torch.cuda.tunable.get_results())
