"""Timing / memory / correctness harness with the interface and the log layout
of the reference's python/graphiler/utils/bench.py:10-62, and the table writer
of artifact/plot.py:88-96.

``bench`` fills a ``pandas.Series`` indexed by (tag, metric); a dictionary
{dataset: Series} turned into a ``DataFrame`` and pickled is the file format
the reference's plot script reads (examples/GAT/GAT.py:175-187,
artifact/plot.py:115), so results written here line up with its figures:
time in ms per inference, memory in MiB of intermediate data, 0.0 for a run
that ran out of memory and -1.0 ("N/A" in the plots, plot.py:24) for a baseline
that cannot run here.
"""
from __future__ import annotations

import os
import time
from typing import Callable, Iterable, Optional

import numpy as np
import pandas as pd
import torch

NOT_AVAILABLE = -1.0


def check_equal(first, second, rtol: float = 1e-3) -> bool:
    """bench.py:10-16: relative tolerance 1e-3 between two results; a missing
    result (out of memory) only prints a notice."""
    if first is None or second is None:
        print("cannot guarantee correctness because of OOM")
        return False
    np.testing.assert_allclose(first.detach().float().cpu().numpy(),
                               second.detach().float().cpu().numpy(), rtol=rtol)
    print("correctness check passed!")
    return True


WARM_UP_CALLS = 5


def is_out_of_memory(err: RuntimeError) -> bool:
    # torch.cuda.OutOfMemoryError is a RuntimeError; raised inside a TorchScript
    # plan it arrives as a plain RuntimeError with the same text
    return "out of memory" in str(err).lower()


def _timed_calls(net: Callable, params: tuple, repeat: int, mark_range: bool):
    """``repeat`` back-to-back calls between two device synchronisations;
    returns (last result, wall-clock milliseconds per call)."""
    result = None
    if mark_range:
        torch.cuda.profiler.start()
    t0 = time.perf_counter()
    for _ in range(repeat):
        result = net(*params)
    torch.cuda.synchronize()
    per_call_ms = (time.perf_counter() - t0) * 1e3 / max(repeat, 1)
    if mark_range:
        torch.cuda.profiler.stop()
    return result, per_call_ms


def bench(net: Callable, net_params: Iterable, tag: str = "", nvprof: bool = False,
          memory: bool = False, repeat: int = 1000, log: Optional[pd.Series] = None):
    """Same contract as bench.py:19-49: five warm-up calls, ``repeat`` timed calls
    between two device synchronisations, wall clock per call in ms into
    ``log[tag, "time"]``; with ``memory`` the peak of newly allocated device
    memory in MiB into ``log[tag, "mem"]``.  ``nvprof`` brackets the timed loop
    with the profiler's start / stop marks (a range for rocprofv3's marker trace).
    Out of memory prints "<tag> OOM", leaves the log entries at 0 and returns
    None; any other error propagates."""
    params = tuple(net_params)
    try:
        for _ in range(WARM_UP_CALLS):
            net(*params)
        torch.cuda.synchronize()
        baseline_bytes = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        result, per_call_ms = _timed_calls(net, params, repeat, nvprof)
    except RuntimeError as err:
        if not is_out_of_memory(err):
            raise
        print("{} OOM".format(tag))
        torch.cuda.empty_cache()
        return None
    print("{} elapsed time: {} ms/infer".format(tag, per_call_ms))
    if log is not None:
        log.at[(tag, "time")] = per_call_ms
    if memory:
        peak_mib = (torch.cuda.max_memory_allocated() - baseline_bytes) / 2 ** 20
        print("intermediate data memory usage: {} MB".format(peak_mib))
        if log is not None:
            log.at[(tag, "mem")] = peak_mib
    return result


def init_log(tags, metrics) -> pd.Series:
    """bench.py:52-57."""
    index = pd.MultiIndex.from_product([tags, metrics], names=["tag", "metric"])
    return pd.Series(np.zeros((len(tags) * len(metrics),)), index=index)


def mark_unavailable(log: pd.Series, tag: str) -> None:
    """A baseline whose library is not installed: every metric reads N/A."""
    for metric in log.index.levels[1]:
        log.at[(tag, metric)] = NOT_AVAILABLE


def empty_cache(func):
    """bench.py:60-64: release cached device memory before the wrapped run so
    that its peak is its own."""
    def wrapper(*args, **kwargs):
        torch.cuda.empty_cache()
        return func(*args, **kwargs)
    return wrapper


def dat_str(metric: str, log: pd.DataFrame) -> str:
    """The tab-separated table the reference's gnuplot templates read
    (plot.py:88-96): one header row "Dataset <tag>...", one row per dataset."""
    tags = list(log.index.levels[0])
    rows = ["\t".join(["Dataset"] + tags)]
    for dataset in log.columns:
        vals = [log[dataset][(tag, metric)] for tag in tags]
        rows.append("\t".join([dataset] + ["0.0" if v is None else str(v) for v in vals]))
    return "\n".join(rows) + "\n"


def save_logs(logs: dict, name: str, out_dir: str = "output") -> str:
    """{dataset: Series} -> ``<out_dir>/<name>.pkl`` (the DataFrame the
    reference pickles) plus ``<name>_time.dat`` / ``<name>_mem.dat`` tables."""
    os.makedirs(out_dir, exist_ok=True)
    frame = pd.DataFrame(logs)
    path = os.path.join(out_dir, name + ".pkl")
    frame.to_pickle(path)
    for metric in frame.index.levels[1]:
        with open(os.path.join(out_dir, "{}_{}.dat".format(name, metric)), "w") as f:
            f.write(dat_str(metric, frame))
    return path
