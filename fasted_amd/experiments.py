"""Timing and selectivity experiments on the library's native entry points.

What the reference's Python runner does with one full join per probe (results/scripts/experiment/
experiments.py: epsilon search :153-281, time trials and sweeps :341-591) is driven here from the library
itself: the dataset is built and uploaded once (``fasted_load_*``), the epsilon of a target selectivity comes
from the native search on count-only probes (``fasted_find_epsilon`` / ``fasted_find_epsilon_sampled``), and
only the timed runs are real ``reRun`` calls.  The result files keep the reference's record layout
(``results/speed_results/*.json``: ``selectivity``, ``epsilon``, ``iteration``, ``results`` = the fields of
``Results``) and its ``<prefix>_<unix time>.json`` names, so its plotting scripts read them unchanged.

A backend is any object with ``load_exponential(size, dim, lam, value_range)``, ``load_file(path)``,
``run(epsilon, save_pairs) -> Results`` and ``epsilon_for(target, sample_rows) -> (epsilon, selectivity,
probes)``; ``LibraryBackend`` is the real one.
"""
import json
import time
from pathlib import Path

from . import find_pairs as fp


class LibraryBackend:
    """The loaded libfasted.so: one resident dataset at a time."""

    def __init__(self, lib=None):
        self._lib = lib or fp.load_findpairs()

    def _check(self, rc):
        if rc != 0:
            raise fp.FastedError(self._lib.fasted_last_error().decode())

    def load_exponential(self, size, dim, lam=40.0, value_range=10.0):
        self._check(self._lib.fasted_load_exponential_dataset(int(size), int(dim), float(lam), float(value_range)))

    def load_file(self, path):
        self._check(self._lib.fasted_load_file(str(path).encode("utf-8")))

    def run(self, epsilon, save_pairs=False):
        return self._lib.reRun(float(epsilon), bool(save_pairs))

    def epsilon_for(self, target, sample_rows=None):
        if sample_rows:
            return fp.find_epsilon_sampled(target, sample_rows=sample_rows)
        return fp.find_epsilon(target)


def results_record(res) -> dict:
    """The fields of a ``Results`` structure as the plain dictionary the result files hold."""
    shape = lambda s: {"m": s.m, "n": s.n, "k": s.k}
    return {"totalTime": res.totalTime, "TFLOPS": res.TFLOPS, "pairsFound": res.pairsFound,
            "pairsStored": res.pairsStored, "inputProblemShape": shape(res.inputProblemShape),
            "paddedProblemShape": shape(res.paddedProblemShape)}


class SweepDriver:
    def __init__(self, backend=None, output_dir="."):
        self.backend = backend or LibraryBackend()
        self.output_dir = Path(output_dir)

    # ---- building blocks -------------------------------------------------------------------------
    def timed_runs(self, selectivity, epsilon, repetitions=3, save_pairs=False):
        """``repetitions`` joins of the resident dataset at one epsilon; pairs are saved by the first one
        only; a run that raises is reported and left out (the sweep goes on)."""
        records = []
        for i in range(repetitions):
            try:
                res = self.backend.run(epsilon, save_pairs and i == 0)
            except Exception as e:  # noqa: BLE001 -- one failed run must not end a sweep of hours
                print(f"run {i} at epsilon {epsilon} failed: {e}")
                continue
            records.append({"selectivity": selectivity, "epsilon": epsilon, "iteration": i,
                            "results": results_record(res)})
        return records

    def write(self, prefix, records) -> str:
        path = self.output_dir / f"{prefix}_{int(time.time())}.json"
        with open(path, "w", encoding="utf-8") as f:
            json.dump(records, f)
        return str(path)

    # ---- the reference's experiments -------------------------------------------------------------
    def exponential_sweep(self, sizes=None, dims=None, epsilon=0.001, repetitions=3, prefix="ExpoDataSpeedVsSize") -> str:
        """Size x dimensionality grid on the seeded Exp(40) data at a fixed epsilon (default grid: 10 sizes
        from 1e3 to 1e6, log-spaced, x D = 64 ... 4096: experiments.py:550-591)."""
        if sizes is None:
            sizes = [round(10 ** (3 + 3 * i / 9)) for i in range(10)]
        if dims is None:
            dims = [64 << k for k in range(7)]
        records = []
        for size in sizes:
            for dim in dims:
                self.backend.load_exponential(size, dim)
                records += self.timed_runs(0, epsilon, repetitions)
        return self.write(prefix, records)

    def selectivity_sweep(self, targets, size=100000, dim=4096, repetitions=3, sample_rows=None,
                          prefix="selectivityVsSpeed") -> str:
        """Speed against selectivity on one exponential dataset (experiments.py:519-547): the epsilon of every
        target from the native search, then the timed runs."""
        self.backend.load_exponential(size, dim)
        records = []
        for target in targets:
            epsilon, _, _ = self.backend.epsilon_for(target, sample_rows)
            records += self.timed_runs(target, epsilon, repetitions)
        return self.write(prefix, records)

    def file_runs(self, path, epsilons, repetitions=3, save_pairs=False, prefix=None) -> str:
        """Timed runs of a CSV dataset at known (selectivity, epsilon) pairs (experiments.py:430-470)."""
        self.backend.load_file(path)
        records = []
        for selectivity, epsilon in epsilons:
            records += self.timed_runs(selectivity, epsilon, repetitions, save_pairs)
        return self.write(prefix or f"{Path(path).name}_results", records)

    def file_epsilon_search(self, paths, targets, sample_rows=None, prefix="realDatasets") -> str:
        """For every CSV dataset the epsilon of every target selectivity and one timed run at it
        (experiments.py:473-516); the file holds one record list per dataset name."""
        by_dataset = {}
        for path in paths:
            self.backend.load_file(path)
            records = []
            for target in targets:
                epsilon, _, _ = self.backend.epsilon_for(target, sample_rows)
                records += self.timed_runs(target, epsilon, 1)
            by_dataset[Path(path).name] = records
        return self.write(prefix, by_dataset)
