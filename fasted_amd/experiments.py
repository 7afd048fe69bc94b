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


# ---- the reference runner's names ------------------------------------------------------------------------
# Scripts written against results/scripts/experiment/experiments.py (run_experiments.py of the reference builds
# an ``ExperimentRunner(load_findpairs())`` and calls the methods below) keep working on this package: same
# class, method and argument names, same result files.  Everything is carried out by a ``SweepDriver`` over a
# backend that wraps the object handed in -- the loaded library or a mock with the same three methods
# (``runFromExponentialDataset``, ``runFromFile``, ``reRun``; results/scripts/tests/test_experiments.py:14-71).
from dataclasses import dataclass  # noqa: E402


@dataclass
class SearchParameters:
    """One timed configuration (experiments.py:58-64)."""
    target_selectivity: float
    epsilon: float
    save_pairs: bool


@dataclass
class Experiment:
    """One result record (experiments.py:67-73)."""
    selectivity: float
    epsilon: float
    iteration: int
    results: object


class ResultsEncoder(json.JSONEncoder):
    """Writes ``Experiment`` records and ``Results`` structures as the reference's files hold them."""

    def default(self, obj):
        if isinstance(obj, Experiment):
            return {"selectivity": obj.selectivity, "epsilon": obj.epsilon, "iteration": obj.iteration,
                    "results": results_record(obj.results)}
        if hasattr(obj, "pairsFound") and hasattr(obj, "inputProblemShape"):
            return results_record(obj)
        return super().default(obj)


def find_epsilon_binary(target_selectivity, get_selectivity, initial_epsilon=0.0):
    """Epsilon whose selectivity lies within 1 % of the target, for any ``get_selectivity(epsilon)`` callable:
    the procedure of the library's native search (``fasted_find_epsilon``), which is the reference's
    (experiments.py:228-281) -- double from the initial epsilon (0 -> 2) until the target is passed, then half
    steps -- with its guard against a plateau."""
    low = high = float(initial_epsilon)
    seen = 0.0
    while seen < target_selectivity:
        low, high = high, (2.0 if high == 0.0 else 2.0 * high)
        if high > 100000.0:
            raise ValueError(f"no epsilon up to 100000 reaches a selectivity of {target_selectivity}")
        seen = get_selectivity(high)
    previous, epsilon = high, 0.5 * (low + high)
    seen = get_selectivity(epsilon)
    for _ in range(200):
        if abs(seen - target_selectivity) / target_selectivity < 0.01:
            return epsilon
        half_step = 0.5 * abs(epsilon - previous)
        previous, epsilon = epsilon, (epsilon - half_step if seen > target_selectivity else epsilon + half_step)
        if epsilon == previous:
            break
        seen = get_selectivity(epsilon)
    raise ValueError("epsilon search did not converge to within 1% of the target selectivity")


class _CallableBackend:
    """Backend over the three entry points of a pair-finding object (the loaded library or a mock)."""

    def __init__(self, find_pairs):
        self._fp = find_pairs
        self._first = None  # the loading call that a run on fresh data makes

    def load_exponential(self, size, dim, lam=40.0, value_range=10.0):
        self._first = lambda eps, save: self._fp.runFromExponentialDataset(int(size), int(dim), lam, value_range, eps, save)

    def load_file(self, path):
        self._first = lambda eps, save: self._fp.runFromFile(str(path).encode("utf-8"), eps, save)

    def run(self, epsilon, save_pairs=False):
        first, self._first = self._first, None
        return first(epsilon, save_pairs) if first else self._fp.reRun(epsilon, save_pairs)

    def epsilon_for(self, target, sample_rows=None):
        probes = []

        def selectivity(eps):
            probes.append(eps)
            return self.run(eps, False).get_selectivity()

        eps = find_epsilon_binary(target, selectivity)
        return eps, selectivity(eps), len(probes)


class ExperimentRunner:
    """The reference's runner (experiments.py:341-591) by name; the work is a ``SweepDriver``'s."""

    def __init__(self, find_pairs, output_dir="."):
        self._find_pairs = find_pairs
        self._driver = SweepDriver(_CallableBackend(find_pairs), output_dir)

    def get_selectivity_rerun(self, epsilon):
        return self._find_pairs.reRun(epsilon, False).get_selectivity()

    def run_time_trials(self, find_pairs, search_params, iterations):
        out = []
        for p in search_params:
            for i in range(iterations):
                try:
                    out.append(Experiment(p.target_selectivity, p.epsilon, i, find_pairs(p.epsilon, p.save_pairs and i == 0)))
                except Exception as e:  # noqa: BLE001
                    print(f"Failed to run iteration {i}. {e}")
        return out

    def run_selectivity_experiment(self, selectivities, find_pairs, iterations=3, save_pairs=False):
        out = []
        for target in selectivities:
            eps = find_epsilon_binary(target, lambda e: find_pairs(e, False).get_selectivity())
            out += self.run_time_trials(find_pairs, [SearchParameters(target, eps, save_pairs)], iterations)
        return out

    def build_file_pairs_finder(self, base_path, dataset):
        path = str(Path(base_path) / dataset).encode("utf-8")
        return lambda epsilon, save_pairs: self._find_pairs.runFromFile(path, epsilon, save_pairs)

    def build_rerunnable_file_pairs_finder(self, base_path, dataset):
        return fp.RerunnablePairsFinder(self.build_file_pairs_finder(base_path, dataset), self._find_pairs.reRun)

    def run_real_dataset_known_epsilons_experiments(self, dataset_path, dataset, search_params, num_repetitions=3):
        runs = [(p.target_selectivity, p.epsilon) for p in search_params]
        save = any(p.save_pairs for p in search_params)
        return self._driver.file_runs(Path(dataset_path) / dataset, runs, num_repetitions, save, prefix=f"{dataset}_results")

    def run_real_datasets_epsilon_finder_experiments(self, target_selectivities, base_path=".", datasets=()):
        """The reference lists its datasets and their directory in the method body (experiments.py:497-508);
        here they are arguments."""
        return self._driver.file_epsilon_search([Path(base_path) / d for d in datasets], target_selectivities)

    def run_selectivity_vs_speed_experiment(self, target_selectivities):
        return self._driver.selectivity_sweep(target_selectivities)

    def run_speed_sweeps_exponential_data_experiment(self):
        return self._driver.exponential_sweep()
