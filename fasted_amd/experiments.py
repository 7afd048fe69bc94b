"""Epsilon search and accuracy metrics, mirroring the reference's experiment helpers.

Same names and behaviour as results/scripts/experiment/experiments.py (`within_percent` :74-84,
`bound_epsilon` :153-195, `adjust_epsilon_binary` :198-225, `find_epsilon_binary` :228-281) and as the
accuracy scripts (`compute_pair_stats`, results/scripts/compute_accuracy.py:70-130; per-point
intersection-over-union, results/scripts/compute_accuracy_real_datasets.py:10-37), so drivers written
against the reference run on this package.  `get_selectivity` is any callable epsilon -> selectivity,
e.g. ``lambda e: fasted_amd.compute_selectivity(fasted_amd.count_pairs(e)[0], n)``.
"""
from dataclasses import dataclass
from typing import Callable, Tuple

import numpy as np


def within_percent(actual_value: float, target_value: float, percent: float) -> bool:
    return (abs(actual_value - target_value) / target_value) < percent


def bound_epsilon(initial_epsilon: float, max_epsilon: float, target_selectivity: float,
                  get_selectivity: Callable[[float], float]) -> Tuple[float, float]:
    """Doubles epsilon (0 -> 2) until the target selectivity is reached; returns (lower, upper)."""
    current_selectivity = 0
    new_epsilon = initial_epsilon
    old_epsilon = initial_epsilon
    while current_selectivity < target_selectivity:
        old_epsilon = new_epsilon
        new_epsilon = 2.0 if old_epsilon == 0 else old_epsilon * 2.0
        if new_epsilon > max_epsilon:
            raise ValueError(f"Epsilon of {new_epsilon} exceed the maximum value of {max_epsilon}. "
                             "Giving up trying to find the upper bound.")
        current_selectivity = get_selectivity(new_epsilon)
    return (old_epsilon, new_epsilon)


def adjust_epsilon_binary(current_epsilon: float, last_epsilon: float, target_selectivity: float,
                          actual_selectivity: float) -> float:
    """Half a step back after an overshoot, half a step forward otherwise."""
    last_step = abs(current_epsilon - last_epsilon)
    if actual_selectivity > target_selectivity:
        return current_epsilon - (0.5 * last_step)
    return current_epsilon + (0.5 * last_step)


def find_epsilon_binary(target_selectivity: float, get_selectivity: Callable[[float], float],
                        initial_epsilon: float = 0.0, max_iterations: int = 200) -> float:
    """Bound, then bisect until the selectivity is within 1 % of the target."""
    lower_epsilon, upper_epsilon = bound_epsilon(initial_epsilon, 100000, target_selectivity, get_selectivity)
    new_epsilon = ((upper_epsilon - lower_epsilon) / 2.0) + lower_epsilon
    last_epsilon = upper_epsilon
    current_selectivity = get_selectivity(new_epsilon)
    iteration = 0
    while not within_percent(current_selectivity, target_selectivity, 0.01):
        iteration += 1
        if iteration > max_iterations:
            raise RuntimeError("epsilon search did not converge to within 1% of the target selectivity")
        new_epsilon, last_epsilon = (
            adjust_epsilon_binary(new_epsilon, last_epsilon, target_selectivity, current_selectivity), new_epsilon)
        current_selectivity = get_selectivity(new_epsilon)
    return new_epsilon


@dataclass
class PairsStats:
    both_sides: int = 0
    right_only: int = 0
    left_only: int = 0
    total_test_pairs: int = 0
    total_truth_pairs: int = 0


def _keys(pairs) -> np.ndarray:
    p = np.asarray(pairs).reshape(-1, 2).astype(np.int64)
    return (p[:, 0] << 32) | p[:, 1]


def compute_pair_stats(test_pairs, truth_pairs) -> PairsStats:
    """Pairs in both lists, only in the truth (right) list, only in the test (left) list."""
    left, right = np.unique(_keys(test_pairs)), np.unique(_keys(truth_pairs))
    both = int(np.intersect1d(left, right, assume_unique=True).size)
    return PairsStats(both, int(right.size) - both, int(left.size) - both, int(len(np.asarray(test_pairs).reshape(-1, 2))),
                      int(len(np.asarray(truth_pairs).reshape(-1, 2))))


def per_point_iou(test_pairs, truth_pairs, num_points: int) -> np.ndarray:
    """Intersection over union of each point's neighbour set in the two pair lists (1.0 when both
    are empty)."""
    left, right = np.unique(_keys(test_pairs)), np.unique(_keys(truth_pairs))
    inter = np.intersect1d(left, right, assume_unique=True)
    cnt = lambda k: np.bincount((k >> 32).astype(np.int64), minlength=num_points)[:num_points]
    i, l, r = cnt(inter), cnt(left), cnt(right)
    union = l + r - i
    return np.where(union > 0, i / np.maximum(union, 1), 1.0)


# ---------------------------------------------------------------------------------------------
# Experiment driver: same class and method names, same JSON records as the reference's
# results/scripts/experiment/experiments.py:42-73,328-591, so its result files
# (results/speed_results/*.json) and the scripts that read them keep working.  `find_pairs` is the
# loaded library (fasted_amd.load_findpairs()) or any object with runFromExponentialDataset /
# runFromFile / reRun.  Differences: result files go to `output_dir` (default: the current directory)
# instead of the script's directory, and the sweep ranges are arguments with the reference's values
# as defaults.
import ctypes  # noqa: E402
import json  # noqa: E402
import time  # noqa: E402
from pathlib import Path  # noqa: E402

from .find_pairs import RerunnablePairsFinder, Results  # noqa: E402


def generate_unique_filename(prefix: str, file_type: str) -> str:
    return f"{prefix}_{int(time.time())}{file_type}"


@dataclass
class SearchParameters:
    target_selectivity: float
    epsilon: float
    save_pairs: bool


@dataclass
class Experiment:
    selectivity: float
    epsilon: float
    iteration: int
    results: Results


class ResultsEncoder(json.JSONEncoder):
    """ctypes structures and Experiment records as plain dictionaries."""

    def default(self, o):
        if isinstance(o, ctypes.Structure):
            return {name: getattr(o, name) for name, *_ in o._fields_}
        if isinstance(o, Experiment):
            return dict(o.__dict__)
        return super().default(o)


def save_json_results(filename: str, results, output_dir: str = ".") -> str:
    path = Path(output_dir) / generate_unique_filename(filename, ".json")
    with open(path, "w", encoding="utf-8") as f:
        json.dump(results, f, cls=ResultsEncoder)
    return str(path)


class ExperimentRunner:
    def __init__(self, find_pairs, output_dir: str = "."):
        self._find_pairs = find_pairs
        self._output_dir = output_dir

    def get_selectivity_rerun(self, epsilon: float) -> float:
        return self._find_pairs.reRun(epsilon, False).get_selectivity()

    def run_time_trials(self, find_pairs: Callable[[float, bool], Results], search_params, iterations: int):
        """`iterations` runs per parameter set; pairs are saved on the first run only; a run that fails
        is reported and skipped."""
        results = []
        for param in search_params:
            for i in range(iterations):
                try:
                    results.append(Experiment(param.target_selectivity, param.epsilon, i,
                                              find_pairs(param.epsilon, param.save_pairs and i == 0)))
                except Exception as e:  # noqa: BLE001 -- the reference carries on after any failure
                    print(f"Failed to run iteration {i}. {e}")
        return results

    def run_selectivity_experiment(self, selectivities, find_pairs: Callable[[float, bool], Results],
                                   iterations: int = 3, save_pairs: bool = False):
        """Finds the epsilon of every target selectivity (bound, then bisect), then times each."""
        search_params = [
            SearchParameters(s, find_epsilon_binary(s, lambda e: find_pairs(e, False).get_selectivity()), save_pairs)
            for s in selectivities
        ]
        return self.run_time_trials(find_pairs, search_params, iterations)

    def build_file_pairs_finder(self, base_path: str, dataset: str) -> Callable[[float, bool], Results]:
        name = str(Path(base_path) / dataset).encode("utf-8")
        return lambda epsilon, save_pairs: self._find_pairs.runFromFile(name, epsilon, save_pairs)

    def build_rerunnable_file_pairs_finder(self, base_path: str, dataset: str) -> Callable[[float, bool], Results]:
        """Reads and uploads the file once; later calls only change epsilon (not for time trials)."""
        return RerunnablePairsFinder(self.build_file_pairs_finder(base_path, dataset), self._find_pairs.reRun)

    def run_real_dataset_known_epsilons_experiments(self, dataset_path: str, dataset: str, search_params,
                                                    num_repetitions: int = 3) -> str:
        print(f"Running on dataset: {dataset}")
        finder = self.build_file_pairs_finder(dataset_path, dataset)  # from scratch every time: honest timings
        results = self.run_time_trials(finder, search_params, num_repetitions)
        return save_json_results(f"{dataset}_results", results, self._output_dir)

    def run_real_datasets_epsilon_finder_experiments(self, target_selectivities, base_path: str = ".",
                                                     datasets=("cifar60k_unscaled.txt",)) -> str:
        results = {}
        for dataset in datasets:
            print(f"Running on dataset: {dataset}")
            finder = self.build_rerunnable_file_pairs_finder(base_path, dataset)
            results[dataset] = self.run_selectivity_experiment(target_selectivities, finder, iterations=1)
        return save_json_results("realDatasets", results, self._output_dir)

    def run_selectivity_vs_speed_experiment(self, target_selectivities, size: int = 100000, dim: int = 4096) -> str:
        finder = RerunnablePairsFinder(
            lambda epsilon, save_pairs: self._find_pairs.runFromExponentialDataset(size, dim, 40, 10, epsilon,
                                                                                   save_pairs),
            self._find_pairs.reRun)
        results = self.run_selectivity_experiment(target_selectivities, finder)
        return save_json_results("selectivityVsSpeed", results, self._output_dir)

    def run_speed_sweeps_exponential_data_experiment(self, sizes=None, dims=None, epsilon: float = 0.001,
                                                     iterations: int = 3) -> str:
        """Size x dimensionality sweep on the seeded exponential data at a fixed epsilon (default: 10
        sizes from 1e3 to 1e6, log-spaced, and D = 64, 128, ... 4096, as the reference)."""
        sizes = [round(s) for s in np.logspace(3, 6, 10)] if sizes is None else list(sizes)
        dims = [64 << k for k in range(7)] if dims is None else list(dims)
        results = []
        for size in sizes:
            for dim in dims:
                finder = RerunnablePairsFinder(
                    lambda eps, save, size=size, dim=dim: self._find_pairs.runFromExponentialDataset(
                        size, dim, 40, 10, eps, save),
                    self._find_pairs.reRun)
                results += self.run_time_trials(finder, [SearchParameters(0, epsilon, False)], iterations)
        return save_json_results("ExpoDataSpeedVsSize", results, self._output_dir)
