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
