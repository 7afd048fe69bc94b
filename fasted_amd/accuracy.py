"""Pair-set accuracy metrics on numpy arrays of (query, candidate) pairs.

The quantities the reference's accuracy scripts report -- pairs on both sides / only in the truth list / only
in the tested list (results/scripts/compute_accuracy.py:70-130) and the per-point intersection over union
of neighbour sets (results/scripts/compute_accuracy_real_datasets.py:10-37) -- computed as set operations
on packed 64-bit keys instead of a merge walk over sorted files.
"""
from dataclasses import dataclass

import numpy as np


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
