"""Test infrastructure: restatement of the reference's epsilon search, probe for probe
(results/scripts/experiment/experiments.py): `within_percent` :74-84, `bound_epsilon` :153-195 (0 -> 2, then
doubling until the target selectivity is reached), `adjust_epsilon_binary` :198-225 (half the last step, back
after an overshoot, forward otherwise), `find_epsilon_binary` :228-281 (midpoint of the bounds, then half
steps until within 1 %); `compute_gamma` :87-96, `adjust_epsilon_volume` :99-150 (ball volumes in decimal
arithmetic) and `find_epsilon_volumetric` :284-323 (here the adjusted epsilon is probed; the reference's loop
probes the initial one again, :314, and cannot end).  The library's native searches are checked against them;
nothing shipped imports this file.
Pinned by the sequences of probes the procedures fix on closed-form selectivities (tests/test_oracle.py)."""
import math
from decimal import Decimal


def within_percent(actual, target, percent):
    return abs(actual - target) / target < percent


def bound_epsilon(initial, maximum, target, selectivity_of):
    lower = upper = initial
    current = 0
    while current < target:
        lower = upper
        upper = 2.0 if lower == 0 else lower * 2.0
        if upper > maximum:
            raise ValueError(f"Epsilon of {upper} exceed the maximum value of {maximum}. "
                             "Giving up trying to find the upper bound.")
        current = selectivity_of(upper)
    return lower, upper


def adjust_epsilon_binary(current, last, target, actual):
    step = abs(current - last)
    return current - 0.5 * step if actual > target else current + 0.5 * step


def find_epsilon_binary(target, selectivity_of, initial=0.0, max_iterations=200):
    lower, upper = bound_epsilon(initial, 100000, target, selectivity_of)
    eps, last = (upper - lower) / 2.0 + lower, upper
    current = selectivity_of(eps)
    for _ in range(max_iterations):
        if within_percent(current, target, 0.01):
            return eps
        eps, last = adjust_epsilon_binary(eps, last, target, current), eps
        current = selectivity_of(eps)
    raise RuntimeError("epsilon search did not converge to within 1% of the target selectivity")


def compute_gamma(dims):
    return Decimal(math.lgamma(dims / 2.0 + 1)).exp()


def adjust_epsilon_volume(epsilon, selectivity, target, dims):
    if selectivity == 0:
        return epsilon * 2.0
    d, pi, gamma = Decimal(dims), Decimal(math.pi), compute_gamma(dims)
    unit_ball = (pi ** (d / Decimal(2.0))) / gamma
    old_volume = unit_ball * Decimal(epsilon) ** d
    target_volume = (Decimal(target) / Decimal(selectivity)) * old_volume
    return float(((target_volume * gamma) / (pi ** (dims / Decimal(2.0)))) ** (Decimal(1.0) / d))


def find_epsilon_volumetric(dims, target, selectivity_of, initial=0.1, max_iterations=200):
    eps = initial
    current = selectivity_of(eps)
    for _ in range(max_iterations):
        if within_percent(current, target, 0.1):
            return eps
        eps = adjust_epsilon_volume(eps, current, target, dims)
        current = selectivity_of(eps)
    raise RuntimeError("volumetric epsilon search did not converge to within 10% of the target selectivity")
