"""Test infrastructure: restatement of the reference's epsilon search, probe for probe
(results/scripts/experiment/experiments.py): `within_percent` :74-84, `bound_epsilon` :153-195 (0 -> 2, then
doubling until the target selectivity is reached), `adjust_epsilon_binary` :198-225 (half the last step, back
after an overshoot, forward otherwise), `find_epsilon_binary` :228-281 (midpoint of the bounds, then half
steps until within 1 %).  The library's native search is checked against it; nothing shipped imports it.
Pinned by the sequences of probes the procedure fixes on a closed-form selectivity (tests/test_oracle.py)."""


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
