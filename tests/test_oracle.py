"""Pins the CPU checker (oracle/fasted_oracle.c) against the golden vectors of the reference's own
data loader, the reference's closed-form test patterns and what the mathematics fixes."""
import ctypes
import json
import os

import numpy as np
import pytest

import oracle

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_loader.json")))


# ---------------------------------------------------------------- quantisation
def test_quantize_round_trips_every_half():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float64)
    finite = np.isfinite(vals)
    assert np.array_equal(oracle.quantize(vals[finite]), bits[finite])
    back = np.empty(finite.sum(), dtype=np.float64)
    oracle.lib().oracle_widen(bits[finite], int(finite.sum()), back)
    assert np.array_equal(back, vals[finite])


def test_quantize_matches_numpy_double_rounding():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(300000) * rng.choice([1e-8, 1e-6, 1e-4, 1e-2, 1.0, 100.0, 7e4], 300000)
    # exact ties between neighbouring halves, in the normal and the subnormal range
    h = np.arange(0, 0x7BFF, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = 0.5 * (h[:-1] + h[1:])
    x = np.concatenate([x, ties, -ties])
    with np.errstate(over="ignore"):
        want = x.astype(np.float32).astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.quantize(x), want)


def test_quantize_matches_reference_cast_value_golden():
    inputs = np.array(GOLDEN["cast_value"]["inputs"], dtype=np.float64)
    want = np.array(GOLDEN["cast_value"]["bits"], dtype=np.uint16)
    assert np.array_equal(oracle.quantize(inputs), want)


@pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref not built (no reference checkout)")
def test_quantize_matches_reference_half_hpp_live():
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.exponential(1 / 40.0, 20000), rng.standard_normal(20000) * 300, [65519.99, 65520.0, 1e-9]])
    ref = oracle.ref()
    want = np.array([ref.ref_cast_value(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(oracle.quantize(x), want)


# ---------------------------------------------------------------- seeded generator + padding
@pytest.mark.parametrize("case", GOLDEN["exponential"], ids=lambda c: c["name"])
def test_exponential_generator_matches_reference_golden(case):
    pts = oracle.exponential_points(case["n"], case["d"], case["lambda"], case["max"])
    assert pts.min() >= 0.0 and pts.max() <= case["max"]
    padded = oracle.build_padded(pts, case["dim_factor"], case["points_factor"])
    assert padded.shape == (case["n_pad"], case["d_pad"])
    assert np.array_equal(padded[: case["n"], : case["d"]], np.array(case["bits"], dtype=np.uint16))
    assert int(padded.sum()) - int(padded[: case["n"], : case["d"]].sum()) == case["padding_sum"] == 0


def test_known_first_points_of_the_reference_seed():
    # first two points of the seeded Exp(40) stream, dims 0-3, as FP16 bit patterns
    bits = oracle.quantize(oracle.exponential_points(5, 4, 40.0, 10.0))
    assert [hex(v) for v in bits[0]] == ["0x1c2f", "0x2dc3", "0x9ee", "0x2b3b"]
    assert [hex(v) for v in bits[1]] == ["0x2d04", "0x2539", "0x2846", "0x212a"]


@pytest.mark.skipif(not oracle.ref_available(), reason="oracle/_ref not built (no reference checkout)")
def test_exponential_generator_matches_reference_live():
    ref = oracle.ref()
    assert ref.ref_build_exponential(200, 96, 40.0, 1.0, 64, 768) == 0
    want = oracle.ref_values()
    got = oracle.build_padded(oracle.exponential_points(200, 96, 40.0, 1.0), 64, 768)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- squared norms
def test_sum_squared_closed_form_consecutive_integers():
    """tests/python/sumSquared/sumSquared.py of the reference: row r = 64 consecutive integers from
    64 r.  Sum_{v=a}^{a+63} v^2 in closed form; FP32 is exact while the sum stays below 2^24."""
    rows, d = 32, 64
    bits = oracle.quantize(np.arange(rows * d, dtype=np.float64).reshape(rows, d))  # < 2048: exact halves

    def closed(a):  # sum of squares a .. a+63
        f = lambda m: m * (m + 1) * (2 * m + 1) // 6
        return f(a + 63) - f(a - 1) if a > 0 else f(63)

    expect = np.array([closed(64 * r) for r in range(rows)], dtype=np.float64)
    assert np.array_equal(oracle.sum_squared(bits, "f64"), expect)
    exact_rows = expect < 2 ** 24
    assert exact_rows.sum() >= 6
    for mode in ("rz", "rn"):
        got = oracle.sum_squared(bits, mode).astype(np.float64)
        assert np.array_equal(got[exact_rows], expect[exact_rows])
        assert np.allclose(got, expect, rtol=d * 2.0 ** -24)


def test_sum_squared_round_toward_zero_invariants():
    rng = np.random.default_rng(5)
    bits = oracle.quantize(rng.exponential(1 / 40.0, (300, 512)))
    exact = oracle.sum_squared(bits, "f64")
    rz = oracle.sum_squared(bits, "rz").astype(np.float64)
    rn = oracle.sum_squared(bits, "rn").astype(np.float64)
    d = bits.shape[1]
    assert np.all(rz <= exact)  # truncation never overshoots a sum of non-negative terms
    assert np.all(exact - rz <= d * 2.0 ** -23 * exact)
    assert np.all(np.abs(rn - exact) <= d * 2.0 ** -24 * exact)
    assert np.any(rz < rn)  # the two rounding modes really differ


def test_sum_squared_odd_dimension_and_zero_row():
    bits = oracle.quantize(np.array([[3.0, 4.0, 12.0], [0.0, 0.0, 0.0]]))
    for mode in ("rz", "rn", "f64"):
        assert list(oracle.sum_squared(bits, mode)) == [169.0, 0.0]


# ---------------------------------------------------------------- reference rasterizer
def test_reference_rasterizer_is_a_permutation_with_8x8_locality():
    rows = cols = 24
    seen = {}
    for idx in range(rows * cols):
        rc = oracle.raster_coord(idx, rows, cols, 8, 96, 96)
        assert rc is not None and rc[0] % 96 == 0 and rc[1] % 96 == 0
        seen[idx] = (rc[0] // 96, rc[1] // 96)
    assert sorted(seen.values()) == [(r, c) for r in range(rows) for c in range(cols)]
    assert oracle.raster_coord(rows * cols, rows, cols, 8, 96, 96) is None
    for start in range(0, rows * cols, 64):  # 64 consecutive indices = one 8x8 square, row-major inside
        block = [seen[i] for i in range(start, start + 64)]
        r0, c0 = block[0]
        assert r0 % 8 == 0 and c0 % 8 == 0
        assert block == [(r0 + i // 8, c0 + i % 8) for i in range(64)]
    assert seen[64] == (0, 8) and seen[3 * 64] == (8, 0)  # squares advance along a row of squares first


# ---------------------------------------------------------------- pair buffer model
def test_pairs_get_space_overflow_semantics():
    lib = oracle.lib()
    found, stored = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    slots = [lib.oracle_pairs_get_space(ctypes.byref(found), ctypes.byref(stored), 5, 1) for _ in range(9)]
    assert slots == [0, 1, 2, 3, 4, -1, -1, -1, -1]
    assert (found.value, stored.value) == (9, 5)
    found, stored = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    # a request that does not fit entirely is dropped whole but still counted
    assert lib.oracle_pairs_get_space(ctypes.byref(found), ctypes.byref(stored), 5, 3) == 0
    assert lib.oracle_pairs_get_space(ctypes.byref(found), ctypes.byref(stored), 5, 3) == -1
    assert lib.oracle_pairs_get_space(ctypes.byref(found), ctypes.byref(stored), 5, 1) == -1
    assert (found.value, stored.value) == (7, 3)


# ---------------------------------------------------------------- joins
def brute_force_numpy(bits, eps):
    x = bits.view(np.float16).astype(np.float64)
    d2 = ((x[:, None, :] - x[None, :, :]) ** 2).sum(-1)
    q, c = np.nonzero(d2 <= eps * eps)
    return np.stack([q, c], axis=1).astype(np.int32)


def test_join_f64_equals_textbook_brute_force():
    rng = np.random.default_rng(1)
    bits = oracle.quantize(rng.random((150, 24)))
    for eps in (0.0, 1.2, 1.6, 10.0):
        got = oracle.self_join_f64(bits, eps)
        assert np.array_equal(got, brute_force_numpy(bits, eps))
    assert len(oracle.self_join_f64(bits, 0.0)) == 150  # eps = 0 keeps exactly the self pairs
    assert len(oracle.self_join_f64(bits, 10.0)) == 150 * 150


def test_join_is_symmetric_sorted_and_respects_padding():
    rng = np.random.default_rng(2)
    bits = oracle.quantize(rng.random((90, 16)))
    padded = np.vstack([bits, np.zeros((38, 16), dtype=np.uint16)])
    full = oracle.self_join_f64(bits, 0.9)
    assert np.array_equal(oracle.self_join_f64(padded, 0.9, n=90), full)  # padded zero rows are excluded
    key = full[:, 0].astype(np.int64) * 1000 + full[:, 1]
    assert np.all(np.diff(key) > 0)
    assert {tuple(p) for p in full} == {(c, q) for q, c in full}
    rows = oracle.self_join_f64(bits, 0.9, rows=(10, 30))
    assert np.array_equal(rows, full[(full[:, 0] >= 10) & (full[:, 0] < 30)])


def test_join_identity_fixture():
    """GenerateIdentityMatrixPoints (main.cu:113-131): unit vectors; distinct ones are sqrt(2) apart."""
    n = 48
    bits = np.eye(n, 64, dtype=np.float16).view(np.uint16)
    assert len(oracle.self_join_f64(bits, 1.0)) == n
    assert len(oracle.self_join_f64(bits, 1.42)) == n * n
    assert len(oracle.self_join_f32(bits, 1.0)) == n
    assert len(oracle.self_join_f32(bits, 1.42)) == n * n


def test_join_increasing_fixture_exact_in_fp32():
    """GenerateIncreasingPoints (main.cu:86-104) with small values: consecutive rows differ by d in
    every coordinate, so dist(i, j) = |i-j| * d * sqrt(d) exactly."""
    n, d = 20, 8
    bits = oracle.quantize(np.arange(n * d, dtype=np.float64).reshape(n, d))
    step = d * np.sqrt(d)
    for k in (0, 1, 3):
        eps = step * k + 0.5
        want = np.array([(i, j) for i in range(n) for j in range(n) if abs(i - j) <= k], dtype=np.int32)
        assert np.array_equal(oracle.self_join_f64(bits, eps), want)
        assert np.array_equal(oracle.self_join_f32(bits, eps), want)


def test_fp32_model_agrees_with_fp64_inside_the_band():
    bits = oracle.quantize(np.clip(np.random.default_rng(4).exponential(1 / 40.0, (600, 128)), 0, 1))
    from tests import datasets

    eps = datasets.epsilon_for_neighbours(bits, 12)
    model = oracle.self_join_f32(bits, eps)
    rep = oracle.epsilon_band_report(bits, model, eps)
    assert rep["outside_band"] == 0 and rep["both"] > 600
    # a deliberately wrong answer (one far pair added, one true pair removed) is caught
    truth = oracle.self_join_f64(bits, eps)
    d = oracle.pair_distances_f64(bits, truth)
    victim = int(np.argmin(np.where(truth[:, 0] != truth[:, 1], d, np.inf)))
    far = np.array([[0, int(np.argmax(oracle.pair_distances_f64(bits, np.stack([np.zeros(600, int), np.arange(600)], 1))))]])
    broken = oracle.sort_pairs(np.vstack([np.delete(truth, victim, axis=0), far]))
    rep = oracle.epsilon_band_report(bits, broken, eps)
    assert rep["outside_band"] == 2 and rep["got_only"] == 1 and rep["truth_only"] == 1


# ---------------------------------------------------------------- merge-walk pair statistics
def _five():
    return np.array([[1, 1], [2, 2], [3, 3], [4, 4], [5, 5]], dtype=np.int32)


def test_pair_distances_f64_against_numpy_and_closed_forms():
    """The distances the epsilon-band classifier judges disagreements by: the sum of squared differences in
    FP64 (exact on FP16 inputs up to FP64 rounding), against numpy on random pairs, and on pairs whose
    distance is known in closed form (a point with itself; unit vectors; a 3-4-5 triangle).  A swapped
    index, a missed square root or a distance formed from the expansion s_q + s_c - 2 q.c (which cancels)
    fails one of them."""
    rng = np.random.default_rng(21)
    n, d = 300, 77  # odd dimensionality: no padding column may be touched
    x = (rng.standard_normal((n, d)) * 3.0).astype(np.float16)
    bits = x.view(np.uint16)
    pairs = rng.integers(0, n, size=(5000, 2)).astype(np.int32)
    got = oracle.pair_distances_f64(bits, pairs)
    x64 = x.astype(np.float64)
    want = np.sqrt(((x64[pairs[:, 0]] - x64[pairs[:, 1]]) ** 2).sum(1))
    assert got.dtype == np.float64
    np.testing.assert_allclose(got, want, rtol=1e-14, atol=0.0)
    # not symmetric inputs by accident: (q, c) and (c, q) give the same distance, but different pairs do not
    np.testing.assert_array_equal(got, oracle.pair_distances_f64(bits, pairs[:, ::-1]))
    assert len(np.unique(got)) > 4000

    fix = np.zeros((5, 8), dtype=np.float16)
    fix[1, 0] = 1.0
    fix[2, 1] = 1.0
    fix[3, 0], fix[3, 1] = 3.0, 4.0
    fix[4] = 1000.0  # large norm: the expansion would lose the small difference to fix[4] itself
    fb = fix.view(np.uint16)
    closed = oracle.pair_distances_f64(fb, [(0, 0), (4, 4), (0, 1), (1, 2), (0, 3), (3, 0), (1, 3)])
    np.testing.assert_array_equal(closed[:2], [0.0, 0.0])
    np.testing.assert_allclose(closed[2:], [1.0, np.sqrt(2.0), 5.0, 5.0, np.sqrt(4.0 + 16.0)], rtol=1e-15)
    assert oracle.pair_distances_f64(fb, np.zeros((0, 2), dtype=np.int32)).shape == (0,)


@pytest.mark.parametrize("delete,side,expect", [
    # the cases of results/scripts/test_accuracy.py: (both, right_only, left_only, left_total, right_total)
    (None, None, (5, 0, 0, 5, 5)),
    ([0], "right", (4, 0, 1, 5, 4)),
    ([2], "right", (4, 0, 1, 5, 4)),
    ([4], "right", (4, 0, 1, 5, 4)),
    ([2, 3, 4], "right", (2, 0, 3, 5, 2)),
    ([0], "left", (4, 1, 0, 4, 5)),
    ([2], "left", (4, 1, 0, 4, 5)),
    ([4], "left", (4, 1, 0, 4, 5)),
])
def test_pair_stats_reference_cases(delete, side, expect):
    left, right = _five(), _five()
    if side == "right":
        right = np.delete(right, delete, axis=0)
    elif side == "left":
        left = np.delete(left, delete, axis=0)
    s = oracle.pair_stats(left, right)
    assert (s["both"], s["right_only"], s["left_only"], s["left_total"], s["right_total"]) == expect


def test_pair_stats_reports_the_one_sided_pairs():
    left = np.array([[0, 0], [0, 3], [1, 1], [2, 2]], dtype=np.int32)
    right = np.array([[0, 0], [1, 1], [1, 2], [2, 2], [9, 9]], dtype=np.int32)
    s, diff, side = oracle.pair_stats(left, right, want_diff=True)
    assert (s["both"], s["left_only"], s["right_only"]) == (3, 1, 2)
    assert diff.tolist() == [[0, 3], [1, 2], [9, 9]] and side.tolist() == [0, 1, 1]


# ---- the CPU baseline (oracle/blocked_join.c): a blocked GEMM-form join, pinned against the checker
def _vector_widths():
    native = oracle.blocked_join_vector_bits()
    return [256, 512] if native == 512 else [256]


@pytest.mark.parametrize("nq,nc,d", [(1, 1, 1), (7, 129, 3), (200, 333, 64), (1537, 257, 300), (50, 1000, 520)])
def test_blocked_join_equals_the_checker(nq, nc, d):
    """Ragged in every blocking direction (6-row panels, 128-candidate blocks, 256-wide K slices, 1536-row query
    blocks).  Integer coordinates make both forms exact, so FP64 and FP32, 256- and 512-bit, must give exactly the
    checker's list; indices carry the offsets handed in."""
    from tests import datasets

    bits = datasets.small_integers(nq + nc, d, high=3, seed=nq + nc + d)
    x = bits.view(np.float16).astype(np.float64)
    d2 = ((x[: min(nq + nc, 48), None, :] - x[None, : min(nq + nc, 48), :]) ** 2).sum(-1)
    eps = float(np.sqrt(np.median(d2) + 0.5))
    truth = oracle.self_join_f64(bits, eps)
    want = truth[(truth[:, 0] < nq) & (truth[:, 1] >= nq)]
    native = oracle.blocked_join_vector_bits()
    try:
        for width in _vector_widths():
            oracle.blocked_join_vector_bits(width)
            for precision in (64, 32):
                got, found, secs = oracle.blocked_join(bits[:nq], bits[nq:], eps, precision, q_offset=0, c_offset=nq)
                assert found == len(want) and np.array_equal(got, want), (width, precision)
                assert secs >= 0.0
                _, count_only, _ = oracle.blocked_join(bits[:nq], bits[nq:], eps, precision, want_pairs=False)
                assert count_only == len(want)
    finally:
        oracle.blocked_join_vector_bits(native)


def test_blocked_join_on_real_valued_data_stays_inside_the_band():
    """Exp(40) data: the GEMM form in FP64 agrees with the difference-form checker pair for pair; in FP32 every
    disagreement lies inside the relative 1e-3 band (count and largest error printed)."""
    from tests import datasets

    n, d = 1500, 192
    bits = datasets.exponential(n, d, seed=5)
    eps = datasets.epsilon_for_neighbours(bits, 20)
    truth = oracle.self_join_f64(bits, eps)
    got64, found64, _ = oracle.blocked_join(bits, bits, eps, 64)
    rep64 = oracle.epsilon_band_report(bits, got64, eps, truth_pairs=truth, band=1e-9)
    assert rep64["outside_band"] == 0, rep64
    got32, found32, _ = oracle.blocked_join(bits, bits, eps, 32)
    rep32 = oracle.epsilon_band_report(bits, got32, eps, truth_pairs=truth)
    assert rep32["outside_band"] == 0, rep32
    assert {(i, i) for i in range(n)} <= {tuple(p) for p in got32}
    print("blocked join vs checker:", rep64, rep32)
