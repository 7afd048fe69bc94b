"""CPU-side tests of the shipped library: every symbol of include/fasted.h is exported, the
`Results` layout matches the reference's ctypes mirror, the host data path reproduces the
reference's datasets, and the host mirror of the tile queues covers every tile exactly once.
No compute entry point is called here (there is no GPU and no CPU fallback)."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

import fasted_amd
import oracle
from fasted_amd import find_pairs as fp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")
GOLDEN = json.load(open(os.path.join(GOLDEN_DIR, "reference_loader.json")))


@pytest.fixture(scope="module")
def lib():
    return fasted_amd.load_findpairs()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "fasted.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{]*\)\s*;", text)
    return sorted(set(names))


def test_every_declared_symbol_is_exported(lib):
    names = declared_functions()
    assert {"runFromExponentialDataset", "runFromFile", "reRun", "releaseResources", "fasted_self_join",
            "fasted_self_join_device", "fasted_sum_squared_device"} <= set(names)
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/fasted.h but not exported"


def test_results_layout_matches_the_reference_mirror():
    # results/scripts/experiment/find_pairs.py:24-44 of the reference: 56 bytes, same offsets
    assert ctypes.sizeof(fp.mmaShape) == 12
    assert ctypes.sizeof(fp.Results) == 56
    offs = {n: getattr(fp.Results, n).offset for n, _ in fp.Results._fields_}
    assert offs == {"totalTime": 0, "TFLOPS": 8, "pairsFound": 16, "pairsStored": 24, "inputProblemShape": 32,
                    "paddedProblemShape": 44}
    assert ctypes.sizeof(fp.FastedPair) == 8
    assert lib_signature_ok()


def lib_signature_ok():
    lib = fasted_amd.load_findpairs()
    return (lib.runFromExponentialDataset.restype is fp.Results and lib.reRun.restype is fp.Results
            and lib.runFromFile.argtypes == [ctypes.c_char_p, ctypes.c_double, ctypes.c_bool])


def test_selectivity_and_rerunnable_finder_follow_the_reference():
    assert fp.compute_selectivity(300, 100) == 2.0
    assert fp.compute_selectivity(50, 100) == 0.0  # never negative
    r = fp.Results(pairsFound=1100, inputProblemShape=fp.mmaShape(100, 100, 8))
    assert r.get_selectivity() == 10.0
    calls = []
    finder = fp.RerunnablePairsFinder(lambda e, s: calls.append(("first", e, s)) or "A",
                                      lambda e, s: calls.append(("rerun", e, s)) or "B")
    assert [finder(0.1), finder(0.2, True), finder(0.3)] == ["A", "B", "B"]
    assert calls == [("first", 0.1, False), ("rerun", 0.2, True), ("rerun", 0.3, False)]


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(OSError):
        fasted_amd.load_findpairs(str(tmp_path / "nope.so"))


# ---------------------------------------------------------------- host data path
@pytest.mark.parametrize("case", GOLDEN["exponential"], ids=lambda c: c["name"])
def test_exponential_dataset_equals_reference_golden(lib, case):
    assert lib.fasted_load_exponential_dataset(case["n"], case["d"], case["lambda"], case["max"]) == 0
    bits, n, d, name = fasted_amd.resident_points()
    assert (n, d, name) == (case["n"], case["d"], case["name"])
    assert bits.shape[1] == case["d_pad"] and bits.shape[0] % 256 == 0 and bits.shape[0] >= n
    assert np.array_equal(bits[:n, :d], np.array(case["bits"], dtype=np.uint16))
    assert bits[n:].sum() == 0 and bits[:, d:].sum() == 0


def test_exponential_dataset_equals_oracle_on_a_larger_case(lib):
    assert lib.fasted_load_exponential_dataset(700, 200, 40.0, 10.0) == 0
    bits, n, d, _ = fasted_amd.resident_points()
    assert np.array_equal(bits[:n, :d], oracle.quantize(oracle.exponential_points(700, 200, 40.0, 10.0)))


@pytest.mark.parametrize("n,d,lam,mx", [(3000, 400, 40.0, 10.0), (5000, 333, 10.0, 0.05), (2049, 1000, 40.0, 0.02)])
def test_exponential_dataset_built_by_several_threads(lib, n, d, lam, mx, monkeypatch):
    """Above 2^20 values the dataset is built by an engine thread and converter threads; the result is
    the sequential generator's, value for value, also when most candidates are rejected (second and
    third case: 61 % and 45 % fall outside [0, max]) and when rows straddle the blocks."""
    want = oracle.quantize(oracle.exponential_points(n, d, lam, mx))
    for threads in ("1", "3", "8"):
        monkeypatch.setenv("FASTED_GEN_THREADS", threads)
        assert lib.fasted_load_exponential_dataset(n, d, lam, mx) == 0
        bits, got_n, got_d, name = fasted_amd.resident_points()
        assert (got_n, got_d) == (n, d) and name == "Exponential_%d_%d_%f" % (n, d, lam)
        assert np.array_equal(bits[:n, :d], want), threads
        assert bits[n:].sum() == 0 and bits[:, d:].sum() == 0


def test_csv_dataset_equals_reference_golden(lib):
    g = GOLDEN["csv"]
    assert lib.fasted_load_file(os.path.join(GOLDEN_DIR, g["file"]).encode()) == 0
    bits, n, d, name = fasted_amd.resident_points()
    assert (n, d, name, bits.shape[1]) == (g["n"], g["d"], g["name"], g["d_pad"])
    assert np.array_equal(bits[:n, :d], np.array(g["bits"], dtype=np.uint16))
    # the same values through the checker's quantiser
    vals = np.loadtxt(os.path.join(GOLDEN_DIR, g["file"]), delimiter=",")
    with np.errstate(over="ignore"):
        assert np.array_equal(bits[:n, :d], oracle.quantize(vals))


def test_csv_error_paths(lib, tmp_path):
    assert lib.fasted_load_file(str(tmp_path / "missing.csv").encode()) != 0
    assert b"Failed to open file" in lib.fasted_last_error()
    ragged = tmp_path / "ragged.csv"
    ragged.write_text("1,2,3\n4,5\n")
    assert lib.fasted_load_file(str(ragged).encode()) != 0
    assert lib.fasted_last_error().decode() == GOLDEN["ragged_error"]
    empty = tmp_path / "empty.csv"
    empty.write_text("")
    assert lib.fasted_load_file(str(empty).encode()) != 0
    assert lib.fasted_last_error().decode() == GOLDEN["empty_error"]
    bad = tmp_path / "bad.csv"
    bad.write_text("1,2\n3,x\n")
    assert lib.fasted_load_file(str(bad).encode()) != 0
    trailing = tmp_path / "trail.csv"
    trailing.write_text("0.5,0.25,\n1,2,\n")  # a trailing delimiter adds no field
    assert lib.fasted_load_file(str(trailing).encode()) == 0
    _, n, d, name = fasted_amd.resident_points()
    assert (n, d, name) == (2, 2, "trail")


def test_raw_entry_rejects_bad_arguments_without_touching_a_gpu(lib):
    found, stored = ctypes.c_ulonglong(), ctypes.c_ulonglong()
    assert lib.fasted_self_join(None, 10, 8, 0.1, None, 0, ctypes.byref(found), ctypes.byref(stored)) != 0
    assert b"null" in lib.fasted_last_error()
    st = fp.FastedJoinStats()
    assert lib.fasted_self_join_device(None, 10, 64, 64, 0.1, None, None, 0, 0, None, ctypes.byref(st)) != 0
    buf = (ctypes.c_uint16 * 64)()
    for n, d, ld in [(0, 64, 64), (10, 0, 64), (10, 64, 60), (10, 100, 64), (10, 64, 1 << 23), (2 ** 31 - 1, 64, 64)]:
        rc = lib.fasted_self_join_device(ctypes.addressof(buf), n, d, ld, 0.1, None, None, 0, 0, None, ctypes.byref(st))
        assert rc != 0 and lib.fasted_last_error()
    assert lib.fasted_self_join_blocked(ctypes.addressof(buf), 10, 8, 0.1, 0, None, 0, None, None) != 0
    assert b"block" in lib.fasted_last_error()
    # a NaN epsilon is refused by every entry that takes one, before any device call (the reference's comparison
    # with NaN is false for every pair, source/warpMma.cuh:257; here it would poison the accumulator start values)
    nan = float("nan")
    assert lib.fasted_self_join(ctypes.addressof(buf), 4, 8, nan, None, 0, ctypes.byref(found), ctypes.byref(stored)) != 0
    assert b"NaN" in lib.fasted_last_error()
    assert lib.fasted_self_join_device(ctypes.addressof(buf), 1, 64, 64, nan, None, None, 0, 0, None, ctypes.byref(st)) != 0
    assert b"NaN" in lib.fasted_last_error()
    assert lib.fasted_self_join_device_noalloc(ctypes.addressof(buf), 1, 64, 64, nan, None, 0, 0, None, ctypes.byref(st)) != 0
    assert lib.fasted_join_device(ctypes.addressof(buf), 1, 64, ctypes.addressof(buf), 1, 64, 64, nan, None, None, None, 0,
                                  0, None, ctypes.byref(st)) != 0
    assert lib.fasted_self_join_blocked(ctypes.addressof(buf), 4, 8, nan, 256, None, 0, None, None) != 0
    assert b"NaN" in lib.fasted_last_error()
    assert lib.fasted_pair_distances_device(None, 1, 64, None, 1, 64, 64, None, 0, None, None) != 0


# ---------------------------------------------------------------- tile queues (host mirror)
@pytest.mark.parametrize("n", [1, 256, 257, 4096, 5000, 100_000])
def test_tile_queues_cover_every_tile_exactly_once(lib, n):
    tiles = -(-n // 256)
    total = lib.fasted_raster_count(n)
    assert total % (8 * 32) == 0 and total >= tiles * tiles
    row, col = ctypes.c_int(), ctypes.c_int()
    seen = np.zeros((tiles, tiles), dtype=np.int32)
    padding = 0
    step = 1 if total <= 300_000 else None
    idxs = range(total) if step else None
    for idx in idxs:
        kind = lib.fasted_raster_coord(idx, n, ctypes.byref(row), ctypes.byref(col))
        assert kind in (1, 2)
        assert row.value % 256 == 0 and col.value % 256 == 0
        if kind == 1:
            seen[row.value // 256, col.value // 256] += 1
        else:
            padding += 1
            assert row.value >= n or col.value >= n
    assert (seen == 1).all()
    assert padding == total - tiles * tiles
    assert lib.fasted_raster_coord(total, n, ctypes.byref(row), ctypes.byref(col)) == 0


@pytest.mark.parametrize("n", [1, 256, 4097, 5000, 70_000, 150_000])
def test_symmetric_tile_queues_cover_the_upper_triangle_exactly_once(lib, n):
    """The order of a FASTED_SYMMETRIC join: every tile on or above the diagonal exactly once, nothing
    else marked as work, and about half as many queue positions as the full order."""
    total = lib.fasted_raster_count_symmetric(n)
    tiles = -(-n // 256)
    seen = np.zeros((tiles, tiles), dtype=np.int32)
    row, col = ctypes.c_int(), ctypes.c_int()
    for idx in range(total):
        kind = lib.fasted_raster_coord_symmetric(idx, n, ctypes.byref(row), ctypes.byref(col))
        assert kind in (1, 2)
        if kind == 1:
            assert row.value <= col.value
            seen[row.value // 256, col.value // 256] += 1
    assert lib.fasted_raster_coord_symmetric(total, n, ctypes.byref(row), ctypes.byref(col)) == 0
    assert np.array_equal(seen, np.triu(np.ones((tiles, tiles), dtype=np.int32)))
    if tiles >= 64:
        # super-squares are 32 x 8 tiles: row i of them keeps the squares from column 4 * i on
        square_rows, square_cols = -(-tiles // 32), -(-tiles // 8)
        expected = 256 * sum(square_cols - 4 * i for i in range(square_rows))
    else:
        # small matrices: 16 x 16 super-squares, the upper triangle of them
        squares = -(-tiles // 16)
        expected = 256 * squares * (squares + 1) // 2
    assert total == expected <= lib.fasted_raster_count(n)


def test_tile_queue_locality(lib):
    """32 consecutive positions of one queue are one block of tiles (one XCD's share of a super-square), the 8
    queues together tile that super-square, and consecutive super-squares follow each other along the
    candidates (the query panels stay).  Matrices of 64 x 64 tiles and more: blocks of 8 x 4, super-squares of
    32 x 8; smaller ones: 4 x 8 and 16 x 16."""
    row, col = ctypes.c_int(), ctypes.c_int()
    for n_tiles, (br, bc), expected in ((96, (8, 4), [(0, 0), (0, 8), (0, 32), (32, 0), (32, 8)]),
                                       (48, (4, 8), [(0, 0), (0, 16), (16, 16), (32, 0), (32, 16)])):
        n = 256 * n_tiles
        origins = []
        squares = (0, 1, 4, 12, 13) if n_tiles == 96 else (0, 1, 4, 6, 7)
        for square in squares:
            cover = set()
            for q in range(8):
                block = []
                for t in range(32):
                    idx = (square * 32 + t) * 8 + q
                    assert lib.fasted_raster_coord(idx, n, ctypes.byref(row), ctypes.byref(col)) == 1
                    block.append((row.value // 256, col.value // 256))
                r0, c0 = block[0]
                assert block == [(r0 + t // bc, c0 + t % bc) for t in range(32)]
                cover |= set(block)
            rs, cs = min(r for r, _ in cover), min(c for _, c in cover)
            assert cover == {(rs + i, cs + j) for i in range(4 * br) for j in range(2 * bc)}
            origins.append((rs, cs))
        assert origins == expected


# ---------------------------------------------------------------- LDS swizzle (host mirror)
# lane groups that gfx950 serves together in one phase of a ds_read_b128
B128_PHASES = [[*range(0, 4), *range(12, 16), *range(20, 24), *range(24, 28)],
               [*range(4, 8), *range(8, 12), *range(16, 20), *range(28, 32)],
               [*range(32, 36), *range(44, 48), *range(52, 56), *range(56, 60)],
               [*range(36, 40), *range(40, 44), *range(48, 52), *range(60, 64)]]


def test_lds_swizzle_is_a_bijection_and_bank_conflict_free(lib):
    lib.fasted_lds_chunk_slot.restype = ctypes.c_int
    lib.fasted_lds_chunk_slot.argtypes = [ctypes.c_int, ctypes.c_int]
    for row in range(256):  # every row keeps its 8 chunks in 8 distinct slots
        assert sorted(lib.fasted_lds_chunk_slot(row, c) for c in range(8)) == list(range(8))
    # fragment read of v_mfma_f32_16x16x32_f16: lane l -> row base + l%16, chunk 4*ks + l//16.
    # A row is 128 B: its parity selects the half of the 64 banks, the slot 4 banks inside it.
    for base in range(0, 256, 16):
        for ks in (0, 1):
            for phase in B128_PHASES:
                touched = {((base + l % 16) & 1, lib.fasted_lds_chunk_slot(base + l % 16, 4 * ks + l // 16))
                           for l in phase}
                assert len(touched) == 16, (base, ks, phase)


# ---------------------------------------------------------------- epsilon search + accuracy helpers
class MockFindPairs:
    """Stand-in backend in the manner of the reference's tests (results/scripts/tests/
    test_experiments.py:14-71): pairsFound is a monotone function of epsilon."""

    def __init__(self, n=10_000, density=700.0):
        self.n, self.density, self.calls = n, density, []

    def selectivity(self, eps):
        self.calls.append(eps)
        found = int(self.n + self.density * eps ** 3 * self.n)
        return fp.compute_selectivity(found, self.n)


def test_epsilon_search_restatement_follows_the_reference_procedure():
    """The checker's restatement of the reference's search (oracle/epsilon_search.py) against what the
    procedure fixes on a closed-form selectivity: the exact sequence of probes."""
    from oracle import epsilon_search as ex

    assert ex.within_percent(100.5, 100, 0.01) and not ex.within_percent(102, 100, 0.01)
    assert ex.adjust_epsilon_binary(4.0, 8.0, 64, 100) == 2.0  # overshoot: half a step back
    assert ex.adjust_epsilon_binary(2.0, 4.0, 64, 10) == 3.0   # undershoot: half a step forward
    mock = MockFindPairs()
    lo, hi = ex.bound_epsilon(0.0, 100000, 64, mock.selectivity)
    assert mock.calls == [2.0] and (lo, hi) == (0.0, 2.0)  # 0 -> 2, then doubling
    mock = MockFindPairs(density=0.001)
    assert ex.bound_epsilon(0.0, 100000, 64, mock.selectivity) == (32.0, 64.0)
    assert mock.calls == [2.0, 4.0, 8.0, 16.0, 32.0, 64.0]
    with pytest.raises(ValueError):
        ex.bound_epsilon(0.0, 10.0, 1e12, MockFindPairs().selectivity)
    mock = MockFindPairs()
    eps = ex.find_epsilon_binary(64, mock.selectivity)
    assert ex.within_percent(700.0 * eps ** 3, 64, 0.011)
    assert mock.calls[:2] == [2.0, 1.0]  # the upper bound, then the midpoint of (0, 2)
    # selectivity = 1000 eps: target 250 is hit exactly by the probes 2 (bound), 1, 0.5, 0.25
    calls = []
    assert ex.find_epsilon_binary(250, lambda e: calls.append(e) or 1000.0 * e) == 0.25
    assert calls == [2.0, 1.0, 0.5, 0.25]


def test_volumetric_epsilon_search_restatement():
    """The restated volume scaling against what the mathematics fixes: the constants of the two ball volumes
    cancel, so a step is eps * (target / s)^(1/D); on a selectivity that is exactly c * eps^D one step lands on
    the target; an empty probe doubles epsilon."""
    from oracle import epsilon_search as ex

    assert abs(float(ex.compute_gamma(4)) - 2.0) < 1e-12            # Gamma(3) = 2
    assert abs(float(ex.compute_gamma(5)) - 3.323350970447843) < 1e-12  # Gamma(7/2) = 15 sqrt(pi) / 8
    assert ex.adjust_epsilon_volume(0.3, 0, 10.0, 64) == 0.6
    for eps, s, t, d in [(0.1, 3.0, 64.0, 2), (2.5, 1000.0, 16.0, 128), (0.03, 0.5, 200.0, 4096), (7.0, 9.0, 9.5, 17)]:
        assert abs(ex.adjust_epsilon_volume(eps, s, t, d) / (eps * (t / s) ** (1.0 / d)) - 1.0) < 1e-12
    calls = []
    eps = ex.find_epsilon_volumetric(3, 64.0, lambda e: calls.append(e) or 700.0 * e ** 3)
    assert len(calls) == 2 and calls[0] == 0.1 and abs(700.0 * eps ** 3 - 64.0) < 1e-9
    calls = []
    eps = ex.find_epsilon_volumetric(8, 5.0, lambda e: calls.append(e) or (0.0 if e < 0.35 else 40.0 * e ** 2))
    assert calls[:3] == [0.1, 0.2, 0.4] and ex.within_percent(40.0 * eps ** 2, 5.0, 0.1)
    with pytest.raises(RuntimeError):
        ex.find_epsilon_volumetric(2, 5.0, lambda e: 1.0, max_iterations=20)  # a plateau never gets there


def test_pair_statistics_and_per_point_iou():
    from fasted_amd import accuracy as ex

    five = np.array([[1, 1], [2, 2], [3, 3], [4, 4], [5, 5]])
    assert ex.compute_pair_stats(five, five) == ex.PairsStats(5, 0, 0, 5, 5)
    assert ex.compute_pair_stats(five, np.delete(five, 2, axis=0)) == ex.PairsStats(4, 0, 1, 5, 4)
    assert ex.compute_pair_stats(np.delete(five, 0, axis=0), five) == ex.PairsStats(4, 1, 0, 4, 5)
    # agrees with the checker's merge walk on random lists
    rng = np.random.default_rng(9)
    a = oracle.sort_pairs(np.unique(rng.integers(0, 40, (300, 2)), axis=0))
    b = oracle.sort_pairs(np.unique(rng.integers(0, 40, (300, 2)), axis=0))
    s, o = ex.compute_pair_stats(a, b), oracle.pair_stats(a, b)
    assert (s.both_sides, s.right_only, s.left_only) == (o["both"], o["right_only"], o["left_only"])
    iou = ex.per_point_iou([[0, 0], [0, 1], [1, 1], [2, 2]], [[0, 0], [0, 2], [1, 1]], 4)
    assert iou.tolist() == [1 / 3, 1.0, 0.0, 1.0]


def test_csv_loader_multithreaded_equals_numpy_parse(lib, tmp_path, monkeypatch):
    rng = np.random.default_rng(12)
    vals = rng.exponential(1 / 40.0, (5003, 37))
    path = tmp_path / "big.csv"
    with open(path, "w") as f:
        for i, row in enumerate(vals):
            sep = ",  " if i % 7 == 0 else ","  # leading blanks are skipped like std::stod does
            f.write(sep.join(repr(float(v)) for v in row) + ("\r\n" if i % 11 == 0 else "\n"))
    want = oracle.quantize(vals)
    for threads in ("1", "3", "16"):
        monkeypatch.setenv("FASTED_CSV_THREADS", threads)
        assert lib.fasted_load_file(str(path).encode()) == 0
        bits, n, d, name = fasted_amd.resident_points()
        assert (n, d, name) == (5003, 37, "big") and bits.shape == (5120, 64)
        assert np.array_equal(bits[:n, :d], want) and bits[n:].sum() == 0 and bits[:, d:].sum() == 0
    # the first bad line wins, whichever thread meets it
    lines = open(path).read().split("\n")
    lines[4000] = "1,2,3"
    lines[900] = lines[900].replace(",", ",oops,", 1)
    bad = tmp_path / "bad.csv"
    bad.write_text("\n".join(lines))
    assert lib.fasted_load_file(str(bad).encode()) != 0
    assert lib.fasted_last_error() == b"stod"
    no_newline = tmp_path / "nonl.csv"
    no_newline.write_text("1,2\n3,4")  # last line without a newline still counts
    assert lib.fasted_load_file(str(no_newline).encode()) == 0
    assert fasted_amd.resident_points()[1] == 2
    blank = tmp_path / "blank.csv"
    blank.write_text("1,2\n\n3,4\n")  # an empty line is a point with no dimensions
    assert lib.fasted_load_file(str(blank).encode()) != 0
    assert lib.fasted_last_error().decode() == GOLDEN["ragged_error"]


def test_host_quantisation_rounds_twice_like_the_reference(lib, tmp_path):
    """double -> float -> half is not double -> half: doubles whose float image is an exact tie between
    two halves round differently.  The loader must take the two-step route (PointListBuilder.hpp:57-73)."""
    rng = np.random.default_rng(99)
    x = rng.exponential(1 / 40.0, 4_000_000)
    two_step = x.astype(np.float32).astype(np.float16).view(np.uint16)
    one_step = x.astype(np.float16).view(np.uint16)
    tricky = np.concatenate([[0.01198196413320991], x[two_step != one_step][:63]])
    assert len(tricky) >= 8
    path = tmp_path / "ties.csv"
    path.write_text("\n".join(repr(float(v)) for v in tricky) + "\n")
    assert lib.fasted_load_file(str(path).encode()) == 0
    bits, n, d, _ = fasted_amd.resident_points()
    assert (n, d) == (len(tricky), 1)
    assert np.array_equal(bits[:n, 0], tricky.astype(np.float32).astype(np.float16).view(np.uint16))
    assert np.array_equal(bits[:n, 0], oracle.quantize(tricky))


# ---------------------------------------------------------------- experiment driver
class MockBackend:
    """Backend in the manner of the reference's MockFindPairs (results/scripts/tests/
    test_experiments.py:14-71): the selectivity equals epsilon, nothing is computed."""

    def __init__(self):
        self.size, self.dim, self.log = 0, 0, []

    def load_exponential(self, size, dim, lam=40.0, value_range=10.0):
        self.size, self.dim = size, dim
        self.log.append(("exp", size, dim, lam, value_range))

    def load_file(self, path):
        self.size, self.dim = 100000, 15
        self.log.append(("file", str(path)))

    def run(self, epsilon, save_pairs=False):
        self.log.append(("run", epsilon, save_pairs))
        r = fp.Results()
        r.TFLOPS = 1.0
        r.pairsFound = r.pairsStored = int(epsilon * self.size) + self.size
        r.inputProblemShape = fp.mmaShape(self.size, self.size, self.dim)
        r.paddedProblemShape = fp.mmaShape(self.size, self.size, self.dim)
        return r

    def epsilon_for(self, target, sample_rows=None):
        self.log.append(("search", target, sample_rows))
        return float(target), float(target), 5


def reference_record_keys():
    with open(os.path.join(os.path.dirname(__file__), "golden", "speed_results_records.json")) as f:
        gold = json.load(f)
    rec = gold["sweep"][0]
    return set(rec), set(rec["results"]), gold


def test_sweep_driver_writes_the_reference_result_schema(tmp_path):
    from fasted_amd import experiments as ex

    top, inner, _ = reference_record_keys()
    backend = MockBackend()
    driver = ex.SweepDriver(backend, output_dir=str(tmp_path))

    # size x dimensionality sweep: dataset built once per shape, 3 timed runs each
    path = driver.exponential_sweep(sizes=[1000, 2154], dims=[64, 128])
    assert re.fullmatch(r"ExpoDataSpeedVsSize_\d+\.json", os.path.basename(path))
    records = json.load(open(path))
    assert len(records) == 2 * 2 * 3
    for r in records:
        assert set(r) == top and inner <= set(r["results"])
        assert r["epsilon"] == 0.001 and r["selectivity"] == 0
        assert r["results"]["inputProblemShape"]["m"] in (1000, 2154)
    assert [r["iteration"] for r in records[:3]] == [0, 1, 2]
    builds = [e for e in backend.log if e[0] == "exp"]
    assert [(e[1], e[2]) for e in builds] == [(1000, 64), (1000, 128), (2154, 64), (2154, 128)]
    assert all(e[3:5] == (40.0, 10.0) for e in builds)  # lambda 40, range 10 (experiments.py:556-557)
    assert len([e for e in backend.log if e[0] == "run"]) == 12
    # the default grid is the reference's: 10 log-spaced sizes x 7 dimensionalities
    backend.log.clear()
    driver.exponential_sweep(repetitions=0)
    builds = [e for e in backend.log if e[0] == "exp"]
    assert [e[1] for e in builds[::7]] == [1000, 2154, 4642, 10000, 21544, 46416, 100000, 215443, 464159, 1000000]
    assert [e[2] for e in builds[:7]] == [64, 128, 256, 512, 1024, 2048, 4096]

    # selectivity sweep: one build, one native search per target (epsilon == selectivity for the mock), 3 runs each
    backend.log.clear()
    path = driver.selectivity_sweep([1, 10, 100], size=5000, dim=64, sample_rows=512)
    records = json.load(open(path))
    assert len(records) == 9 and [r["selectivity"] for r in records[::3]] == [1, 10, 100]
    assert all(r["epsilon"] == r["selectivity"] for r in records)
    assert [e for e in backend.log if e[0] in ("exp", "search")] == [
        ("exp", 5000, 64, 40.0, 10.0), ("search", 1, 512), ("search", 10, 512), ("search", 100, 512)]

    # known epsilons on a file: loaded once, pairs saved by the first run of a parameter set only
    backend.log.clear()
    path = driver.file_runs("base/data.csv", [(64, 1.2), (128, 3.4)], repetitions=2, save_pairs=True)
    assert os.path.basename(path).startswith("data.csv_results_")
    assert backend.log == [("file", "base/data.csv"), ("run", 1.2, True), ("run", 1.2, False), ("run", 3.4, True),
                           ("run", 3.4, False)]

    # epsilon search over datasets: a dictionary of record lists keyed by dataset
    path = driver.file_epsilon_search(["base/a.txt", "base/b.txt"], [1, 10])
    by_dataset = json.load(open(path))
    assert set(by_dataset) == {"a.txt", "b.txt"} and all(len(v) == 2 for v in by_dataset.values())


def test_timed_runs_skip_failed_runs():
    from fasted_amd import experiments as ex

    class Flaky(MockBackend):
        def run(self, epsilon, save_pairs=False):
            if len([e for e in self.log if e[0] == "run"]) == 1:
                self.log.append(("run", epsilon, save_pairs))
                raise RuntimeError("device lost")
            return super().run(epsilon, save_pairs)

    backend = Flaky()
    out = ex.SweepDriver(backend).timed_runs(1, 0.5, 3, save_pairs=True)
    assert [r["iteration"] for r in out] == [0, 2]
    assert [e[1:] for e in backend.log] == [(0.5, True), (0.5, False), (0.5, False)]


class MockLibrary:
    """The three entry points a reference script drives (results/scripts/tests/test_experiments.py:14-71)."""

    def __init__(self):
        self.n, self.calls = 1000, []

    def _results(self, eps):
        r = fp.Results()
        r.pairsFound = r.pairsStored = int(self.n + 50.0 * eps * self.n)
        r.inputProblemShape.m = r.inputProblemShape.n = self.n
        r.inputProblemShape.k = 64
        r.TFLOPS, r.totalTime = 1.0, 0.1
        return r

    def runFromExponentialDataset(self, size, dim, lam, rng, eps, save):
        self.calls.append(("exp", size, dim, eps, save))
        self.n = size
        return self._results(eps)

    def runFromFile(self, path, eps, save):
        self.calls.append(("file", path, eps, save))
        return self._results(eps)

    def reRun(self, eps, save):
        self.calls.append(("rerun", eps, save))
        return self._results(eps)


def test_reference_named_runner_drives_a_mock_and_writes_the_reference_files(tmp_path):
    """ExperimentRunner / SearchParameters / find_epsilon_binary under the reference's names
    (results/scripts/experiment/experiments.py:58-73,228-281,341-591): a script written against them runs on
    this package, here over a mock library; the Python search makes the probes of the restated procedure."""
    import json

    from fasted_amd import experiments as ex
    from oracle import epsilon_search as restated

    calls, calls_restated = [], []
    sel = lambda log: (lambda e: log.append(e) or 700.0 * e ** 3)  # noqa: E731
    assert ex.find_epsilon_binary(64, sel(calls)) == restated.find_epsilon_binary(64, sel(calls_restated))
    assert calls == calls_restated and len(calls) > 3
    with pytest.raises(ValueError):
        ex.find_epsilon_binary(1e12, lambda e: 0.0)
    with pytest.raises(ValueError):
        ex.find_epsilon_binary(10.0, lambda e: 0.0 if e < 1.5 else 20.0)  # a step: never within 1 %

    mock = MockLibrary()
    runner = ex.ExperimentRunner(mock, output_dir=str(tmp_path))
    path = runner.run_real_dataset_known_epsilons_experiments(str(tmp_path), "x.txt",
                                                              [ex.SearchParameters(64, 0.5, True)], 2)
    records = json.load(open(path))
    assert [r["iteration"] for r in records] == [0, 1] and records[0]["epsilon"] == 0.5
    assert set(records[0]["results"]) == {"totalTime", "TFLOPS", "pairsFound", "pairsStored", "inputProblemShape",
                                          "paddedProblemShape"}
    assert mock.calls[0][0] == "file" and mock.calls[0][3] is True and mock.calls[1] == ("rerun", 0.5, False)
    path = runner.run_selectivity_vs_speed_experiment([10, 100])
    records = json.load(open(path))
    assert len(records) == 6 and abs(50.0 * records[0]["epsilon"] - 10) < 0.1
    finder = runner.build_rerunnable_file_pairs_finder(str(tmp_path), "q.txt")
    out = runner.run_selectivity_experiment([20], finder, iterations=2)
    assert len(out) == 2 and isinstance(out[0], ex.Experiment)
    assert json.loads(json.dumps(out, cls=ex.ResultsEncoder))[1]["iteration"] == 1
    assert runner.get_selectivity_rerun(0.2) == pytest.approx(10.0)
