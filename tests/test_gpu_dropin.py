"""GPU tests of the drop-in boundary: the reference's entry points, the `.pairs` text output and the
command-line driver, checked against the CPU checker."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

import oracle
from tests import datasets

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    import fasted_amd

    return fasted_amd.load_findpairs()


def write_csv(path, values):
    with open(path, "w") as f:
        for row in values:
            f.write(",".join(repr(float(v)) for v in row) + "\n")


def test_run_from_file_saves_sorted_pairs_text(lib, tmp_path):
    import fasted_amd

    rng = np.random.default_rng(21)
    vals = np.round(rng.random((900, 40)), 6)
    csv = tmp_path / "points900.csv"
    write_csv(csv, vals)
    bits = oracle.quantize(vals)
    eps = datasets.epsilon_for_neighbours(bits, 6)
    lib.fasted_set_output_dir(str(tmp_path).encode())
    r = lib.runFromFile(str(csv).encode(), eps, True)
    assert (r.inputProblemShape.m, r.inputProblemShape.k) == (900, 40)
    assert (r.paddedProblemShape.m, r.paddedProblemShape.k) == (1024, 64)
    assert r.pairsFound == r.pairsStored
    # file name: <dataset name>_<std::to_string(eps)>.pairs ; lines "q, c"
    out = tmp_path / ("points900_%f.pairs" % eps)
    assert out.exists(), os.listdir(tmp_path)
    text = out.read_text().splitlines()
    assert all(re.fullmatch(r"\d+, \d+", line) for line in text)
    got = np.array([[int(x) for x in line.split(", ")] for line in text], dtype=np.int32)
    assert len(got) == r.pairsFound
    assert np.array_equal(got, oracle.sort_pairs(got))  # already row-major
    rep = oracle.epsilon_band_report(bits, got, eps)
    assert rep["outside_band"] == 0 and rep["both"] > 900
    # the resident dataset is what the reference's builder would hold
    resident, n, d, name = fasted_amd.resident_points()
    assert (n, d, name) == (900, 40, "points900")
    assert np.array_equal(resident[:900, :40], bits)
    # reRun on the resident data, no file this time
    r2 = lib.reRun(eps * 1.1, False)
    assert r2.pairsFound > r.pairsFound
    assert len(list(tmp_path.glob("*.pairs"))) == 1
    # reRun with saving: the file keeps the dataset's name
    r3 = lib.reRun(eps * 1.1, True)
    again = tmp_path / ("points900_%f.pairs" % (eps * 1.1))
    assert again.exists() and len(again.read_text().splitlines()) == r3.pairsStored == r2.pairsStored
    lib.releaseResources()
    lib.fasted_set_output_dir(b"")


def test_results_fields_and_tflops_formula(lib):
    n, d = 5000, 256
    r = lib.runFromExponentialDataset(n, d, 40.0, 10.0, 0.5, False)
    assert r.totalTime > 0
    # TFLOPS = 2 N^2 D / kernel time with unpadded N, D: kernel time must be below the total time
    kernel_s = 2.0 * n * n * d / (r.TFLOPS * 1e12)
    assert 0 < kernel_s <= r.totalTime
    assert r.get_selectivity() == max(0, r.pairsFound - n) / n
    lib.releaseResources()


def test_command_line_driver(tmp_path):
    exe = os.path.join(ROOT, "fasted_amd", "fasted")
    assert os.path.exists(exe), "build the CLI with make -C fasted_amd/csrc release"
    out = subprocess.run([exe, "-e", "3000", "128", "0.001"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "Pairs found: 3000" in out.stdout  # only the self pairs at eps = 0.001
    assert re.search(r"Estimated TFLOPS [\d.]+", out.stdout)
    bad = subprocess.run([exe, "-e", "10"], capture_output=True, text=True, timeout=60)
    assert bad.returncode == 1 and "Usage" in bad.stderr
    missing = subprocess.run([exe, str(tmp_path / "nope.csv"), "0.1"], capture_output=True, text=True, timeout=60)
    assert missing.returncode != 0 and "Failed" in missing.stdout


def test_native_epsilon_search_matches_the_python_procedure(lib):
    """fasted_find_epsilon follows the reference's bound-then-bisect search probe for probe: the
    Python mirror driven by count-only probes lands on the same epsilon."""
    import fasted_amd
    from oracle import epsilon_search as ex

    n, d = 6000, 64
    assert lib.fasted_load_exponential_dataset(n, d, 40.0, 10.0) == 0
    eps, sel, probes = fasted_amd.find_epsilon(16.0)
    assert ex.within_percent(sel, 16.0, 0.01) and probes >= 3
    calls = []

    def get_selectivity(e):
        calls.append(e)
        return fasted_amd.compute_selectivity(fasted_amd.count_pairs(e)[0], n)

    assert ex.find_epsilon_binary(16.0, get_selectivity) == eps
    assert len(calls) == probes
    # the count-only probe agrees with a storing reRun and with the FP64 checker
    found, secs = fasted_amd.count_pairs(eps)
    r = lib.reRun(eps, False)
    assert found == r.pairsFound and secs > 0
    bits, _, _, _ = fasted_amd.resident_points()
    truth = oracle.self_join_f64(bits, eps, n=n)
    assert abs(int(found) - len(truth)) <= max(4, len(truth) // 500)
    lib.releaseResources()


@pytest.mark.parametrize("n,d", [(3000, 320), (20000, 192)])
def test_count_only_probe_equals_the_full_join_count(lib, n, d):
    """The count-only probe computes the tiles on and above the diagonal only and doubles what it finds off the
    diagonal; a storing reRun computes the whole matrix.  The two counts must be equal at every epsilon (144 tiles
    one per workgroup, and 6241 tiles through the queues in the tall order)."""
    import fasted_amd

    assert lib.fasted_load_exponential_dataset(n, d, 40.0, 10.0) == 0
    eps, sel, _ = fasted_amd.find_epsilon_sampled(24.0, sample_rows=2000)
    for e in (eps, 0.8 * eps, 1e-4):
        found, secs = fasted_amd.count_pairs(e)
        r = lib.reRun(e, False)
        assert found == r.pairsFound >= n and secs > 0, e
    lib.releaseResources()


def test_pairs_can_stay_on_the_device(lib):
    """With the download switched off a run that does not save reports the same Results and leaves the sorted pairs
    in the library's device buffer, where fasted_last_pairs_device finds them; a saving run still writes its file."""
    import torch

    import fasted_amd

    n, d = 3000, 64
    assert lib.fasted_load_exponential_dataset(n, d, 40.0, 10.0) == 0
    bits, _, _, _ = fasted_amd.resident_points()
    eps = datasets.epsilon_for_neighbours(bits[:n, :d].copy(), 12)
    want, found = fasted_amd.self_join(bits[:n, :d].copy(), eps)
    r_down = lib.reRun(eps, False)
    fasted_amd.set_download_pairs(False)
    try:
        r = lib.reRun(eps, False)
        assert (r.pairsFound, r.pairsStored) == (r_down.pairsFound, r_down.pairsStored) == (found, found)
        ptr, stored = fasted_amd.last_pairs_device()
        assert stored == found and ptr
        out = torch.empty((stored, 2), dtype=torch.int32, device="cuda")
        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        assert hip.hipMemcpy(out.data_ptr(), ptr, stored * 8, 3) == 0  # device to device
        assert np.array_equal(out.cpu().numpy(), want)
    finally:
        fasted_amd.set_download_pairs(True)
    lib.releaseResources()
    ptr, stored = fasted_amd.last_pairs_device()
    assert stored == 0


def test_native_volumetric_epsilon_search(lib):
    """fasted_find_epsilon_volumetric against the restated procedure driven by count-only probes: the same
    probes (the decimal and the double form of a step agree to rounding), an epsilon within 10 % of the target."""
    import ctypes

    import fasted_amd
    from oracle import epsilon_search as ex

    n, d = 6000, 64
    assert lib.fasted_load_exponential_dataset(n, d, 40.0, 10.0) == 0
    eps, sel, probes = fasted_amd.find_epsilon_volumetric(16.0, 0.1)
    assert ex.within_percent(sel, 16.0, 0.1) and probes >= 2
    calls = []

    def get_selectivity(e):
        calls.append(e)
        return fasted_amd.compute_selectivity(fasted_amd.count_pairs(e)[0], n)

    want = ex.find_epsilon_volumetric(d, 16.0, get_selectivity, 0.1)
    assert len(calls) == probes and abs(want - eps) <= 1e-9 * eps
    assert fasted_amd.compute_selectivity(fasted_amd.count_pairs(eps)[0], n) == sel
    # bad arguments come back as errors, not as a loop
    e, s_, p_ = ctypes.c_double(), ctypes.c_double(), ctypes.c_int()
    assert lib.fasted_find_epsilon_volumetric(16.0, 0.0, ctypes.byref(e), ctypes.byref(s_), ctypes.byref(p_)) != 0
    assert lib.fasted_find_epsilon_volumetric(-1.0, 0.1, ctypes.byref(e), ctypes.byref(s_), ctypes.byref(p_)) != 0
    lib.releaseResources()


def test_sampled_epsilon_search(lib):
    """The search on sampled probes: the sampled count equals the count of the same rows in the full pair
    list, and the epsilon found lands close to the full search's at a fraction of the work."""
    import ctypes

    import fasted_amd
    from oracle import epsilon_search as ex

    n, d = 20000, 64
    assert lib.fasted_load_exponential_dataset(n, d, 40.0, 10.0) == 0
    eps_full, sel_full, probes_full = fasted_amd.find_epsilon(30.0)
    eps_s, sel_s, probes_s = fasted_amd.find_epsilon_sampled(30.0, sample_rows=2000)
    assert probes_s >= 4 and abs(eps_s - eps_full) / eps_full < 0.01
    assert ex.within_percent(sel_s, 30.0, 0.05)  # the dataset's selectivity at the sampled search's epsilon
    # the sampled probe counts exactly the pairs whose query point is one of the sampled rows
    found, rows, secs = ctypes.c_ulonglong(), ctypes.c_int(), ctypes.c_double()
    assert lib.fasted_count_pairs_sampled(eps_s, 2000, ctypes.byref(found), ctypes.byref(rows), ctypes.byref(secs)) == 0
    assert rows.value == 2000
    bits, _, _, _ = fasted_amd.resident_points()
    pairs, total = fasted_amd.self_join(bits[:n, :d].copy(), eps_s)
    sampled_rows = np.arange(2000) * (n // 2000)
    assert found.value == int(np.isin(pairs[:, 0], sampled_rows).sum())
    lib.releaseResources()


def test_experiment_sweep_reproduces_the_reference_result_records(lib, tmp_path):
    """The size x dimensionality sweep of the reference's experiment driver, run on the library: for
    the shapes small enough to run here the records of results/speed_results/
    ExpoDataSpeedVsSize_OnDemandRasterizer.json (pairs found, input shape, epsilon) are reproduced."""
    import json

    from fasted_amd import experiments as ex

    with open(os.path.join(ROOT, "tests", "golden", "speed_results_records.json")) as f:
        gold = json.load(f)["sweep"]
    sizes = sorted({r["results"]["inputProblemShape"]["m"] for r in gold})
    dims = sorted({r["results"]["inputProblemShape"]["k"] for r in gold})
    driver = ex.SweepDriver(ex.LibraryBackend(lib), output_dir=str(tmp_path))
    records = json.load(open(driver.exponential_sweep(sizes=sizes, dims=dims, repetitions=1)))
    key = lambda r: (r["results"]["inputProblemShape"]["m"], r["results"]["inputProblemShape"]["k"])
    ours = {key(r): r for r in records}
    assert len(ours) == len(gold)
    for g in gold:
        r = ours[key(g)]
        assert set(g) == set(r) and set(g["results"]) <= set(r["results"])
        assert (r["selectivity"], r["epsilon"], r["iteration"]) == (g["selectivity"], g["epsilon"], g["iteration"])
        for field in ("pairsFound", "pairsStored", "inputProblemShape"):
            assert r["results"][field] == g["results"][field], (field, key(g))
        assert r["results"]["paddedProblemShape"]["k"] == g["results"]["paddedProblemShape"]["k"]
        assert r["results"]["TFLOPS"] > 0
    lib.releaseResources()


def test_pairs_file_with_the_distance_column(lib, tmp_path):
    """Opt-in third column "q, c, dist" (the form results/scripts/neighbor_tables.py:102-115 parses)."""
    rng = np.random.default_rng(5)
    vals = np.round(rng.random((700, 70)), 6)
    csv = tmp_path / "dist700.csv"
    write_csv(csv, vals)
    bits = oracle.quantize(vals)
    eps = datasets.epsilon_for_neighbours(bits, 8)
    lib.fasted_set_output_dir(str(tmp_path).encode())
    lib.fasted_set_save_distances(1)
    try:
        r = lib.runFromFile(str(csv).encode(), eps, True)
    finally:
        lib.fasted_set_save_distances(0)
    lines = (tmp_path / ("dist700_%f.pairs" % eps)).read_text().splitlines()
    assert len(lines) == r.pairsStored
    parsed = [re.fullmatch(r"(\d+), (\d+)(, (.+))?", line).group(1, 2, 4) for line in lines]
    got = np.array([[int(q), int(c)] for q, c, _ in parsed], dtype=np.int32)
    dist = np.array([float(x) for _, _, x in parsed])
    assert np.allclose(dist, oracle.pair_distances_f64(bits, got), rtol=1e-5, atol=1e-6)
    assert (dist <= eps * (1 + 1e-3)).all()
    lib.releaseResources()
    lib.fasted_set_output_dir(b"")


def test_large_pair_list_leaves_the_device_in_pieces(lib, tmp_path):
    """More stored pairs than one download piece holds (4 Mi records): the .pairs file must still be the whole
    sorted list, with and without the distance column, and a second reRun (which reuses the pair buffer, the
    sort buffers and the pinned pieces) must write the same bytes."""
    import torch

    import fasted_amd

    n, d = 20000, 64  # the pair buffer holds N*256 records: 230 neighbours per point fit, in two pieces
    assert lib.fasted_load_exponential_dataset(n, d, 40.0, 10.0) == 0
    bits, n_, d_, name = fasted_amd.resident_points()
    eps = datasets.epsilon_for_neighbours(bits[:n, :d], 230)
    lib.fasted_set_output_dir(str(tmp_path).encode())
    r = lib.reRun(eps, True)
    assert r.pairsStored == r.pairsFound > 4 * (1 << 20)
    path = tmp_path / ("%s_%f.pairs" % (name, eps))
    first = path.read_bytes()
    got = np.loadtxt(path, delimiter=",", dtype=np.int64)
    assert got.shape == (r.pairsStored, 2)
    key = got[:, 0] * n + got[:, 1]
    assert np.all(key[1:] > key[:-1])  # row-major, no duplicates, across the piece boundaries too
    # the same list through the device entry
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = int(r.pairsStored) + 1024
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    st = fasted_amd.self_join_device(pts.data_ptr(), n, d, bits.shape[1], eps, pairs.data_ptr(), cap)
    assert st.pairsStored == r.pairsStored
    assert np.array_equal(pairs[: st.pairsStored].cpu().numpy().astype(np.int64), got)
    # again: nothing is allocated this time, the bytes are the same
    r2 = lib.reRun(eps, True)
    assert r2.pairsStored == r.pairsStored and path.read_bytes() == first
    # with the distance column
    lib.fasted_set_save_distances(1)
    r3 = lib.reRun(eps, True)
    lib.fasted_set_save_distances(0)
    with open(path) as f:
        head = [next(f) for _ in range(3)]
    assert all(re.fullmatch(r"\d+, \d+, [0-9.e+-]+\n", line) for line in head)
    with open(path) as f:
        assert sum(1 for _ in f) == r3.pairsStored
    lib.releaseResources()
    lib.fasted_set_output_dir(b"")


def test_sampled_probe_counts_a_points_own_pair_like_the_full_count(lib):
    """At a tiny epsilon only the self pairs remain: the sampled probe (sample x all points) must report
    exactly its sampled rows, as the full count reports exactly N -- large norms included, where the
    expansion s_q + s_c - 2 q.c alone would lose some of them."""
    import ctypes

    n, d = 6000, 512
    assert lib.fasted_load_exponential_dataset(n, d, 40.0, 10.0) == 0
    found, rows, secs = ctypes.c_ulonglong(), ctypes.c_int(), ctypes.c_double()
    assert lib.fasted_count_pairs(1e-4, ctypes.byref(found), ctypes.byref(secs)) == 0
    assert found.value == n
    assert lib.fasted_count_pairs_sampled(1e-4, 1000, ctypes.byref(found), ctypes.byref(rows), ctypes.byref(secs)) == 0
    assert rows.value == 1000 and found.value == 1000
    lib.releaseResources()
