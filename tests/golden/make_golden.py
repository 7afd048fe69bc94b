#!/usr/bin/env python3
"""Writes tests/golden/reference_loader.json from the REFERENCE's own host data loader, and
tests/golden/speed_results_records.json from the result files the reference holds.

The reference's DataLoader/*.hpp (ExponentialPointGenerator, FilePointGenerator,
PointListBuilder<half>, half.hpp) are compiled in place into oracle/_ref/libfasted_ref.so by
oracle/Makefile; this script calls that library and records inputs and outputs as plain data.
Run it in a checkout where /root/reference exists:  python tests/golden/make_golden.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import numpy as np  # noqa: E402

import oracle  # noqa: E402


def main():
    oracle.build()
    ref = oracle.ref()
    if ref is None:
        raise SystemExit("oracle/_ref is not built: the reference checkout is needed")
    out = {"source": "reference DataLoader headers via oracle/_ref (g++ -std=c++17, libstdc++)"}

    # PointListBuilder<half>::castValue on hand-picked doubles: ties, subnormals, overflow, signs
    probes = [0.0, -0.0, 1.0, 0.1, 1.0 / 3.0, 0.00408554, 65504.0, 65519.9, 65520.0, 70000.0, -70000.0, 1e-8, 2.98e-8,
              2.9802322387695312e-08, 5.960464477539063e-08, 8.940696716308594e-08, 6.097555160522461e-05,
              6.103515625e-05, 0.0009765625, 1.0009765625, 1.00048828125, 1.00146484375, 2049.0, 2051.0, 2050.0,
              0.333251953125, 0.3332519531250001, 0.99951171875, 0.999755859375, 0.9997558593750001]
    rng = np.random.default_rng(7)
    probes += list(np.round(rng.exponential(1 / 40.0, 40), 12))
    probes += list(rng.standard_normal(20) * 1000.0)
    out["cast_value"] = {"inputs": [float(p) for p in probes],
                         "bits": [int(ref.ref_cast_value(float(p))) for p in probes]}

    # seeded exponential datasets: (n, d, lambda, max, dimFactor, pointsFactor)
    exp_cases = []
    for n, d, lam, mx, df, pf in [(5, 4, 40.0, 10.0, 64, 768), (7, 70, 40.0, 1.0, 64, 256), (3, 130, 10.0, 0.05, 64, 8)]:
        assert ref.ref_build_exponential(n, d, lam, mx, df, pf) == 0
        v = oracle.ref_values()
        exp_cases.append({"n": n, "d": d, "lambda": lam, "max": mx, "dim_factor": df, "points_factor": pf,
                          "name": ref.ref_dataset_name().decode(), "n_pad": int(v.shape[0]), "d_pad": int(v.shape[1]),
                          "bits": v[:n, :d].tolist(), "padding_sum": int(v.sum() - v[:n, :d].sum())})
    out["exponential"] = exp_cases

    # CSV reader on the committed sample file
    csv = os.path.join(HERE, "sample_points.csv")
    assert ref.ref_build_file(csv.encode(), 64, 256) == 0
    v = oracle.ref_values()
    n, d = ref.ref_actual_num_points(), ref.ref_actual_dimensions()
    out["csv"] = {"file": "sample_points.csv", "n": n, "d": d, "name": ref.ref_dataset_name().decode(),
                  "n_pad": int(v.shape[0]), "d_pad": int(v.shape[1]), "bits": v[:n, :d].tolist()}

    # error texts of the builder
    ragged = os.path.join(HERE, "_ragged.csv")
    with open(ragged, "w") as f:
        f.write("1,2,3\n4,5\n")
    assert ref.ref_build_file(ragged.encode(), 64, 256) == 1
    out["ragged_error"] = ref.ref_last_error().decode()
    os.remove(ragged)
    empty = os.path.join(HERE, "_empty.csv")
    open(empty, "w").close()
    assert ref.ref_build_file(empty.encode(), 64, 256) == 1
    out["empty_error"] = ref.ref_last_error().decode()
    os.remove(empty)

    with open(os.path.join(HERE, "reference_loader.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote reference_loader.json")
    speed_result_records()


def speed_result_records(reference="/root/reference"):
    """Records of the reference's stored experiment results (plain JSON data): the cells of the size x
    dimensionality sweep that are small enough to re-run in a test and whose pair counts do not depend on
    the A100's rounding (D <= 256: exactly the self pairs), plus one record of the selectivity
    experiment for its schema."""
    base = os.path.join(reference, "results", "speed_results")
    with open(os.path.join(base, "ExpoDataSpeedVsSize_OnDemandRasterizer.json")) as f:
        sweep = json.load(f)
    with open(os.path.join(base, "selectivityVsSpeed.json")) as f:
        selectivity = json.load(f)
    keep = [r for r in sweep if r["iteration"] == 0 and r["results"]["inputProblemShape"]["m"] <= 2200
            and r["results"]["inputProblemShape"]["k"] <= 256]
    out = {"source": "results/speed_results/ExpoDataSpeedVsSize_OnDemandRasterizer.json (records with iteration 0, "
                     "N <= 2200, D <= 256) and the first record of selectivityVsSpeed.json",
           "sweep": keep, "selectivity_record": selectivity[0]}
    with open(os.path.join(HERE, "speed_results_records.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote speed_results_records.json")


if __name__ == "__main__":
    main()
