"""GPU tests at the benchmark configurations' full sizes.  A full FP64 join is out of reach there,
so these check size-independent properties of the pair list (sorted, duplicate free, symmetric, every
self pair present, nothing lost) and compare a seeded sample of query rows against FP64 distances
with the epsilon-band rule: a pair may disagree with FP64 only if |d - eps| / eps <= 1e-3."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

BAND = 1e-3


@pytest.fixture(scope="module")
def env():
    import torch

    import bench
    import fasted_amd

    fasted_amd.load_findpairs()
    return torch, bench, fasted_amd


def run_config(env, name, n=None, sample_rows=256, oracle_rows=0):
    torch, bench, fasted = env
    n0, d, kind, neighbours, _ = bench.CONFIGS[name]
    n = n or n0
    pts = bench.generate_points(torch, kind, n, d, seed=777 + d)
    eps = bench.calibrate_epsilon(torch, pts, neighbours, sample=512)
    cap = int(max(n * 64, 2.0 * n * (neighbours + 1)))
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap)
    print(f"{name}: N={n} D={d} eps={eps:.6g} found={st.pairsFound} neighbours/point={(st.pairsFound - n) / n:.1f} "
          f"join={st.joinMs:.1f} ms ({2.0 * n * n * d / st.joinMs / 1e9:.0f} TFLOPS) sort={st.sortMs:.1f} ms")
    assert st.pairsFound == st.pairsStored <= cap, "pair buffer overflowed: nothing may be lost here"
    got = pairs[: st.pairsStored]
    q, c = got[:, 0].to(torch.int64), got[:, 1].to(torch.int64)

    # sorted row-major, hence duplicate free
    keys = q * n + c
    assert bool((keys[1:] > keys[:-1]).all())
    del keys
    assert int(q.min()) >= 0 and int(q.max()) < n and int(c.min()) >= 0 and int(c.max()) < n
    # every self pair is there
    assert int((q == c).sum()) == n
    # symmetric: the multiset of (c, q) equals the multiset of (q, c)
    swapped = torch.sort(c * n + q).values
    assert bool((swapped == q * n + c).all())
    del swapped
    # neighbours per point in the right ballpark of the calibration target
    mean_nb = (st.pairsFound - n) / n
    assert 0.25 * neighbours < mean_nb < 4.0 * neighbours, mean_nb

    # seeded sample of query rows against FP64 distances to all points (computed in chunks)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    rows = torch.sort(torch.randperm(n, generator=g, device="cuda")[:sample_rows]).values
    xs = pts[rows].to(torch.float64)
    xs2 = (xs * xs).sum(1)
    start = torch.searchsorted(q.contiguous(), rows)
    stop = torch.searchsorted(q.contiguous(), rows + 1)
    got_mask = torch.zeros((len(rows), n), dtype=torch.bool, device="cuda")
    for i in range(len(rows)):
        got_mask[i, c[start[i]:stop[i]]] = True
    band_pairs, worst, outside = 0, 0.0, 0
    chunk = max(1, (1 << 26) // d)
    for c0 in range(0, n, chunk):
        y = pts[c0:c0 + chunk].to(torch.float64)
        d2 = (xs2[:, None] + (y * y).sum(1)[None, :] - 2.0 * (xs @ y.T)).clamp_min(0.0)
        truth = d2 <= eps * eps
        diff = truth != got_mask[:, c0:c0 + chunk]
        if bool(diff.any()):
            rel = (d2[diff].sqrt() - eps).abs() / eps
            band_pairs += int(diff.sum())
            worst = max(worst, float(rel.max()))
            outside += int((rel > BAND).sum())
    print(f"{name}: {sample_rows} sampled rows vs FP64: {band_pairs} pairs inside the band, "
          f"max relative distance error {worst:.2e}, outside the band {outside}")
    assert outside == 0

    # a few rows against the CPU checker as well (needs the points on the host)
    if oracle_rows:
        host = pts.cpu().numpy().view(np.uint16)
        r0 = int(rows[0])
        ref = oracle.self_join_f64(host, eps, n=n, rows=(r0, r0 + oracle_rows))
        lo = int(torch.searchsorted(q.contiguous(), torch.tensor([r0], device="cuda"))[0])
        hi = int(torch.searchsorted(q.contiguous(), torch.tensor([r0 + oracle_rows], device="cuda"))[0])
        mine = got[lo:hi].cpu().numpy()
        rep = oracle.epsilon_band_report(host, mine, eps, truth_pairs=ref, band=BAND)
        print(f"{name}: rows [{r0}, {r0 + oracle_rows}) vs CPU checker: {rep}")
        assert rep["outside_band"] == 0
    return st


def test_config2_low_dim_100k_x_128(env):
    run_config(env, "c2", sample_rows=1024, oracle_rows=64)


def test_config4_clustered_500k_x_960(env):
    run_config(env, "c4", sample_rows=1024, oracle_rows=4)


def test_config5_output_heavy_2m_x_384(env):
    st = run_config(env, "c5", sample_rows=1024, oracle_rows=4)
    assert st.pairsFound > 2e8  # the output-heavy case really is output heavy


def test_config3_headline_1m_x_4096(env):
    run_config(env, "c3", sample_rows=1024, oracle_rows=4)
