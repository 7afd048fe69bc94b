"""GPU parity tests of mid-size matrices: more tiles than two rounds of the workgroups (so the tiles come from the
per-XCD work queues, not one workgroup per tile), fewer than 64 tile rows (the 16 x 16 super-square order), several
slabs per tile.  The size band of the reference's own sweep rows of 10 000 and 21 544 points
(results/speed_results/ExpoDataSpeedVsSize_OnDemandRasterizer.json); kernel counterpart
source/findPairs.cuh:360-546 with source/rasterizer/onDemandRasterizer.cuh:78-108."""
import numpy as np
import pytest

import oracle
from tests import datasets

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fasted():
    import fasted_amd

    fasted_amd.load_findpairs()
    return fasted_amd


def integer_case(n, d, seed, rank=10):
    """Integer coordinates (every product and sum exact in FP32) and an epsilon whose square lies half-way between
    two integers: the pair list must equal the FP64 checker's record for record."""
    bits = datasets.small_integers(n, d, high=3, seed=seed)
    x = bits[:64].view(np.float16).astype(np.float64)
    d2 = ((x[:, None, :] - x[None, :, :]) ** 2).sum(-1)
    eps = float(np.sqrt(np.sort(d2[np.triu_indices(64, 1)])[rank] + 0.5))
    return bits, eps


@pytest.mark.parametrize("n,d", [(7000, 128), (7000, 320), (12000, 128), (12000, 320)])
def test_queue_mode_exact_pair_lists(fasted, n, d, monkeypatch):
    """784 and 2209 tiles of 256 rows (1540 and 4418 of 128 rows, the latter in the tall order): default and
    symmetric, both tile heights, with and without squared norms brought by the caller."""
    import torch
    from fasted_amd import find_pairs as fp

    bits, eps = integer_case(n, d, seed=n + d)
    truth = oracle.self_join_f64(bits, eps)
    assert len(truth) > 2 * n  # off-diagonal pairs are what is being checked
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = len(truth) + 1024
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    sums = torch.empty(n, dtype=torch.float32, device="cuda")
    fasted.sum_squared_device(pts.data_ptr(), n, d, d, sums.data_ptr())
    for rows in ("256", "128"):
        monkeypatch.setenv("FASTED_TILE_ROWS", rows)
        for flags in (fp.FASTED_SORT_PAIRS, fp.FASTED_SORT_PAIRS | fp.FASTED_SYMMETRIC,
                      fp.FASTED_SORT_PAIRS | fp.FASTED_SKIP_SUMS):
            pairs.fill_(-1)
            st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr(),
                                         flags=flags)
            assert st.pairsFound == st.pairsStored == len(truth), (rows, flags)
            assert np.array_equal(pairs[: st.pairsStored].cpu().numpy(), truth), (rows, flags)


def test_queue_mode_two_set_exact_pair_list(fasted, monkeypatch):
    """6000 queries x 9000 candidates: 24 x 36 = 864 tiles (47 x 36 of 128 rows), none forced."""
    import torch
    from fasted_amd import find_pairs as fp

    nq, nc, d = 6000, 9000, 192
    bits, eps = integer_case(nq + nc, d, seed=77)
    stacked = oracle.self_join_f64(bits, eps)
    want = stacked[(stacked[:, 0] < nq) & (stacked[:, 1] >= nq)].copy()
    want[:, 1] -= nq
    assert len(want) > nq
    q = torch.from_numpy(bits[:nq].view(np.int16).copy()).cuda()
    c = torch.from_numpy(bits[nq:].view(np.int16).copy()).cuda()
    cap = len(want) + 1024
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    sq = torch.empty(nq, dtype=torch.float32, device="cuda")
    sc = torch.empty(nc, dtype=torch.float32, device="cuda")
    fasted.sum_squared_device(q.data_ptr(), nq, d, d, sq.data_ptr())
    fasted.sum_squared_device(c.data_ptr(), nc, d, d, sc.data_ptr())
    for rows in ("256", "128"):
        monkeypatch.setenv("FASTED_TILE_ROWS", rows)
        for flags in (fp.FASTED_SORT_PAIRS, fp.FASTED_SORT_PAIRS | fp.FASTED_SKIP_SUMS):
            pairs.fill_(-1)
            st = fasted.join_device(q.data_ptr(), nq, d, c.data_ptr(), nc, d, d, eps, pairs.data_ptr(), cap, flags=flags,
                                    sums_queries_ptr=sq.data_ptr(), sums_candidates_ptr=sc.data_ptr())
            assert st.pairsFound == st.pairsStored == len(want), (rows, flags)
            assert np.array_equal(pairs[: st.pairsStored].cpu().numpy(), want), (rows, flags)


def test_queue_mode_band_check_exponential_10000x1024(fasted):
    """Exp(40) data of the headline kind at 10 000 x 1024 (1600 tiles, 16 slabs): the whole pair set against the
    FP64 checker under the relative 1e-3 band rule, default and symmetric."""
    import torch
    from fasted_amd import find_pairs as fp

    n, d = 10000, 1024
    bits = datasets.exponential(n, d, seed=31)
    eps = datasets.epsilon_for_neighbours(bits, 16)
    truth = oracle.self_join_f64(bits, eps)
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = 4 * len(truth)
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    lists = []
    for flags in (fp.FASTED_SORT_PAIRS, fp.FASTED_SORT_PAIRS | fp.FASTED_SYMMETRIC):
        st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, flags=flags)
        got = pairs[: st.pairsStored].cpu().numpy()
        rep = oracle.epsilon_band_report(bits, got, eps, truth_pairs=truth)
        assert rep["outside_band"] == 0, rep
        assert 8 < (st.pairsFound - n) / n < 32
        lists.append(got)
        print("10000 x 1024:", rep)
    assert np.array_equal(lists[0], lists[1])


def test_skip_sums_needs_the_buffers_and_gives_the_same_list(fasted):
    """FASTED_SKIP_SUMS: the caller's squared norms (from fasted_sum_squared_device) are read instead of computed;
    same pair list as the default on ordinary data; refused without a buffer."""
    import torch
    from fasted_amd import find_pairs as fp

    n, d = 3000, 192
    bits = datasets.uniform_bytes(n, d, seed=8)
    eps = datasets.epsilon_for_neighbours(bits, 12)
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = 300 * n
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    sums = torch.empty(n, dtype=torch.float32, device="cuda")
    st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr())
    want = pairs[: st.pairsStored].cpu().numpy().copy()
    assert np.allclose(sums.cpu().numpy(), oracle.sum_squared(bits, "f64"), rtol=d * 2.0 ** -24)
    fasted.sum_squared_device(pts.data_ptr(), n, d, d, sums.data_ptr())
    pairs.fill_(-1)
    st2 = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr(),
                                  flags=fp.FASTED_SORT_PAIRS | fp.FASTED_SKIP_SUMS)
    assert st2.pairsFound == st.pairsFound
    assert np.array_equal(pairs[: st2.pairsStored].cpu().numpy(), want)
    # an infinite squared norm handed in by the caller: that point pairs with nothing but itself
    spoiled = sums.clone()
    spoiled[17] = float("inf")
    st3 = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=spoiled.data_ptr(),
                                  flags=fp.FASTED_SORT_PAIRS | fp.FASTED_SKIP_SUMS)
    got3 = pairs[: st3.pairsStored].cpu().numpy()
    keep = want[(want[:, 0] != 17) & (want[:, 1] != 17)]
    expect = oracle.sort_pairs(np.vstack([keep, [[17, 17]]]).astype(np.int32))
    assert np.array_equal(got3, expect)
    with pytest.raises(fp.FastedError):
        fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=None,
                                flags=fp.FASTED_SKIP_SUMS)
