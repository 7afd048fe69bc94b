"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle."""
import ctypes

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


def device_join(fasted, bits, eps, cap=None, flags=1, d=None, ld=None):
    """bits: (n, ld) uint16 on host -> torch upload -> fasted_self_join_device."""
    import torch

    n = bits.shape[0]
    ld = bits.shape[1] if ld is None else ld
    d = ld if d is None else d
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = int(cap if cap is not None else max(1024, 300 * n))
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    sums = torch.empty(n, dtype=torch.float32, device="cuda")
    st = fasted.self_join_device(pts.data_ptr(), n, d, ld, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr(),
                                 flags=flags)
    torch.cuda.synchronize()
    return pairs[: st.pairsStored].cpu().numpy(), st, sums.cpu().numpy()


def check_against_fp64(bits, n, eps, got, band=1e-3):
    rep = oracle.epsilon_band_report(bits, got, eps, n=n, band=band)
    assert rep["outside_band"] == 0, rep
    return rep


@pytest.mark.parametrize("n,d", [(256, 64), (1000, 128), (4096, 128), (777, 4096), (3000, 960)])
def test_sum_squared_matches_oracle(fasted, n, d):
    import torch

    bits = datasets.exponential(n, d, seed=n + d)
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    sums = torch.zeros(n, dtype=torch.float32, device="cuda")
    fasted.sum_squared_device(pts.data_ptr(), n, d, d, sums.data_ptr())
    got = sums.cpu().numpy().astype(np.float64)
    exact = oracle.sum_squared(bits, "f64")
    # FP32 accumulation of exact squares: relative error bounded by D * 2^-24
    assert np.all(np.abs(got - exact) <= d * 2.0 ** -24 * exact + 1e-30)
    # the reference's sequential round-toward-zero fold lies in the same band below the exact value
    rz = oracle.sum_squared(bits, "rz").astype(np.float64)
    assert np.all(np.abs(got - rz) <= 2 * d * 2.0 ** -24 * exact + 1e-30)


def test_sum_squared_closed_form_integer_rows(fasted):
    """Row r holds the 64 consecutive integers from 64 r (tests/python/sumSquared/sumSquared.py of
    the reference); every partial sum is an integer below 2^24, so FP32 is exact in any order."""
    import torch

    rows, d = 32, 64
    vals = np.arange(rows * d, dtype=np.float64).reshape(rows, d)
    bits = oracle.quantize(vals)  # exact up to 2048
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    sums = torch.zeros(rows, dtype=torch.float32, device="cuda")
    fasted.sum_squared_device(pts.data_ptr(), rows, d, d, sums.data_ptr())
    expect = np.array([sum(v * v for v in range(64 * r, 64 * r + 64)) for r in range(rows)], dtype=np.float64)
    got = sums.cpu().numpy().astype(np.float64)
    assert np.array_equal(got[:6], expect[:6])  # rows whose running sums stay below 2^24
    assert np.allclose(got, expect, rtol=64 * 2.0 ** -24)


@pytest.mark.parametrize("n,d", [(256, 64), (512, 128), (300, 64), (1025, 192), (2048, 1024), (700, 1536), (1300, 2048)])
def test_integer_points_exact_pair_set(fasted, n, d):
    """Integer coordinates make every dot product exact, so the pair set must equal the FP64
    join bit for bit (epsilon^2 sits between two integers: no pair is near the threshold).  Tiles of up to 16
    slabs (D <= 1024) gather their hit bits in their last slab, longer ones screen their accumulators behind the
    k-loop: both kinds are here."""
    bits = datasets.small_integers(n, d, high=3, seed=7 * n + d)
    x = bits.view(np.float16).astype(np.float64)
    d2 = ((x[:64, None, :] - x[None, :64, :]) ** 2).sum(-1)
    target = np.sort(d2[np.triu_indices(64, 1)])[40]
    eps = float(np.sqrt(target + 0.5))
    got, st, _ = device_join(fasted, bits, eps)
    truth = oracle.self_join_f64(bits, eps)
    assert st.pairsFound == len(truth) and st.pairsStored == len(truth)
    assert np.array_equal(got, truth)


def test_identity_points(fasted):
    """Unit vectors e_i (the reference's GenerateIdentityMatrixPoints fixture, main.cu:113-131):
    distinct points are sqrt(2) apart, duplicates are at distance 0."""
    n, d = 512, 256
    x = np.zeros((n, d), dtype=np.float16)
    x[np.arange(n), np.arange(n) % d] = 1.0
    bits = x.view(np.uint16)
    got, st, _ = device_join(fasted, bits, 1.0)
    expect = np.array([(i, j) for i in range(n) for j in range(n) if i % d == j % d], dtype=np.int32)
    assert np.array_equal(got, expect)
    got, st, _ = device_join(fasted, bits, 1.5)
    assert st.pairsFound == n * n


def test_plumbing_config_full_fp64_check(fasted):
    """N=4096 x D=128 Exp(40) clipped to [0,1], ~32 neighbours/point, entire pair set vs FP64."""
    n, d = 4096, 128
    bits = datasets.exponential(n, d, seed=2024)
    eps = datasets.epsilon_for_neighbours(bits, 32)
    got, st, _ = device_join(fasted, bits, eps)
    rep = check_against_fp64(bits, n, eps, got)
    sel = (st.pairsFound - n) / n
    assert 20 < sel < 50, sel
    assert rep["both"] >= rep["truth_total"] - rep["band_pairs"]
    print("plumbing config:", rep, "selectivity", sel)
    # the reference's own arithmetic model (RZ norms, FP32 dot) agrees up to the same band
    model = oracle.self_join_f32(bits, eps)
    check_against_fp64(bits, n, eps, model)


@pytest.mark.parametrize("n,d", [(1, 64), (2, 64), (255, 64), (257, 128), (1000, 320), (5000, 64), (300, 16384), (513, 8000)])
def test_ragged_sizes(fasted, n, d):
    bits = datasets.uniform_bytes(n, d, seed=n)
    eps = datasets.epsilon_for_neighbours(bits, min(8, max(n - 1, 0) / 2)) if n > 2 else 0.5
    got, st, _ = device_join(fasted, bits, eps)
    check_against_fp64(bits, n, eps, got)
    assert st.pairsFound >= n  # every self pair is reported
    assert set(map(tuple, got[got[:, 0] == got[:, 1]])) == {(i, i) for i in range(n)}


def test_dimension_padding_through_host_entry(fasted):
    """D not a multiple of 64 goes through the host entry, which zero-pads on upload."""
    n, d = 700, 100
    bits = datasets.uniform_bytes(n, d, seed=5)
    eps = datasets.epsilon_for_neighbours(bits, 10)
    got, found = fasted.self_join(bits, eps)
    assert found == len(got)
    check_against_fp64(bits, n, eps, got)


def test_tiny_epsilon_reports_exactly_the_self_pairs(fasted):
    """eps = 0.001 on the seeded Exp(40) data finds exactly N pairs (the self pairs), the count the
    reference's ExpoDataSpeedVsSize_OnDemandRasterizer.json holds for D in {64,128,256}."""
    lib = fasted.load_findpairs()
    for n, d in [(1000, 64), (2154, 128), (1000, 256)]:
        r = lib.runFromExponentialDataset(n, d, 40.0, 10.0, 0.001, False)
        assert r.pairsFound == n and r.pairsStored == n
        assert (r.inputProblemShape.m, r.inputProblemShape.n, r.inputProblemShape.k) == (n, n, d)
        assert r.paddedProblemShape.k % 64 == 0 and r.paddedProblemShape.m % 256 == 0
    lib.releaseResources()


def test_pair_buffer_overflow_is_soft(fasted):
    """found keeps counting, stored stops at the capacity, nothing is written past it
    (source/pair.cuh:123-133)."""
    import torch

    n, d = 1024, 64
    bits = datasets.uniform_bytes(n, d, seed=3)
    eps = datasets.epsilon_for_neighbours(bits, 20)
    full, st_full, _ = device_join(fasted, bits, eps)
    cap = 1000
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    buf = torch.full((cap + 64, 2), -7, dtype=torch.int32, device="cuda")
    st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, buf.data_ptr(), cap, flags=0)
    assert st.pairsFound == st_full.pairsFound
    assert st.pairsStored == cap
    host = buf.cpu().numpy()
    assert (host[cap:] == -7).all()
    stored = {tuple(p) for p in host[:cap]}
    assert len(stored) == cap and stored <= {tuple(p) for p in full}


def test_rerun_changes_epsilon_on_resident_data(fasted):
    lib = fasted.load_findpairs()
    n, d = 3000, 128
    r0 = lib.runFromExponentialDataset(n, d, 40.0, 10.0, 0.3, False)
    np_, dp_, npad, dpad = (ctypes.c_int() for _ in range(4))
    ptr = lib.fasted_resident_points(ctypes.byref(np_), ctypes.byref(dp_), ctypes.byref(npad), ctypes.byref(dpad))
    bits = np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(ctypes.c_uint16)), (npad.value, dpad.value)).copy()
    assert (np_.value, dp_.value) == (n, d)
    assert np.array_equal(bits[:n, :d], oracle.quantize(oracle.exponential_points(n, d, 40.0, 10.0)))
    truth0 = oracle.self_join_f64(bits, 0.3, n=n)
    r1 = lib.reRun(0.33, False)
    truth1 = oracle.self_join_f64(bits, 0.33, n=n)
    assert abs(int(r0.pairsFound) - len(truth0)) <= max(4, len(truth0) // 1000)
    assert abs(int(r1.pairsFound) - len(truth1)) <= max(4, len(truth1) // 1000)
    assert r1.pairsFound > r0.pairsFound
    assert r0.TFLOPS > 0 and r0.totalTime > 0
    lib.releaseResources()


@pytest.mark.parametrize("nq,nc,d", [(300, 1000, 64), (1000, 300, 128), (257, 5000, 192), (4100, 513, 64)])
def test_two_set_join_matches_the_checker(fasted, nq, nc, d):
    """Queries and candidates from different sets (no forced pairs).  Checked by running the
    checker's self-join on the stacked sets and keeping the (query, candidate) block."""
    import torch

    both = datasets.uniform_bytes(nq + nc, d, seed=nq + nc)
    # plant exact duplicates across the two sets: distance 0 pairs must be found, none is forced
    both[nq + 5] = both[3]
    both[nq + 17] = both[nq - 1]
    eps = datasets.epsilon_for_neighbours(both, 6)
    q = torch.from_numpy(both[:nq].view(np.int16).copy()).cuda()
    c = torch.from_numpy(both[nq:].view(np.int16).copy()).cuda()
    cap = 200 * (nq + nc)
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    st = fasted.join_device(q.data_ptr(), nq, d, c.data_ptr(), nc, d, d, eps, pairs.data_ptr(), cap)
    got = pairs[: st.pairsStored].cpu().numpy()
    assert st.pairsFound == st.pairsStored
    stacked = oracle.self_join_f64(both, eps)
    block = stacked[(stacked[:, 0] < nq) & (stacked[:, 1] >= nq)].copy()
    block[:, 1] -= nq
    stats, diff, side = oracle.pair_stats(got, block, want_diff=True)
    # disagreements only inside the band (distances from the stacked data: shift the candidate index back)
    shifted = diff.copy()
    shifted[:, 1] += nq
    dist = oracle.pair_distances_f64(both, shifted)
    assert np.all(np.abs(dist - eps) / eps <= 1e-3), (stats, dist)
    assert {(3, 5), (nq - 1, 17)} <= {tuple(p) for p in got}
    assert stats["both"] > 0


@pytest.mark.parametrize("n,d", [(700, 64), (2048, 128), (5000, 192)])
def test_symmetric_option_gives_the_same_pair_set(fasted, n, d):
    """FASTED_SYMMETRIC computes only the tiles on and above the diagonal and mirrors the pairs: the
    sorted pair list must be identical to the default full computation."""
    from fasted_amd import find_pairs as fp

    bits = datasets.uniform_bytes(n, d, seed=3 * n + d)
    eps = datasets.epsilon_for_neighbours(bits, 12)
    full, st_full, _ = device_join(fasted, bits, eps)
    half, st_half, _ = device_join(fasted, bits, eps, flags=fp.FASTED_SORT_PAIRS | fp.FASTED_SYMMETRIC)
    assert st_half.pairsFound == st_full.pairsFound
    assert np.array_equal(half, full)
    check_against_fp64(bits, n, eps, half)


@pytest.mark.parametrize("n,d,block", [(3000, 100, 1024), (2600, 64, 256), (1500, 192, 4096), (5000, 128, 1000)])
def test_blocked_join_equals_the_whole_join(fasted, n, d, block):
    """The dataset streamed through the device in row blocks gives the pair list of the one-shot join,
    record for record (same arithmetic per pair, row-major order across the blocks)."""
    bits = datasets.uniform_bytes(n, d, seed=11 * n + d)
    eps = datasets.epsilon_for_neighbours(bits, 15)
    whole, found_whole = fasted.self_join(bits, eps)
    blocked, found_blocked = fasted.self_join_blocked(bits, eps, block)
    assert found_blocked == found_whole == len(whole)
    assert np.array_equal(blocked, whole)
    check_against_fp64(bits, n, eps, blocked)


def test_blocked_join_overflow_is_soft(fasted):
    n, d = 2000, 64
    bits = datasets.uniform_bytes(n, d, seed=21)
    eps = datasets.epsilon_for_neighbours(bits, 20)
    whole, found_whole = fasted.self_join(bits, eps)
    cap = len(whole) // 3
    part, found = fasted.self_join_blocked(bits, eps, 512, cap=cap)
    assert found == found_whole and len(part) == cap
    assert np.array_equal(part, whole[:cap])  # row-major prefix: the first query blocks come first


def test_pair_distances_match_fp64(fasted):
    """Distance column of a pair list: FP32 sum of squared differences against the FP64 checker; every
    reported pair lies within epsilon (up to the band); a pair naming a missing point yields NaN."""
    import torch

    n, d = 1500, 192
    bits = datasets.uniform_bytes(n, d, seed=77)
    eps = datasets.epsilon_for_neighbours(bits, 12)
    got, st, _ = device_join(fasted, bits, eps)
    want = oracle.pair_distances_f64(bits, got)
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    pairs = torch.from_numpy(np.vstack([got, [[n, 0]], [[0, -1]]]).astype(np.int32)).cuda()
    dist = torch.full((len(got) + 2,), -1.0, dtype=torch.float32, device="cuda")
    fasted.pair_distances_device(pts.data_ptr(), n, d, pts.data_ptr(), n, d, d, pairs.data_ptr(), len(got) + 2,
                                 dist.data_ptr())
    host = dist.cpu().numpy()
    assert np.isnan(host[-2:]).all()
    assert np.allclose(host[:-2], want, rtol=2e-6, atol=1e-6)  # FP32 accumulation of <= 192 exact-ish terms
    assert (host[:-2] <= eps * (1 + 1e-3)).all()
    self_pairs = got[:, 0] == got[:, 1]
    assert (host[:-2][self_pairs] == 0).all()

    # two different sets, ragged sizes and row strides
    nq, nc = 300, 1000
    q_bits, c_bits = bits[:nq], bits[n - nc:]
    some = np.array([[0, 0], [299, 999], [17, 503]], dtype=np.int32)
    qd, cd = (torch.from_numpy(b.view(np.int16).copy()).cuda() for b in (q_bits, c_bits))
    out = torch.empty(3, dtype=torch.float32, device="cuda")
    fasted.pair_distances_device(qd.data_ptr(), nq, d, cd.data_ptr(), nc, d, d, torch.from_numpy(some).cuda().data_ptr(), 3,
                                 out.data_ptr())
    both = np.vstack([q_bits, c_bits])
    want2 = oracle.pair_distances_f64(both, some + np.array([0, nq], dtype=np.int32))
    assert np.allclose(out.cpu().numpy(), want2, rtol=2e-6)


def test_caller_stream_and_repeatability(fasted):
    """The device entry on a stream of the caller's: work queued on that stream before the call is seen,
    the call returns with the stream drained (it sorts, and the sort waits for the stream), and repeated calls
    give the same sorted list."""
    import torch

    n, d = 3000, 128
    bits = datasets.uniform_bytes(n, d, seed=99)
    eps = datasets.epsilon_for_neighbours(bits, 10)
    want, st_want, _ = device_join(fasted, bits, eps)
    stream = torch.cuda.Stream()  # default priority
    cap = 300 * n
    host = torch.from_numpy(bits.view(np.int16).copy()).pin_memory()
    with torch.cuda.stream(stream):
        pts = torch.empty((n, d), dtype=torch.int16, device="cuda")
        pts.copy_(host, non_blocking=True)  # still in flight on `stream` when the join is queued behind it
        pairs = torch.full((cap, 2), -1, dtype=torch.int32, device="cuda")
        runs = []
        for _ in range(3):
            st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, stream=stream.cuda_stream)
            assert stream.query()  # nothing left on the stream: the sort synchronised it
            runs.append(pairs[: st.pairsStored].cpu().numpy().copy())
    torch.cuda.synchronize()
    assert st.pairsFound == st_want.pairsFound
    for got in runs:
        assert np.array_equal(got, want)


def test_points_with_infinite_coordinates_pair_with_nothing_but_themselves(fasted):
    """Values beyond the FP16 range quantise to infinity (source/DataLoader/PointListBuilder.hpp:57-73); the
    distances of such a point are NaN or infinite, every comparison with them is false
    (source/warpMma.cuh:257), so it has no neighbours; only its self pair is reported (forced here)."""
    n, d = 1200, 64
    bits = datasets.uniform_bytes(n, d, seed=123)
    eps = datasets.epsilon_for_neighbours(bits, 25)
    odd = [5, 300, 777, 1199]
    spoiled = bits.copy()
    for k, i in enumerate(odd):
        spoiled[i, (7 * k) % d] = 0x7C00 if k % 2 == 0 else 0xFC00  # +inf / -inf
    got, st, _ = device_join(fasted, spoiled, eps)
    clean, _, _ = device_join(fasted, bits, eps)
    keep = ~(np.isin(clean[:, 0], odd) | np.isin(clean[:, 1], odd))
    want = oracle.sort_pairs(np.vstack([clean[keep], [[i, i] for i in odd]]).astype(np.int32))
    assert np.array_equal(got, want)


def test_padding_columns_are_checked(fasted):
    """D % 64 != 0: the device entries read whole 64-wide slabs, so the padding columns must be zeros;
    fasted_check_padding_device counts the rows where they are not."""
    import torch

    n, d, ld = 700, 40, 64
    bits = np.zeros((n, ld), dtype=np.uint16)
    bits[:, :d] = datasets.exponential(n, d, seed=3)
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    assert fasted.check_padding_device(pts.data_ptr(), n, d, ld) == 0
    bits[5, 41] = 0x3C00   # 1.0 in a padding column
    bits[699, 63] = 0x0001  # the smallest subnormal
    bits[9, 50] = 0x8000   # -0.0 is as good as zero
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    assert fasted.check_padding_device(pts.data_ptr(), n, d, ld) == 2
    assert fasted.check_padding_device(pts.data_ptr(), n, 64, ld) == 0  # no padding columns at all


def test_join_is_deterministic_over_many_tiles_per_workgroup(fasted):
    """Every workgroup walks hundreds of tiles here, with the next tile's operands in flight during each
    epilogue: two runs must give the same pair set (a transfer that a barrier did not wait for shows up as a
    few pairs that differ from run to run), and sampled rows must agree with FP64."""
    import torch

    n, d = 90000, 192
    g = torch.Generator(device="cuda")
    g.manual_seed(1234)
    centers = torch.rand((300, d), generator=g, device="cuda")
    which = torch.randint(0, 300, (n,), generator=g, device="cuda")
    pts = (centers[which] + 0.05 * torch.randn((n, d), generator=g, device="cuda")).to(torch.float16)
    x = pts[:2048].double()
    d2 = ((x * x).sum(1)[:, None] + (x * x).sum(1)[None, :] - 2.0 * x @ x.T)
    eps = float(torch.quantile(d2[d2 > 1e-6].flatten()[:1 << 20], 0.004).sqrt())
    cap = 400 * n
    keys = []
    for _ in range(2):
        pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
        st = fasted.self_join_device(pts.view(torch.int16).data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, flags=0)
        assert st.pairsFound == st.pairsStored > 10 * n
        got = pairs[: st.pairsStored]
        keys.append(torch.sort(got[:, 0].to(torch.int64) * n + got[:, 1].to(torch.int64)).values)
        del pairs
    assert keys[0].shape == keys[1].shape and bool((keys[0] == keys[1]).all())
    rows = torch.arange(0, n, n // 256, device="cuda")[:256]
    xs = pts[rows].double()
    d2 = ((xs * xs).sum(1)[:, None] + (pts.double() ** 2).sum(1)[None, :] - 2.0 * xs @ pts.double().T).clamp_min(0)
    truth = d2 <= eps * eps
    mask = torch.zeros_like(truth)
    q, c = keys[0] // n, keys[0] % n
    sel = torch.isin(q, rows)
    mask[torch.searchsorted(rows, q[sel]), c[sel]] = True
    diff = truth != mask
    rel = (d2[diff].sqrt() - eps).abs() / eps
    assert int((rel > 1e-3).sum()) == 0, (int(diff.sum()), float(rel.max()))


def test_tall_tile_order_exact_pair_sets(fasted):
    """From 64 x 64 tiles on, the work queues walk super-squares of 32 x 8 tiles.  Integer coordinates make the
    join exact, so on a ragged matrix of 65 x 65 tiles the default order, the symmetric option (upper part of
    the tall super-squares, mirrored) and a rectangular two-set join (65 x 3 tiles: most super-square positions
    are padding) must each give exactly the pair list of a blockwise FP64 computation."""
    import torch
    from fasted_amd import find_pairs as fp

    n, d, nc = 64 * 256 + 37, 64, 600
    bits = datasets.small_integers(n, d, high=3, seed=91)
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    x = pts.view(torch.float16).double()
    norms = (x * x).sum(1)
    d2_head = norms[:64, None] + norms[None, :64] - 2.0 * x[:64] @ x[:64].T
    target = torch.sort(d2_head[torch.triu_indices(64, 64, 1).unbind()]).values[30]
    eps = float(torch.sqrt(target + 0.5))

    def truth(cols):
        out = []
        for r0 in range(0, n, 4096):
            blk = norms[r0:r0 + 4096, None] + norms[None, :cols] - 2.0 * x[r0:r0 + 4096] @ x[:cols].T
            q, c = torch.nonzero(blk <= eps * eps, as_tuple=True)
            out.append(torch.stack([q + r0, c], 1))
        return torch.cat(out).to(torch.int32)

    want = truth(n)
    cap = int(want.shape[0]) + 1024
    for flags in (fp.FASTED_SORT_PAIRS, fp.FASTED_SORT_PAIRS | fp.FASTED_SYMMETRIC):
        pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
        st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, flags=flags)
        assert st.pairsFound == st.pairsStored == want.shape[0]
        assert bool((pairs[: st.pairsStored] == want).all())
    want2 = truth(nc)
    pairs = torch.empty((int(want2.shape[0]) + 1024, 2), dtype=torch.int32, device="cuda")
    st = fasted.join_device(pts.data_ptr(), n, d, pts.data_ptr(), nc, d, d, eps, pairs.data_ptr(), pairs.shape[0])
    assert st.pairsFound == st.pairsStored == want2.shape[0]
    assert bool((pairs[: st.pairsStored] == want2).all())


@pytest.mark.parametrize("n,d", [(300, 64), (1025, 192), (2154, 128), (4642, 64), (64 * 128 + 37, 64)])
def test_both_tile_heights_give_the_exact_pair_set(fasted, n, d, monkeypatch):
    """Matrices of few tiles are cut into tiles of 128 query rows instead of 256 (FASTED_TILE_ROWS forces either).
    Integer coordinates make the join exact: both heights, on a self-join, on a two-set join with a ragged
    query count and with non-finite points present, must give exactly the FP64 pair list.  The last shape has
    65 tile rows of 128: the tall tile order with that height."""
    import torch

    bits = datasets.small_integers(n, d, high=3, seed=3 * n + d)
    x = bits.view(np.float16).astype(np.float64)
    d2 = ((x[:64, None, :] - x[None, :64, :]) ** 2).sum(-1)
    eps = float(np.sqrt(np.sort(d2[np.triu_indices(64, 1)])[40] + 0.5))
    truth = oracle.self_join_f64(bits, eps)
    nq = n - 131  # a ragged query set against the first 700 points (or all of them)
    nc = min(n, 700)
    truth2 = truth[(truth[:, 0] < nq) & (truth[:, 1] < nc)]
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    for rows in ("256", "128"):
        monkeypatch.setenv("FASTED_TILE_ROWS", rows)
        got, st, _ = device_join(fasted, bits, eps)
        assert st.pairsFound == len(truth) and np.array_equal(got, truth), rows
        buf = torch.empty((len(truth2) + 64, 2), dtype=torch.int32, device="cuda")
        st2 = fasted.join_device(pts.data_ptr(), nq, d, pts.data_ptr(), nc, d, d, eps, buf.data_ptr(), buf.shape[0])
        assert st2.pairsFound == len(truth2) and np.array_equal(buf[: st2.pairsStored].cpu().numpy(), truth2), rows
    # a point with an infinite coordinate pairs with nothing but itself, under both heights
    bad = bits.copy()
    bad[5, 0] = 0x7C00
    keep = truth[(truth[:, 0] != 5) & (truth[:, 1] != 5)]
    want = np.concatenate([keep, np.array([[5, 5]], dtype=np.int32)])
    want = want[np.lexsort((want[:, 1], want[:, 0]))]
    for rows in ("256", "128"):
        monkeypatch.setenv("FASTED_TILE_ROWS", rows)
        got, st, _ = device_join(fasted, bad, eps)
        assert np.array_equal(got, want), rows


def test_small_joins_time_themselves_with_the_device_clock(fasted):
    """Joins of at most 512 tiles are timed by clock readings of the kernels themselves instead of events: the two
    times must be positive, add up to less than the wall time of the call, and agree with the event-timed figure
    of the same kernel on a matrix just large enough to be timed with events (same D, per-tile time within 3x: a
    check of the unit of the clock, not of the speed)."""
    import time

    import torch

    n, d = 4096, 128
    bits = datasets.exponential(n, d, seed=2024)
    eps = datasets.epsilon_for_neighbours(bits, 32)
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = 300 * n
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    best = None
    for _ in range(20):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, flags=0)
        wall_ms = (time.perf_counter() - t0) * 1000.0
        assert st.sumSquaredMs > 0.0 and st.joinMs > 0.0
        assert st.sumSquaredMs + st.joinMs < wall_ms
        best = st.joinMs if best is None else min(best, st.joinMs)
    assert 0.003 < best < 0.2, best  # 256 tiles of two slabs: some tens of microseconds
    # the same join timed with events on the stream (FASTED_EVENT_TIMING): the dispatch as the command processor
    # sees it, a little longer than first instruction to last sign-off, and the same pairs
    from fasted_amd import find_pairs as fp

    timed = [fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, flags=fp.FASTED_EVENT_TIMING)
             for _ in range(10)]
    assert all(t.pairsFound == st.pairsFound for t in timed)
    by_events = min(t.joinMs for t in timed)
    assert 0.5 * best < by_events < 5.0 * best, (best, by_events)
    # event-timed neighbour: 6000 points = 576 tiles
    big = datasets.exponential(6000, d, seed=3)
    ptsb = torch.from_numpy(big.view(np.int16).copy()).cuda()
    pb = torch.empty((300 * 6000, 2), dtype=torch.int32, device="cuda")
    tb = min(fasted.self_join_device(ptsb.data_ptr(), 6000, d, d, eps, pb.data_ptr(), pb.shape[0], flags=0).joinMs
             for _ in range(10))
    per_tile_small, per_tile_big = best / 1.0, tb / 3.0  # one round of the 256 workgroups against three
    assert 1.0 / 3.0 < per_tile_small / per_tile_big < 3.0, (best, tb)


def test_small_join_results_are_complete_for_a_reader_on_another_stream(fasted):
    """A join of at most 512 tiles returns when the join kernel's last workgroup has reported to the host, before
    the stream reports idle.  The pair records and the squared norms must be in device memory by then for a reader
    that is not ordered behind the join's stream: each of many unsorted joins on the default stream is read back
    at once through a copy on a second, non-blocking stream, from a buffer that was overwritten in between."""
    import torch

    n, d = 4096, 128
    bits = datasets.uniform_bytes(n, d, seed=321)
    eps = datasets.epsilon_for_neighbours(bits, 24)
    want, st_want, sums_want = device_join(fasted, bits, eps)  # sorted, fully synchronised
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = int(st_want.pairsFound) + 1024
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    sums = torch.empty(n, dtype=torch.float32, device="cuda")
    host_pairs = torch.empty((cap, 2), dtype=torch.int32).pin_memory()
    host_sums = torch.empty(n, dtype=torch.float32).pin_memory()
    reader = torch.cuda.Stream()  # default priority
    key = lambda a: a[:, 0].astype(np.int64) * n + a[:, 1]
    want_keys = key(want)
    for it in range(100):
        pairs.fill_(-1)
        sums.fill_(-1.0)
        torch.cuda.synchronize()
        st = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap, sums_ptr=sums.data_ptr(), flags=0)
        with torch.cuda.stream(reader):
            host_pairs.copy_(pairs, non_blocking=True)
            host_sums.copy_(sums, non_blocking=True)
        reader.synchronize()
        assert st.pairsFound == st_want.pairsFound == st.pairsStored, it
        got = host_pairs[: st.pairsStored].numpy()
        assert np.array_equal(np.sort(key(got)), want_keys), it
        assert np.array_equal(host_sums.numpy(), sums_want), it
