"""GPU parity over seeded random shapes: every entry point against the CPU checker and against each other
on point counts around the 256-point tile edges and dimensionalities around the 64-wide slab edges."""
import numpy as np
import pytest

import oracle
from tests import datasets

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 17, 255, 256, 257, 300, 511, 512, 513, 700, 1023, 1025, 1500, 2049, 3000, 4097]
DIMS = [1, 7, 8, 24, 63, 64, 65, 100, 128, 129, 192, 256, 320, 500, 1000]


def cases(count=48, seed=2024):
    rng = np.random.default_rng(seed)
    return [(int(rng.choice(SIZES)), int(rng.choice(DIMS)), float(rng.choice([0.0, 1, 5, 40])), int(rng.integers(1 << 30)))
            for _ in range(count)]


@pytest.mark.parametrize("tile_rows", ["auto", "256", "128"])  # the library's choice, then each tile height forced
@pytest.mark.parametrize("n,d,neighbours,seed", cases())
def test_random_shape(n, d, neighbours, seed, tile_rows, monkeypatch):
    import torch

    if tile_rows == "auto":
        monkeypatch.delenv("FASTED_TILE_ROWS", raising=False)
    else:
        monkeypatch.setenv("FASTED_TILE_ROWS", tile_rows)

    import fasted_amd
    from fasted_amd import find_pairs as fp

    bits = datasets.uniform_bytes(n, d, seed=seed)
    eps = datasets.epsilon_for_neighbours(bits, neighbours) if (neighbours > 0 and n > 50) else 0.0
    got, found = fasted_amd.self_join(bits, eps)
    assert found == len(got)
    rep = oracle.epsilon_band_report(bits, got, eps, n=n)
    assert rep["outside_band"] == 0 and rep["both"] >= n, rep  # inside the band, every self pair present
    listed = {tuple(p) for p in got}
    assert all((c, q) in listed for q, c in got[:2000])  # closed under swapping q and c
    if d % 64 == 0 and n > 1:
        pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
        cap = len(got) + 16
        buf = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
        st = fasted_amd.self_join_device(pts.data_ptr(), n, d, d, eps, buf.data_ptr(), cap,
                                         flags=fp.FASTED_SORT_PAIRS | fp.FASTED_SYMMETRIC)
        assert st.pairsFound == found and np.array_equal(buf[: st.pairsStored].cpu().numpy(), got)
        nq = max(1, n // 3)  # first third against the rest, as two sets
        st2 = fasted_amd.join_device(pts.data_ptr(), nq, d, pts[nq:].data_ptr(), n - nq, d, d, eps, buf.data_ptr(), cap)
        want = got[(got[:, 0] < nq) & (got[:, 1] >= nq)] - np.array([0, nq], dtype=np.int32)
        assert np.array_equal(buf[: st2.pairsStored].cpu().numpy(), want)
    if n > 600:
        blocked, found_blocked = fasted_amd.self_join_blocked(bits, eps, 256 * (1 + seed % 3))
        assert found_blocked == found and np.array_equal(blocked, got)
