"""fasted_self_join_device_noalloc (scratch in a device array of the library image, no allocation in the
call) against fasted_self_join_device on the same inputs, through the C ABI: the same pair set record for
record (integer work: bit-exact after ordering), the same counts, the same squared norms effect.  Two
calls in a row, the second on a smaller input, so that what the first call left in the shared array
(queue heads, pair counter, norms of rows the second call does not have) must not leak into the second."""
import numpy as np
import pytest

from tests import datasets

pytestmark = pytest.mark.gpu


def _row_major(pairs):
    return pairs[np.lexsort((pairs[:, 1], pairs[:, 0]))]


def _both_entries(fasted, torch, bits, eps):
    n, d = bits.shape
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = 300 * n
    expected = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    ref = fasted.self_join_device(pts.data_ptr(), n, d, d, eps, expected.data_ptr(), cap, flags=1)
    got = torch.full((cap, 2), -1, dtype=torch.int32, device="cuda")
    st = fasted.self_join_device_noalloc(pts.data_ptr(), n, d, d, eps, got.data_ptr(), cap)
    torch.cuda.synchronize()
    assert st.pairsFound == ref.pairsFound and st.pairsStored == ref.pairsStored
    assert st.pairsStored == st.pairsFound  # the buffer was large enough: the whole set is compared
    want = expected[: ref.pairsStored].cpu().numpy()
    have = _row_major(got[: st.pairsStored].cpu().numpy())
    assert np.array_equal(have, want)
    assert bool((got[st.pairsStored:] == -1).all())  # nothing written past the stored pairs
    return st


def test_no_alloc_entry_matches_the_allocating_entry_twice_in_a_row():
    import torch

    import fasted_amd

    fasted_amd.load_findpairs()
    big = datasets.exponential(3000, 192, seed=5)
    eps_big = datasets.epsilon_for_neighbours(big, 12)
    first = _both_entries(fasted_amd, torch, big, eps_big)
    assert first.pairsFound > 3000 * 5
    small = datasets.uniform_bytes(700, 128, seed=6)
    eps_small = datasets.epsilon_for_neighbours(small, 20)
    second = _both_entries(fasted_amd, torch, small, eps_small)
    assert 700 * 5 < second.pairsFound < first.pairsFound


def test_no_alloc_entry_refuses_what_it_cannot_do():
    import torch

    import fasted_amd
    from fasted_amd.find_pairs import FastedError

    fasted_amd.load_findpairs()
    pts = torch.zeros((256, 64), dtype=torch.int16, device="cuda")
    pairs = torch.empty((1024, 2), dtype=torch.int32, device="cuda")
    with pytest.raises(FastedError, match="at most 4194304 points"):
        fasted_amd.self_join_device_noalloc(pts.data_ptr(), (1 << 22) + 1, 64, 64, 0.1, pairs.data_ptr(), 1024)
    with pytest.raises(FastedError, match="cannot sort"):
        fasted_amd.self_join_device_noalloc(pts.data_ptr(), 256, 64, 64, 0.1, pairs.data_ptr(), 1024, flags=1)
