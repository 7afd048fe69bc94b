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


def test_no_alloc_entry_leaves_the_free_device_memory_unchanged_and_needs_no_library_workspace():
    """The property the entry exists for: after the library has dropped everything it ever allocated
    (releaseResources: resident data, workspace, pair and sort buffers), the call still works -- it uses none of
    it -- and the free device memory reported by the driver is the same before and after further calls."""
    import torch

    import fasted_amd

    lib = fasted_amd.load_findpairs()
    bits = datasets.uniform_bytes(2000, 128, seed=9)
    eps = datasets.epsilon_for_neighbours(bits, 10)
    n, d = bits.shape
    pts = torch.from_numpy(bits.view(np.int16).copy()).cuda()
    cap = 100 * n
    pairs = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    lib.releaseResources()
    torch.cuda.synchronize()
    first = fasted_amd.self_join_device_noalloc(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap)  # looks up the array, creates its events
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        st = fasted_amd.self_join_device_noalloc(pts.data_ptr(), n, d, d, eps, pairs.data_ptr(), cap)
        assert st.pairsFound == first.pairsFound > n
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    # the allocating entry on the same input, for contrast and as the reference result
    want = torch.empty((cap, 2), dtype=torch.int32, device="cuda")
    ref = fasted_amd.self_join_device(pts.data_ptr(), n, d, d, eps, want.data_ptr(), cap, flags=1)
    assert ref.pairsFound == first.pairsFound
    assert np.array_equal(_row_major(pairs[: st.pairsStored].cpu().numpy()), want[: ref.pairsStored].cpu().numpy())


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
