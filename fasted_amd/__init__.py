"""fasted_amd -- MI355X (gfx950) epsilon self-join behind the FaSTED C ABI.

The product is ``libfasted.so`` (sources in ``fasted_amd/csrc``, ABI in ``include/fasted.h``).
This package is the thin host-side mirror of the reference's Python FFI wrapper
(results/scripts/experiment/find_pairs.py) plus ctypes access to the raw-buffer entry points.
There is no CPU fallback: loading fails loudly when the HIP library has not been built.
"""
from .find_pairs import (  # noqa: F401
    FastedJoinStats,
    FastedPair,
    check_padding_device,
    RerunnablePairsFinder,
    Results,
    compute_selectivity,
    count_pairs,
    find_epsilon,
    find_epsilon_sampled,
    last_pairs_device,
    set_download_pairs,
    find_epsilon_volumetric,
    join_device,
    library_path,
    load_findpairs,
    mmaShape,
    pair_distances_device,
    resident_points,
    self_join,
    self_join_blocked,
    self_join_device,
    self_join_device_noalloc,
    sum_squared_device,
)

__all__ = [
    "FastedJoinStats", "FastedPair", "check_padding_device", "RerunnablePairsFinder", "Results", "compute_selectivity", "count_pairs", "find_epsilon", "find_epsilon_sampled", "last_pairs_device", "set_download_pairs", "find_epsilon_volumetric", "join_device", "library_path",
    "load_findpairs", "mmaShape", "pair_distances_device", "resident_points", "self_join", "self_join_blocked", "self_join_device", "self_join_device_noalloc", "sum_squared_device",
]
