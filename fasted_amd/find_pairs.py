"""ctypes binding of libfasted.so.

Mirrors results/scripts/experiment/find_pairs.py of the reference: ``mmaShape`` and ``Results``
(:24-54), ``compute_selectivity`` (:9-21), ``RerunnablePairsFinder`` (:57-89) and
``load_findpairs`` (:93-127) keep their names, argument meaning and return types, so the
reference's experiment drivers run unchanged on top of this module.  The raw-buffer entry
points of include/fasted.h are bound in addition.
"""
import ctypes
import os
from typing import Callable

FASTED_SORT_PAIRS = 1
FASTED_NO_EPILOGUE = 2
FASTED_SKIP_SUMS = 4
FASTED_SYMMETRIC = 8
FASTED_EVENT_TIMING = 16


def compute_selectivity(result_set_size: int, dataset_size: int) -> float:
    """Selectivity (|R| - |D|) / |D|: mean neighbours per point with self pairs removed."""
    return max(0, result_set_size * 1.0 - dataset_size * 1.0) / dataset_size * 1.0


class mmaShape(ctypes.Structure):
    _fields_ = [("m", ctypes.c_int), ("n", ctypes.c_int), ("k", ctypes.c_int)]

    def __repr__(self):
        return f"mmaShape(m={self.m}, n={self.n}, k={self.k})"


class Results(ctypes.Structure):
    _fields_ = [
        ("totalTime", ctypes.c_double),
        ("TFLOPS", ctypes.c_double),
        ("pairsFound", ctypes.c_ulonglong),
        ("pairsStored", ctypes.c_ulonglong),
        ("inputProblemShape", mmaShape),
        ("paddedProblemShape", mmaShape),
    ]

    def __repr__(self):
        return (f"Results(totalTime={self.totalTime}, TFLOPS={self.TFLOPS}, pairsFound={self.pairsFound}, "
                f"pairsStored={self.pairsStored}, inputProblemShape={self.inputProblemShape}, "
                f"paddedProblemShape={self.paddedProblemShape})")

    def get_selectivity(self) -> float:
        return compute_selectivity(self.pairsFound, self.inputProblemShape.m)


class FastedPair(ctypes.Structure):
    _fields_ = [("QueryPoint", ctypes.c_int), ("CandidatePoint", ctypes.c_int)]


class FastedJoinStats(ctypes.Structure):
    _fields_ = [
        ("sumSquaredMs", ctypes.c_float),
        ("joinMs", ctypes.c_float),
        ("sortMs", ctypes.c_float),
        ("paddedN", ctypes.c_int),
        ("paddedD", ctypes.c_int),
        ("tiles", ctypes.c_ulonglong),
        ("pairsFound", ctypes.c_ulonglong),
        ("pairsStored", ctypes.c_ulonglong),
    ]


class RerunnablePairsFinder:
    """Runs the full routine once, then only re-runs with a new epsilon on the resident dataset."""

    def __init__(self, first_find_pairs: Callable[[float, bool], Results],
                 rerun_find_pairs: Callable[[float, bool], Results]):
        self._first_find_pairs = first_find_pairs
        self._rerun_find_pairs = rerun_find_pairs
        self._first_run = True

    def __call__(self, epsilon: float, save_pairs: bool = False) -> Results:
        if self._first_run:
            self._first_run = False
            return self._first_find_pairs(epsilon, save_pairs)
        return self._rerun_find_pairs(epsilon, save_pairs)


def library_path() -> str:
    return os.environ.get("FASTED_LIBRARY", os.path.join(os.path.dirname(os.path.abspath(__file__)), "libfasted.so"))


_lib = None


def load_findpairs(path: str = None):
    """Loads libfasted.so and declares every entry point of include/fasted.h."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or library_path()
    if not os.path.exists(p):
        raise OSError(f"{p} is missing: build it with `make -C fasted_amd/csrc` (there is no CPU fallback)")
    lib = ctypes.CDLL(p)
    c = ctypes
    lib.runFromExponentialDataset.restype = Results
    lib.runFromExponentialDataset.argtypes = [c.c_int, c.c_int, c.c_double, c.c_double, c.c_double, c.c_bool]
    lib.runFromFile.restype = Results
    lib.runFromFile.argtypes = [c.c_char_p, c.c_double, c.c_bool]
    lib.reRun.restype = Results
    lib.reRun.argtypes = [c.c_double, c.c_bool]
    lib.releaseResources.restype = None
    lib.releaseResources.argtypes = []

    lib.fasted_self_join.restype = c.c_int
    lib.fasted_self_join.argtypes = [c.c_void_p, c.c_longlong, c.c_int, c.c_double, c.c_void_p, c.c_ulonglong,
                                     c.POINTER(c.c_ulonglong), c.POINTER(c.c_ulonglong)]
    lib.fasted_self_join_blocked.restype = c.c_int
    lib.fasted_self_join_blocked.argtypes = [c.c_void_p, c.c_longlong, c.c_int, c.c_double, c.c_longlong, c.c_void_p,
                                             c.c_ulonglong, c.POINTER(c.c_ulonglong), c.POINTER(c.c_ulonglong)]
    lib.fasted_self_join_device.restype = c.c_int
    lib.fasted_self_join_device.argtypes = [c.c_void_p, c.c_longlong, c.c_int, c.c_longlong, c.c_double, c.c_void_p,
                                            c.c_void_p, c.c_ulonglong, c.c_uint, c.c_void_p,
                                            c.POINTER(FastedJoinStats)]
    lib.fasted_self_join_device_noalloc.restype = c.c_int
    lib.fasted_self_join_device_noalloc.argtypes = [c.c_void_p, c.c_longlong, c.c_int, c.c_longlong, c.c_double,
                                                    c.c_void_p, c.c_ulonglong, c.c_uint, c.c_void_p,
                                                    c.POINTER(FastedJoinStats)]
    lib.fasted_join_device.restype = c.c_int
    lib.fasted_join_device.argtypes = [c.c_void_p, c.c_longlong, c.c_longlong, c.c_void_p, c.c_longlong, c.c_longlong,
                                       c.c_int, c.c_double, c.c_void_p, c.c_void_p, c.c_void_p, c.c_ulonglong, c.c_uint,
                                       c.c_void_p, c.POINTER(FastedJoinStats)]
    lib.fasted_pair_distances_device.restype = c.c_int
    lib.fasted_pair_distances_device.argtypes = [c.c_void_p, c.c_longlong, c.c_longlong, c.c_void_p, c.c_longlong,
                                                 c.c_longlong, c.c_int, c.c_void_p, c.c_ulonglong, c.c_void_p,
                                                 c.c_void_p]
    lib.fasted_set_save_distances.restype = None
    lib.fasted_set_save_distances.argtypes = [c.c_int]
    lib.fasted_find_epsilon_volumetric.restype = c.c_int
    lib.fasted_find_epsilon_volumetric.argtypes = [c.c_double, c.c_double, c.POINTER(c.c_double), c.POINTER(c.c_double),
                                                   c.POINTER(c.c_int)]
    lib.fasted_set_download_pairs.restype = None
    lib.fasted_set_download_pairs.argtypes = [c.c_int]
    lib.fasted_last_pairs_device.restype = c.c_void_p
    lib.fasted_last_pairs_device.argtypes = [c.POINTER(c.c_ulonglong)]
    lib.fasted_count_pairs_sampled.restype = c.c_int
    lib.fasted_count_pairs_sampled.argtypes = [c.c_double, c.c_int, c.POINTER(c.c_ulonglong), c.POINTER(c.c_int),
                                               c.POINTER(c.c_double)]
    lib.fasted_find_epsilon_sampled.restype = c.c_int
    lib.fasted_find_epsilon_sampled.argtypes = [c.c_double, c.c_double, c.c_int, c.POINTER(c.c_double),
                                                c.POINTER(c.c_double), c.POINTER(c.c_int)]
    lib.fasted_check_padding_device.restype = c.c_int
    lib.fasted_check_padding_device.argtypes = [c.c_void_p, c.c_longlong, c.c_int, c.c_longlong,
                                                c.POINTER(c.c_ulonglong), c.c_void_p]
    lib.fasted_sum_squared_device.restype = c.c_int
    lib.fasted_sum_squared_device.argtypes = [c.c_void_p, c.c_longlong, c.c_int, c.c_longlong, c.c_void_p, c.c_void_p]
    lib.fasted_raster_coord.restype = c.c_int
    lib.fasted_raster_coord.argtypes = [c.c_ulonglong, c.c_longlong, c.POINTER(c.c_int), c.POINTER(c.c_int)]
    lib.fasted_raster_count.restype = c.c_ulonglong
    lib.fasted_raster_count.argtypes = [c.c_longlong]
    lib.fasted_raster_coord_symmetric.restype = c.c_int
    lib.fasted_raster_coord_symmetric.argtypes = [c.c_ulonglong, c.c_longlong, c.POINTER(c.c_int), c.POINTER(c.c_int)]
    lib.fasted_raster_count_symmetric.restype = c.c_ulonglong
    lib.fasted_raster_count_symmetric.argtypes = [c.c_longlong]
    lib.fasted_load_exponential_dataset.restype = c.c_int
    lib.fasted_load_exponential_dataset.argtypes = [c.c_int, c.c_int, c.c_double, c.c_double]
    lib.fasted_load_file.restype = c.c_int
    lib.fasted_load_file.argtypes = [c.c_char_p]
    lib.fasted_count_pairs.restype = c.c_int
    lib.fasted_count_pairs.argtypes = [c.c_double, c.POINTER(c.c_ulonglong), c.POINTER(c.c_double)]
    lib.fasted_find_epsilon.restype = c.c_int
    lib.fasted_find_epsilon.argtypes = [c.c_double, c.c_double, c.POINTER(c.c_double), c.POINTER(c.c_double),
                                        c.POINTER(c.c_int)]
    lib.fasted_resident_name.restype = c.c_char_p
    lib.fasted_resident_points.restype = c.c_void_p
    lib.fasted_resident_points.argtypes = [c.POINTER(c.c_int)] * 4
    lib.fasted_set_output_dir.restype = None
    lib.fasted_set_output_dir.argtypes = [c.c_char_p]
    lib.fasted_last_error.restype = c.c_char_p
    lib.fasted_version.restype = c.c_char_p
    if path is None:
        _lib = lib
    return lib


class FastedError(RuntimeError):
    pass


def _check(lib, rc):
    if rc != 0:
        raise FastedError(lib.fasted_last_error().decode())


def self_join(points_fp16, epsilon, cap=None):
    """Host entry: (N, D) numpy float16 (or uint16 bit patterns) -> (pairs[k,2] int32 sorted, found)."""
    import numpy as np

    lib = load_findpairs()
    a = np.ascontiguousarray(points_fp16)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    if a.dtype != np.uint16 or a.ndim != 2:
        raise TypeError("points must be a 2-D float16 / uint16 array")
    n, d = a.shape
    cap = int(cap if cap is not None else n * 256)
    out = np.empty((max(cap, 1), 2), dtype=np.int32)
    found, stored = ctypes.c_ulonglong(), ctypes.c_ulonglong()
    _check(lib, lib.fasted_self_join(a.ctypes.data, n, d, float(epsilon), out.ctypes.data, cap,
                                     ctypes.byref(found), ctypes.byref(stored)))
    return out[:stored.value], found.value


def self_join_blocked(points_fp16, epsilon, block_rows, cap=None):
    """self_join for a dataset streamed through the device in blocks of `block_rows` points."""
    import numpy as np

    lib = load_findpairs()
    a = np.ascontiguousarray(points_fp16)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    if a.dtype != np.uint16 or a.ndim != 2:
        raise TypeError("points must be a 2-D float16 / uint16 array")
    n, d = a.shape
    cap = int(cap if cap is not None else n * 256)
    out = np.empty((max(cap, 1), 2), dtype=np.int32)
    found, stored = ctypes.c_ulonglong(), ctypes.c_ulonglong()
    _check(lib, lib.fasted_self_join_blocked(a.ctypes.data, n, d, float(epsilon), int(block_rows), out.ctypes.data, cap,
                                             ctypes.byref(found), ctypes.byref(stored)))
    return out[:stored.value], found.value


def self_join_device(points_ptr, n, d, ld, epsilon, pairs_ptr, cap, sums_ptr=None, flags=FASTED_SORT_PAIRS,
                     stream=None):
    """Device entry on raw pointers (e.g. torch ``tensor.data_ptr()``); returns FastedJoinStats."""
    lib = load_findpairs()
    st = FastedJoinStats()
    _check(lib, lib.fasted_self_join_device(points_ptr, n, d, ld, float(epsilon), sums_ptr, pairs_ptr, cap, flags,
                                            stream, ctypes.byref(st)))
    return st


def self_join_device_noalloc(points_ptr, n, d, ld, epsilon, pairs_ptr, cap, flags=0, stream=None):
    """self_join_device without any device allocation inside the call (pairs unsorted, n <= 4 Mi)."""
    lib = load_findpairs()
    st = FastedJoinStats()
    _check(lib, lib.fasted_self_join_device_noalloc(points_ptr, n, d, ld, float(epsilon), pairs_ptr, cap, flags,
                                                    stream, ctypes.byref(st)))
    return st


def resident_points():
    """Host copy of the resident dataset: (bits[n_pad, d_pad] uint16, n, d, name)."""
    import numpy as np

    lib = load_findpairs()
    n, d, n_pad, d_pad = (ctypes.c_int() for _ in range(4))
    ptr = lib.fasted_resident_points(ctypes.byref(n), ctypes.byref(d), ctypes.byref(n_pad), ctypes.byref(d_pad))
    if not ptr:
        return None
    arr = np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(ctypes.c_uint16)), (n_pad.value, d_pad.value))
    return arr.copy(), n.value, d.value, lib.fasted_resident_name().decode()


def count_pairs(epsilon):
    """Count-only join on the resident dataset: (pairsFound, kernel seconds)."""
    lib = load_findpairs()
    found, secs = ctypes.c_ulonglong(), ctypes.c_double()
    _check(lib, lib.fasted_count_pairs(float(epsilon), ctypes.byref(found), ctypes.byref(secs)))
    return found.value, secs.value


def pair_distances_device(queries_ptr, n_queries, ld_queries, candidates_ptr, n_candidates, ld_candidates, d,
                          pairs_ptr, count, distances_ptr, stream=None):
    """FP32 Euclidean distance of every listed pair, on raw device pointers."""
    lib = load_findpairs()
    _check(lib, lib.fasted_pair_distances_device(queries_ptr, n_queries, ld_queries, candidates_ptr, n_candidates,
                                                 ld_candidates, d, pairs_ptr, count, distances_ptr, stream))


def set_download_pairs(enabled):
    """False: runs that do not save leave their pairs on the device (the reference always downloads them)."""
    load_findpairs().fasted_set_download_pairs(1 if enabled else 0)


def last_pairs_device():
    """(device pointer, count) of the sorted pairs the last runFrom... / reRun stored; owned by the library."""
    stored = ctypes.c_ulonglong()
    ptr = load_findpairs().fasted_last_pairs_device(ctypes.byref(stored))
    return ptr, stored.value


def find_epsilon(target_selectivity, initial_epsilon=0.0):
    """Native bound-then-bisect epsilon search on the resident dataset: (epsilon, selectivity, probes)."""
    lib = load_findpairs()
    eps, sel, probes = ctypes.c_double(), ctypes.c_double(), ctypes.c_int()
    _check(lib, lib.fasted_find_epsilon(float(target_selectivity), float(initial_epsilon), ctypes.byref(eps),
                                        ctypes.byref(sel), ctypes.byref(probes)))
    return eps.value, sel.value, probes.value


def find_epsilon_volumetric(target_selectivity, initial_epsilon=0.1):
    """Native volume-scaling epsilon search on the resident dataset (within 10 % of the target, as the reference's
    find_epsilon_volumetric): (epsilon, selectivity, probes)."""
    lib = load_findpairs()
    eps, sel, probes = ctypes.c_double(), ctypes.c_double(), ctypes.c_int()
    _check(lib, lib.fasted_find_epsilon_volumetric(float(target_selectivity), float(initial_epsilon), ctypes.byref(eps),
                                                   ctypes.byref(sel), ctypes.byref(probes)))
    return eps.value, sel.value, probes.value


def find_epsilon_sampled(target_selectivity, sample_rows=16384, initial_epsilon=0.0):
    """find_epsilon on sampled probes (sample_rows/N of the work each) plus one full count at the end:
    (epsilon, selectivity of the whole dataset, probes)."""
    lib = load_findpairs()
    eps, sel, probes = ctypes.c_double(), ctypes.c_double(), ctypes.c_int()
    _check(lib, lib.fasted_find_epsilon_sampled(float(target_selectivity), float(initial_epsilon), int(sample_rows),
                                                ctypes.byref(eps), ctypes.byref(sel), ctypes.byref(probes)))
    return eps.value, sel.value, probes.value


def join_device(queries_ptr, n_queries, ld_queries, candidates_ptr, n_candidates, ld_candidates, d, epsilon, pairs_ptr,
                cap, flags=FASTED_SORT_PAIRS, stream=None, sums_queries_ptr=None, sums_candidates_ptr=None):
    """Join of two different point sets on raw device pointers; returns FastedJoinStats.  The two optional
    squared-norm buffers are filled by the call, or read by it with FASTED_SKIP_SUMS."""
    lib = load_findpairs()
    st = FastedJoinStats()
    _check(lib, lib.fasted_join_device(queries_ptr, n_queries, ld_queries, candidates_ptr, n_candidates, ld_candidates,
                                       d, float(epsilon), sums_queries_ptr, sums_candidates_ptr, pairs_ptr, cap, flags,
                                       stream, ctypes.byref(st)))
    return st


def check_padding_device(points_ptr, n, d, ld, stream=None):
    """Rows whose padding columns d..roundup(d,64) are not all zeros (must be 0 for the device entries)."""
    lib = load_findpairs()
    bad = ctypes.c_ulonglong()
    _check(lib, lib.fasted_check_padding_device(points_ptr, n, d, ld, ctypes.byref(bad), stream))
    return bad.value


def sum_squared_device(points_ptr, n, d, ld, sums_ptr, stream=None):
    lib = load_findpairs()
    _check(lib, lib.fasted_sum_squared_device(points_ptr, n, d, ld, sums_ptr, stream))
