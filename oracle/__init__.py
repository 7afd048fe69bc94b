"""ctypes bindings of the CPU checker (oracle/fasted_oracle.c) and of the reference's own
host data loader built in oracle/_ref.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline
leg of bench.py.  The shipped package (fasted_amd) never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libfasted_ref.so")

_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference checkout exists)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    lib.oracle_f32_to_f16.restype = C.c_uint16
    lib.oracle_f32_to_f16.argtypes = [C.c_float]
    lib.oracle_f16_to_f32.restype = C.c_float
    lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
    lib.oracle_quantize.argtypes = [_f64p, C.c_size_t, _u16p]
    lib.oracle_widen.argtypes = [_u16p, C.c_size_t, _f64p]
    lib.oracle_exponential_points.argtypes = [C.c_int, C.c_int, C.c_double, C.c_double, _f64p]
    lib.oracle_build_padded.argtypes = [_f64p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                        C.POINTER(C.c_int), C.POINTER(C.c_int)]
    for name in ("oracle_sum_squared_rz", "oracle_sum_squared_rn"):
        getattr(lib, name).argtypes = [_u16p, C.c_size_t, C.c_size_t, _f32p]
    lib.oracle_sum_squared_f64.argtypes = [_u16p, C.c_size_t, C.c_size_t, _f64p]
    lib.oracle_raster_coord.restype = C.c_int
    lib.oracle_raster_coord.argtypes = [C.c_ulonglong, C.c_ulonglong, C.c_ulonglong, C.c_uint, C.c_int, C.c_int,
                                        C.POINTER(C.c_int), C.POINTER(C.c_int)]
    lib.oracle_pairs_get_space.restype = C.c_longlong
    lib.oracle_pairs_get_space.argtypes = [C.POINTER(C.c_ulonglong), C.POINTER(C.c_ulonglong), C.c_ulonglong, C.c_uint]
    lib.oracle_self_join_f64.restype = C.c_ulonglong
    lib.oracle_self_join_f64.argtypes = [_u16p, C.c_size_t, C.c_size_t, C.c_double, _i32p, _i32p, C.c_ulonglong]
    lib.oracle_self_join_f64_rows.restype = C.c_ulonglong
    lib.oracle_self_join_f64_rows.argtypes = [_u16p, C.c_size_t, C.c_size_t, C.c_double, C.c_size_t, C.c_size_t,
                                              _i32p, _i32p, C.c_ulonglong]
    lib.oracle_self_join_f32.restype = C.c_ulonglong
    lib.oracle_self_join_f32.argtypes = [_u16p, C.c_size_t, C.c_size_t, C.c_double, _f32p, _i32p, _i32p, C.c_ulonglong]
    lib.oracle_pair_distances_f64.argtypes = [_u16p, C.c_size_t, _i32p, _i32p, C.c_size_t, _f64p]
    lib.oracle_pair_stats.argtypes = [_i32p, _i32p, C.c_size_t, _i32p, _i32p, C.c_size_t,
                                      C.POINTER(C.c_ulonglong * 5), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    lib.oracle_num_threads.restype = C.c_int
    lib.oracle_blocked_join.restype = C.c_ulonglong
    lib.oracle_blocked_join.argtypes = [_u16p, C.c_size_t, C.c_size_t, _u16p, C.c_size_t, C.c_size_t, C.c_size_t,
                                        C.c_double, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_ulonglong,
                                        C.POINTER(C.c_double)]
    lib.oracle_blocked_join_vector_bits.restype = C.c_int
    lib.oracle_blocked_join_vector_bits.argtypes = [C.c_int]
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


# ----------------------------------------------------------------------------- wrappers
def quantize(values):
    """double -> float -> half (RNE); returns uint16 bit patterns of the same shape."""
    v = np.ascontiguousarray(values, dtype=np.float64)
    out = np.empty(v.shape, dtype=np.uint16)
    lib().oracle_quantize(v.reshape(-1), v.size, out.reshape(-1))
    return out


def exponential_points(n, d, lam=40.0, max_value=10.0):
    out = np.empty((n, d), dtype=np.float64)
    lib().oracle_exponential_points(n, d, lam, max_value, out.reshape(-1))
    return out


def build_padded(values, dim_factor, points_factor):
    v = np.ascontiguousarray(values, dtype=np.float64)
    n, d = v.shape
    np_, dp_ = C.c_int(), C.c_int()
    lib().oracle_build_padded(v.reshape(-1), n, d, dim_factor, points_factor, None, C.byref(np_), C.byref(dp_))
    out = np.empty((np_.value, dp_.value), dtype=np.uint16)
    lib().oracle_build_padded(v.reshape(-1), n, d, dim_factor, points_factor, out.ctypes.data, C.byref(np_), C.byref(dp_))
    return out


def sum_squared(bits, mode="rz"):
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    n, d = b.shape
    if mode == "f64":
        out = np.empty(n, dtype=np.float64)
        lib().oracle_sum_squared_f64(b.reshape(-1), n, d, out)
        return out
    out = np.empty(n, dtype=np.float32)
    getattr(lib(), "oracle_sum_squared_" + mode)(b.reshape(-1), n, d, out)
    return out


def raster_coord(idx, chunk_rows, chunk_cols, raster_size, tile_m, tile_n):
    r, c = C.c_int(), C.c_int()
    ok = lib().oracle_raster_coord(idx, chunk_rows, chunk_cols, raster_size, tile_m, tile_n, C.byref(r), C.byref(c))
    return (r.value, c.value) if ok else None


def _grow_join(call, guess):
    cap = max(int(guess), 1024)
    while True:
        q = np.empty(cap, dtype=np.int32)
        c = np.empty(cap, dtype=np.int32)
        found = call(q, c, cap)
        if found <= cap:
            return np.stack([q[:found], c[:found]], axis=1)
        cap = int(found)


def self_join_f64(bits, eps, n=None, rows=None):
    """FP64 ground-truth join over the first n rows (default all).  rows=(q0,q1) limits queries."""
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    n = b.shape[0] if n is None else n
    d = b.shape[1]
    flat = b.reshape(-1)
    if rows is None:
        return _grow_join(lambda q, c, cap: lib().oracle_self_join_f64(flat, n, d, eps, q, c, cap), 64 * n)
    q0, q1 = rows
    return _grow_join(lambda q, c, cap: lib().oracle_self_join_f64_rows(flat, n, d, eps, q0, q1, q, c, cap),
                      64 * (q1 - q0))


def self_join_f32(bits, eps, n=None, sums=None):
    """The reference's FP16-in / FP32-accumulate arithmetic model (RZ squared norms by default)."""
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    n = b.shape[0] if n is None else n
    d = b.shape[1]
    if sums is None:
        sums = sum_squared(b, "rz")
    sums = np.ascontiguousarray(sums, dtype=np.float32)
    flat = b.reshape(-1)
    return _grow_join(lambda q, c, cap: lib().oracle_self_join_f32(flat, n, d, eps, sums, q, c, cap), 64 * n)


def blocked_join(queries, candidates, eps, precision=64, q_offset=0, c_offset=0, want_pairs=True):
    """The CPU baseline (oracle/blocked_join.c): cache-blocked GEMM-form join of query rows with candidate rows,
    in FP64 or FP32.  Returns (pairs sorted row-major or None, found, seconds inside the routine)."""
    q = np.ascontiguousarray(queries, dtype=np.uint16)
    c = np.ascontiguousarray(candidates, dtype=np.uint16)
    assert q.ndim == 2 and c.ndim == 2 and q.shape[1] == c.shape[1]
    d = q.shape[1]
    secs = C.c_double()
    call = lambda oq, oc, cap: lib().oracle_blocked_join(  # noqa: E731
        q.reshape(-1), q.shape[0], d, c.reshape(-1), c.shape[0], d, d, float(eps), int(precision), int(q_offset),
        int(c_offset), oq, oc, cap, C.byref(secs))
    if not want_pairs:
        found = call(None, None, 0)
        return None, int(found), secs.value
    cap = max(1024, 64 * q.shape[0])
    while True:
        oq = np.empty(cap, dtype=np.int32)
        oc = np.empty(cap, dtype=np.int32)
        found = int(call(oq.ctypes.data, oc.ctypes.data, cap))
        if found <= cap:
            return sort_pairs(np.stack([oq[:found], oc[:found]], axis=1)), found, secs.value
        cap = found


def blocked_join_vector_bits(force=0):
    """Vector width (256 or 512 bits) the CPU baseline runs with on this host; `force` selects one."""
    return lib().oracle_blocked_join_vector_bits(int(force))


def pair_distances_f64(bits, pairs):
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    p = np.asarray(pairs).reshape(-1, 2)
    q = np.ascontiguousarray(p[:, 0], dtype=np.int32)
    c = np.ascontiguousarray(p[:, 1], dtype=np.int32)
    out = np.empty(len(q), dtype=np.float64)
    if len(q):
        lib().oracle_pair_distances_f64(b.reshape(-1), b.shape[1], q, c, len(q), out)
    return out


def pair_stats(left, right, want_diff=False):
    """Merge-walk diff of two row-major sorted (k,2) pair arrays.

    Returns dict(both, right_only, left_only, left_total, right_total) and, with want_diff,
    the one-sided pairs as (pairs[k,2], side[k]) where side 0 = left only, 1 = right only."""
    l = np.asarray(left).reshape(-1, 2)
    r = np.asarray(right).reshape(-1, 2)
    lq, lc = (np.ascontiguousarray(l[:, i], dtype=np.int32) for i in (0, 1))
    rq, rc = (np.ascontiguousarray(r[:, i], dtype=np.int32) for i in (0, 1))
    stats = (C.c_ulonglong * 5)()
    cap = len(l) + len(r) if want_diff else 0
    oq = np.empty(cap, dtype=np.int32)
    oc = np.empty(cap, dtype=np.int32)
    os_ = np.empty(cap, dtype=np.int32)
    lib().oracle_pair_stats(lq, lc, len(lq), rq, rc, len(rq), C.byref(stats),
                            oq.ctypes.data if want_diff else None, oc.ctypes.data if want_diff else None,
                            os_.ctypes.data if want_diff else None, cap)
    out = dict(both=stats[0], right_only=stats[1], left_only=stats[2], left_total=stats[3], right_total=stats[4])
    if want_diff:
        k = out["right_only"] + out["left_only"]
        return out, np.stack([oq[:k], oc[:k]], axis=1), os_[:k]
    return out


def epsilon_band_report(bits, got_pairs, eps, truth_pairs=None, n=None, band=1e-3):
    """Pair-set parity verdict against FP64.

    Disagreements between `got_pairs` and the FP64 join are allowed only for pairs whose FP64
    distance lies within a relative `band` of eps.  Returns dict with the counts, the number of
    disagreeing pairs outside the band (must be 0) and the max relative distance error
    |d - eps| / eps over the disagreeing pairs."""
    got = sort_pairs(got_pairs)
    truth = self_join_f64(bits, eps, n=n) if truth_pairs is None else truth_pairs
    stats, diff, side = pair_stats(got, truth, want_diff=True)
    dist = pair_distances_f64(bits, diff)
    rel = np.abs(dist - eps) / eps if len(dist) else np.zeros(0)
    return dict(both=int(stats["both"]), got_only=int(stats["left_only"]), truth_only=int(stats["right_only"]),
                band_pairs=int(len(rel)), outside_band=int((rel > band).sum()),
                max_rel_err=float(rel.max()) if len(rel) else 0.0, truth_total=int(stats["right_total"]))


def sort_pairs(pairs):
    p = np.asarray(pairs, dtype=np.int32).reshape(-1, 2)
    key = (p[:, 0].astype(np.int64) << 32) | p[:, 1].astype(np.int64)
    return p[np.argsort(key, kind="stable")]


def num_threads():
    return lib().oracle_num_threads()


# ------------------------------------------------------------- reference's own data loader
def ref_available():
    return os.path.exists(_REF_PATH)


_ref = None


def ref():
    """The reference's DataLoader headers compiled in place (oracle/_ref); None if not built."""
    global _ref
    if _ref is None and ref_available():
        r = C.CDLL(_REF_PATH)
        r.ref_cast_value.restype = C.c_uint16
        r.ref_cast_value.argtypes = [C.c_double]
        r.ref_build_exponential.argtypes = [C.c_int, C.c_int, C.c_double, C.c_double, C.c_int, C.c_int]
        r.ref_build_file.argtypes = [C.c_char_p, C.c_int, C.c_int]
        r.ref_last_error.restype = C.c_char_p
        r.ref_dataset_name.restype = C.c_char_p
        r.ref_copy_values.argtypes = [_u16p]
        _ref = r
    return _ref


def ref_values():
    r = ref()
    out = np.empty((r.ref_num_points(), r.ref_dimensions()), dtype=np.uint16)
    r.ref_copy_values(out.reshape(-1))
    return out
