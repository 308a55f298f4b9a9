"""Host-side mirror of the search driver (main.cc:561-664) over the C ABI."""
import ctypes as C

from . import _capi as capi
from .builder import Builder, _bind


class SearchOptions(C.Structure):
    _fields_ = [("total_time_s", C.c_double), ("struggle_step_num", C.c_uint64), ("padding_rate_up_bound", C.c_double),
                ("device", C.c_int), ("timed_region_ms", C.c_double), ("checkpoint_dir", C.c_char_p), ("verbose", C.c_int),
                ("only_dense_strategy", C.c_int), ("remove_empty_rows", C.c_int),
                ("general_templates", C.c_int), ("skip_verification", C.c_int)]


def _bind_search(L):
    if getattr(L, "_search_bound", False):
        return
    vp = C.c_void_p
    L.as_find_best_graph.restype = vp
    L.as_find_best_graph.argtypes = [vp, C.POINTER(SearchOptions)]
    L.as_search_free.restype = None
    L.as_search_free.argtypes = [vp]
    L.as_search_report.restype = C.c_char_p
    L.as_search_report.argtypes = [vp]
    L.as_search_log.restype = C.c_char_p
    L.as_search_log.argtypes = [vp]
    L.as_search_stats.argtypes = [vp, C.POINTER(C.c_double)]
    L.as_search_best_graph.restype = C.c_int64
    L.as_search_best_graph.argtypes = [vp, capi.longp, C.c_uint64]
    L.as_search_build_best.restype = vp
    L.as_search_build_best.argtypes = [vp, vp]
    L.as_part_execute_code_builder.argtypes = [vp, C.POINTER(C.c_int64), C.c_uint64, C.c_uint64, C.POINTER(C.c_float),
                                               C.POINTER(C.c_float)]
    L.as_execute_code_builder.argtypes = [vp, C.c_double, C.POINTER(C.c_uint64), C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L._search_bound = True


class SearchResult:
    def __init__(self, handle, matrix):
        self._L = capi.lib()
        self._h = handle
        self.matrix = matrix
        out = (C.c_double * 8)()
        capi.check(self._L.as_search_stats(handle, out))
        (self.gflops, self.time_ms, self.candidates, self.failed_candidates, self.seconds, self.seconds_to_best,
         self.n_sub, self.dense_strategy) = [float(x) for x in out]
        self.report = self._L.as_search_report(handle).decode()
        self.log = self._L.as_search_log(handle).decode()

    def best_graph(self):
        """The best graph as the flat list of numbers that as_graph_report takes."""
        n = capi.check(self._L.as_search_best_graph(self._h, None, 0))
        d = (C.c_long * n)()
        capi.check(self._L.as_search_best_graph(self._h, d, n))
        return list(d)

    def build_best(self):
        """Rebuild the best format from the input matrix -> Builder (not yet uploaded)."""
        h = self._L.as_search_build_best(self._h, self.matrix._h)
        if not h:
            raise capi.AlphaSparseError(self._L.as_last_error().decode())
        b = Builder.__new__(Builder)
        b._L, b._h, b.matrix = self._L, h, self.matrix
        info = self.matrix.info()
        b.rows, b.cols, b.nnz = info["rows"], info["cols"], info["origin_nnz"]
        return b

    def close(self):
        if self._h:
            self._L.as_search_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def find_best_graph(matrix, total_time_s=60.0, struggle_step_num=10, device=0, timed_region_ms=20.0, checkpoint_dir=None,
                    verbose=False, only_dense_strategy=0, padding_rate_up_bound=4.0, remove_empty_rows=False,
                    general_templates=False, skip_verification=False):
    """find_best_graph_of_white_list_strategy on a freshly read matrix (no operator applied yet)."""
    L = capi.lib()
    _bind(L)
    _bind_search(L)
    o = SearchOptions(total_time_s, struggle_step_num, padding_rate_up_bound, device, timed_region_ms,
                      checkpoint_dir.encode() if checkpoint_dir else None, int(verbose), only_dense_strategy,
                      int(bool(remove_empty_rows)), int(bool(general_templates)), int(bool(skip_verification)))
    h = L.as_find_best_graph(matrix._h, C.byref(o))
    if not h:
        raise capi.AlphaSparseError(L.as_last_error().decode())
    return SearchResult(h, matrix)


def part_execute_code_builder(builder, sub_matrix_ids, repeat):
    """executor.hpp:12 -> (ok, time_ms, gflops); failures return (False, 0, 0) as upstream returns false."""
    L = capi.lib()
    _bind_search(L)
    ids = (C.c_int64 * max(1, len(sub_matrix_ids)))(*sub_matrix_ids)
    ms, gf = C.c_float(0), C.c_float(0)
    r = L.as_part_execute_code_builder(builder._h, ids, len(sub_matrix_ids), repeat, C.byref(ms), C.byref(gf))
    return (r == 0, ms.value, gf.value)


def execute_code_builder(builder, seconds=8.0):
    """executor.hpp:19: final run of about `seconds` -> (repeat, time_ms, gflops)."""
    L = capi.lib()
    _bind_search(L)
    rep, ms, gf = C.c_uint64(0), C.c_float(0), C.c_float(0)
    capi.check(L.as_execute_code_builder(builder._h, seconds, C.byref(rep), C.byref(ms), C.byref(gf)))
    return rep.value, ms.value, gf.value
