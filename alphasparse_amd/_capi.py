"""ctypes binding of libalphasparse_amd.so (the C ABI in include/alphasparse_amd.h).

The library must have been built (``__graft_entry__.build()`` or ``make -C
alphasparse_amd/csrc``); there is no fallback path: a missing library is an error.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libalphasparse_amd.so")

u64p = C.POINTER(C.c_uint64)
f64p = C.POINTER(C.c_double)
longp = C.POINTER(C.c_long)
intp = C.POINTER(C.c_int)

# enum as_dtype
(CHAR, UNSIGNED_CHAR, SHORT, UNSIGNED_SHORT, INT, UNSIGNED_INT, LONG, UNSIGNED_LONG, LONG_LONG, UNSIGNED_LONG_LONG,
 FLOAT, DOUBLE, BOOL, NONE_DATA_TYPE) = range(14)
TOP_PADDING, END_PADDING = 0, 1   # global_padding_position (op_manager.hpp:13)
DTYPE_NAMES = ["CHAR", "UNSIGNED_CHAR", "SHORT", "UNSIGNED_SHORT", "INT", "UNSIGNED_INT", "LONG", "UNSIGNED_LONG",
               "LONG_LONG", "UNSIGNED_LONG_LONG", "FLOAT", "DOUBLE", "BOOL", "NONE_DATA_TYPE"]
NP_OF_DTYPE = {CHAR: np.int8, UNSIGNED_CHAR: np.uint8, SHORT: np.int16, UNSIGNED_SHORT: np.uint16, INT: np.int32,
               UNSIGNED_INT: np.uint32, LONG: np.int64, UNSIGNED_LONG: np.uint64, LONG_LONG: np.int64,
               UNSIGNED_LONG_LONG: np.uint64, FLOAT: np.float32, DOUBLE: np.float64, BOOL: np.bool_}

# enum as_node_type
(BEGIN_INPUT_FILE, BEGIN_ARTIFICIAL_INPUT, BEGIN_MEMORY_CACHE_INPUT_FILE, DENSE_ROW_COARSE_SORT, DENSE_FINE_SORT,
 DENSE_TOTAL_ROW_LEVEL_PADDING, DENSE_BLOCK_SORT, DENSE_ROW_DIV, DENSE_FIXED_COL_DIV, COMPRESS, COMPRESSED_ROW_PADDING,
 COMPRESSED_BLOCK_SORT, COMPRESSED_THREAD_LEVEL_ROW_DIV, COMPRESSED_THREAD_LEVEL_COL_DIV, COMPRESSED_WARP_LEVEL_ROW_DIV,
 COMPRESSED_WARP_LEVEL_COL_DIV, COMPRESSED_TBLOCK_LEVEL_ROW_DIV, COMPRESSED_TBLOCK_LEVEL_COL_DIV,
 COMPRESSED_THREAD_LEVEL_NNZ_DIV) = range(19)

# enum as_param_strategy
(COMPRESSED_ROW_PADDING_DIRECT, COMPRESSED_TBLOCK_LEVEL_ROW_DIV_EVENLY, COMPRESSED_TBLOCK_LEVEL_ROW_DIV_ACC_TO_LEAST_NNZ,
 COMPRESSED_TBLOCK_LEVEL_COL_DIV_FIXED, COMPRESSED_WARP_LEVEL_ROW_DIV_EVENLY, COMPRESSED_WARP_LEVEL_COL_DIV_FIXED,
 COMPRESSED_THREAD_LEVEL_ROW_DIV_NONE, COMPRESSED_THREAD_LEVEL_COL_DIV_FIXED, COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT,
 DENSE_ROW_COARSE_SORT_FIXED, DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT, COMPRESS_NONE,
 DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE,
 COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE) = range(15)

# enum as_template_type
(DIRECT_ATOM_TEMPLATE, DIRECT_ATOM_TEMPLATE_WARP_COMPRESS, DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS,
 SHARED_MEMORY_TEMPLATE, SHARED_MEMORY_TEMPLATE_WARP_COMPRESS, SHARED_MEMORY_LONG_ROW_TEMPLATE,
 SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE, DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE,
 UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE, UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE,
 EMPTY_TEMPLATE, NONE_TEMPLATE, SHARED_MEMORY_X_SLICE_TEMPLATE, SHARED_MEMORY_TILE_TEMPLATE,
 SHARED_MEMORY_PRODUCT_BIN_TEMPLATE) = range(15)
TEMPLATE_NAMES = ["DIRECT_ATOM_TEMPLATE", "DIRECT_ATOM_TEMPLATE_WARP_COMPRESS", "DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS",
                  "SHARED_MEMORY_TEMPLATE", "SHARED_MEMORY_TEMPLATE_WARP_COMPRESS", "SHARED_MEMORY_LONG_ROW_TEMPLATE",
                  "SHARED_MEMORY_TOTAL_WARP_REDUCE_TEMPLATE", "DIRECT_ATOM_TOTAL_WARP_REDUCE_TEMPLATE",
                  "UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE",
                  "UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE_WITH_WARP_REDUCE", "EMPTY_TEMPLATE", "NONE_TEMPLATE",
                  "SHARED_MEMORY_X_SLICE_TEMPLATE", "SHARED_MEMORY_TILE_TEMPLATE",
                  "SHARED_MEMORY_PRODUCT_BIN_TEMPLATE"]

F_INDEX_ARR, F_FIRST_ROW, F_ROW_NUMBER, F_COO_BEGIN, F_COO_BLOCK_SIZE, F_SCALARS = range(6)
FIELD_NAMES = ["index_arr", "index_of_the_first_row_arr", "row_number_of_block_arr", "coo_begin_index_arr",
               "coo_block_size_arr", "scalars"]
SLOT_SORTED_ROW_INDEX, SLOT_DENSE_ITEM, SLOT_SHARE_FLAGS, SLOT_COO, SLOT_Y_WRITE_INDEX = 100, 101, 102, 103, 104
V_VAL, V_PADDING_VAL, V_STAGGERED_PADDING_VAL, V_COO_VALUE_CACHE = range(4)

_lib = None


class AlphaSparseError(RuntimeError):
    pass


def bind_matrix_api(lib, prefix, handle_t=C.c_void_p):
    """Declare the (sub, slot, field) introspection + node execution signatures shared by the
    product library (prefix ``as_``) and the upstream dump harness (prefix ``ref_``)."""
    def fn(name, restype, argtypes):
        f = getattr(lib, prefix + name)
        f.restype = restype
        f.argtypes = argtypes
        return f
    fn("execute_node", C.c_int, [handle_t, C.c_int, C.c_int64, longp, C.c_int, u64p, C.c_uint64, u64p, C.c_uint64])
    fn("execute_strategy", C.c_int, [handle_t, C.c_int, C.c_int64, longp])
    fn("complete_blocking", C.c_int, [handle_t, C.c_int64])
    fn("matrix_info", C.c_int, [handle_t, u64p])
    g = "matrix_get_" if prefix == "as_" else "get_"
    fn(g + "u64", C.c_int64, [handle_t, C.c_int64, C.c_int, C.c_int, u64p, C.c_uint64, intp])
    fn(g + "f64", C.c_int64, [handle_t, C.c_int64, C.c_int, f64p, C.c_uint64])


def lib():
    """Load the product library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise AlphaSparseError(
            "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C alphasparse_amd/csrc` (there is no CPU fallback)" % LIB_PATH)
    L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    L.as_last_error.restype = C.c_char_p
    L.as_version.restype = C.c_char_p
    L.as_matrix_from_coo.restype = C.c_void_p
    L.as_matrix_from_coo.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, u64p, u64p, f64p, C.c_int, C.c_int]
    L.as_matrix_from_coo_file.restype = C.c_void_p
    L.as_matrix_from_coo_file.argtypes = [C.c_char_p, C.c_int, C.c_int]
    L.as_matrix_clone.restype = C.c_void_p
    L.as_matrix_clone.argtypes = [C.c_void_p]
    L.as_matrix_free.restype = None
    L.as_matrix_free.argtypes = [C.c_void_p]
    L.as_matrix_check_sorted.argtypes = [C.c_void_p]
    L.as_matrix_has_empty_row.argtypes = [C.c_void_p]
    L.as_matrix_set_option.argtypes = [C.c_void_p, C.c_char_p, C.c_long]
    L.as_matrix_write_coo_file.argtypes = [C.c_void_p, C.c_char_p]
    L.as_matrix_write_binary_file.argtypes = [C.c_void_p, C.c_char_p]
    L.as_matrix_remove_empty_rows.argtypes = [C.c_void_p]
    L.as_matrix_long_short_row_decomposition.restype = C.c_int64
    L.as_matrix_long_short_row_decomposition.argtypes = [C.c_void_p, u64p, C.c_uint64, C.POINTER(C.c_void_p), C.c_uint64]
    L.as_matrix_total_row_level_padding.argtypes = [C.c_void_p, C.c_uint64, C.c_int, C.c_uint64]
    L.as_matrix_total_row_level_padding_direct.argtypes = [C.c_void_p, C.c_uint64, C.c_uint, C.c_int, C.c_uint64]
    L.as_matrix_total_row_level_padding_add.argtypes = [C.c_void_p, C.c_uint64, C.c_uint, C.c_int, C.c_uint64]
    L.as_matrix_dense_col_level_padding.argtypes = [C.c_void_p, u64p, u64p, C.c_uint64]
    L.as_matrix_y_rows.restype = C.c_int64
    L.as_matrix_y_rows.argtypes = [C.c_void_p]
    L.as_matrix_from_mtx_file.restype = C.c_void_p
    L.as_matrix_from_mtx_file.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int]
    L.as_matrix_from_binary_file.restype = C.c_void_p
    L.as_matrix_from_binary_file.argtypes = [C.c_char_p, C.c_int]
    bind_matrix_api(L, "as_")
    _lib = L
    return L


def check(status, L=None):
    if status is None or (isinstance(status, int) and status < 0):
        raise AlphaSparseError((L or lib()).as_last_error().decode())
    return status


def as_u64(a):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    return a, a.ctypes.data_as(u64p)


def as_f64(a):
    a = np.ascontiguousarray(a, dtype=np.float64)
    return a, a.ctypes.data_as(f64p)


class MatrixAPI:
    """Node execution + introspection shared by Matrix (product) and RefMatrix (upstream harness)."""
    _prefix = "as_"
    _L = None
    _h = None

    def _f(self, name):
        if self._prefix != "as_" and name.startswith("matrix_get_"):
            name = name[len("matrix_"):]
        return getattr(self._L, self._prefix + name)

    def _chk(self, status):
        if status < 0:
            msg = self._L.as_last_error().decode() if self._prefix == "as_" else "upstream harness call failed"
            raise AlphaSparseError(msg)
        return status

    def execute_node(self, node_type, sub=-1, scalars=(), lst=(), nested=None):
        if nested is not None:
            counts = np.array([len(x) for x in nested], dtype=np.uint64)
            lst = np.concatenate([np.asarray(x, dtype=np.uint64) for x in nested]) if len(nested) else np.zeros(0, np.uint64)
        else:
            counts = np.zeros(0, np.uint64)
        sc = (C.c_long * max(1, len(scalars)))(*scalars)
        l, lp = as_u64(lst)
        c, cp = as_u64(counts)
        self._chk(self._f("execute_node")(self._h, node_type, sub, sc, len(scalars), lp, len(l), cp, len(c)))
        return self

    def execute_strategy(self, strategy, sub=-1, p=()):
        p = list(p) + [0] * (4 - len(p))
        self._chk(self._f("execute_strategy")(self._h, strategy, sub, (C.c_long * 4)(*p)))
        return self

    def complete_blocking(self, sub):
        self._chk(self._f("complete_blocking")(self._h, sub))
        return self

    def info(self):
        out = (C.c_uint64 * 8)()
        self._chk(self._f("matrix_info")(self._h, out))
        keys = ["rows", "cols", "nnz", "origin_nnz", "n_sub", "is_sorted", "is_compressed", "wave"]
        return dict(zip(keys, [int(x) for x in out]))

    def get_u64(self, sub, slot, field):
        """-> (values as uint64 ndarray, dtype ordinal) or None when the array is absent."""
        dt = C.c_int(NONE_DATA_TYPE)
        n = self._f("matrix_get_u64")(self._h, sub, slot, field, None, 0, C.byref(dt))
        if n == -1:
            return None
        self._chk(n)
        out = np.zeros(n, dtype=np.uint64)
        self._f("matrix_get_u64")(self._h, sub, slot, field, out.ctypes.data_as(u64p), n, C.byref(dt))
        return out, dt.value

    def get_f64(self, sub, which):
        n = self._f("matrix_get_f64")(self._h, sub, which, None, 0)
        if n == -1:
            return None
        self._chk(n)
        out = np.zeros(n, dtype=np.float64)
        self._f("matrix_get_f64")(self._h, sub, which, out.ctypes.data_as(f64p), n)
        return out

    def dump(self):
        """Every array of the constructed format, keyed by a readable name.
        Integer arrays map to (values, dtype name); value arrays to float64 ndarrays."""
        d = {}
        info = self.info()
        d["info"] = {k: info[k] for k in ("rows", "cols", "nnz", "origin_nnz", "n_sub", "is_sorted", "is_compressed")}
        s = self.get_u64(-1, SLOT_SORTED_ROW_INDEX, 0)
        if s is not None:
            d["sorted_row_index"] = (s[0], DTYPE_NAMES[s[1]])
        d["coo_row_index_cache"] = self.get_u64(-1, SLOT_COO, 0)[0]
        d["coo_col_index_cache"] = self.get_u64(-1, SLOT_COO, 1)[0]
        d["coo_value_cache"] = self.get_f64(-1, V_COO_VALUE_CACHE)
        for sub in range(info["n_sub"]):
            pre = "sub%d." % sub
            d[pre + "dense_item"] = self.get_u64(sub, SLOT_DENSE_ITEM, 0)[0]
            if not info["is_compressed"]:
                continue
            d[pre + "share_flags"] = self.get_u64(sub, SLOT_SHARE_FLAGS, 0)[0]
            yw = self.get_u64(sub, SLOT_Y_WRITE_INDEX, 0)
            if yw is not None:
                d[pre + "y_write_index"] = (yw[0], DTYPE_NAMES[yw[1]])
            for slot in range(7):
                sc = self.get_u64(sub, slot, F_SCALARS)
                if sc is None:
                    break
                d[pre + "read_index[%d].scalars" % slot] = sc[0]
                for field in range(F_SCALARS):
                    a = self.get_u64(sub, slot, field)
                    if a is not None:
                        d[pre + "read_index[%d].%s" % (slot, FIELD_NAMES[field])] = (a[0], DTYPE_NAMES[a[1]])
            for which, name in ((V_VAL, "val_arr"), (V_PADDING_VAL, "padding_val_arr"),
                                (V_STAGGERED_PADDING_VAL, "staggered_padding_val_arr")):
                v = self.get_f64(sub, which)
                if v is not None:
                    d[pre + name] = v
        return d
