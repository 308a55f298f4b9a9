"""Host-side mirror of code_builder / executor over the C ABI."""
import ctypes as C

import numpy as np

from . import _capi as capi

_bound = False


def _bind(L):
    global _bound
    if _bound:
        return
    vp = C.c_void_p
    L.as_builder_create.restype = vp
    L.as_builder_create.argtypes = [vp]
    L.as_builder_free.restype = None
    L.as_builder_free.argtypes = [vp]
    L.as_template_is_supported.argtypes = [vp, C.c_int64, C.c_int]
    L.as_builder_set_template.argtypes = [vp, C.c_int64, C.c_int]
    L.as_builder_compress.argtypes = [vp, C.c_int64]
    L.as_builder_set_launch.argtypes = [vp, C.c_int64, C.c_long, C.c_long, C.c_long, C.c_long]
    L.as_builder_get_launch.argtypes = [vp, C.c_int64, capi.longp]
    L.as_template_get_u64.restype = C.c_int64
    L.as_template_get_u64.argtypes = [vp, C.c_int64, C.c_char_p, capi.u64p, C.c_uint64, capi.intp, capi.intp]
    L.as_template_get_f64.restype = C.c_int64
    L.as_template_get_f64.argtypes = [vp, C.c_int64, capi.f64p, C.c_uint64]
    L.as_template_describe.restype = C.c_char_p
    L.as_template_describe.argtypes = [vp, C.c_int64]
    L.as_builder_kernel_source.restype = C.c_char_p
    L.as_builder_kernel_source.argtypes = [vp]
    L.as_builder_compile.argtypes = [vp]
    L.as_builder_upload.argtypes = [vp, C.c_int]
    L.as_builder_spmv.argtypes = [vp, vp, vp]
    L.as_builder_set_relative_columns.argtypes = [vp, C.c_int64]
    L.as_builder_set_diagonal_columns.argtypes = [vp, C.c_int64]
    L.as_builder_set_column_runs.argtypes = [vp, C.c_int64]
    L.as_builder_set_row_ownership.argtypes = [vp, C.c_int64]
    L.as_builder_set_row_blocks.argtypes = [vp, C.c_int64, C.c_int]
    L.as_builder_set_x.argtypes = [vp, vp]
    L.as_builder_set_serial_launch.argtypes = [vp, C.c_int]
    L.as_builder_set_finish_carry.argtypes = [vp, C.c_int]
    L.as_builder_finish_carrier.argtypes = [vp, C.c_uint64, C.POINTER(C.c_int64)]
    L.as_builder_set_fuse_launches.argtypes = [vp, C.c_int]
    L.as_builder_launch_is_fused.argtypes = [vp, C.c_uint64]
    L.as_builder_time_sub_matrix.argtypes = [vp, C.c_int64, C.c_uint64, C.POINTER(C.c_float), C.POINTER(C.c_uint64),
                                             C.POINTER(C.c_uint64), C.POINTER(C.c_int)]
    L.as_builder_time_sub_matrix_pass.argtypes = [vp, C.c_int64, C.c_int, C.c_uint64, C.POINTER(C.c_float)]
    L.as_builder_time.argtypes = [vp, C.c_uint64, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.as_builder_algorithmic_bytes.restype = C.c_int64
    L.as_builder_algorithmic_bytes.argtypes = [vp]
    L.as_builder_scratch_bytes.restype = C.c_int64
    L.as_builder_scratch_bytes.argtypes = [vp, C.c_int64]
    L.as_hip_device_count.restype = C.c_int
    L.as_builder_spmv_device.argtypes = [vp, vp, vp]
    L.as_builder_spmv_device_no_alloc.argtypes = [vp, vp, vp]
    L.as_builder_spmv_device_async.argtypes = [vp, vp, vp, vp]
    L.as_builder_spmv_device_no_alloc_async.argtypes = [vp, vp, vp, vp]
    L.as_builder_stream.restype = vp
    L.as_builder_stream.argtypes = [vp]
    L.as_hip_stream_create.argtypes = [C.POINTER(vp)]
    L.as_hip_stream_destroy.argtypes = [vp]
    L.as_hip_stream_sync.argtypes = [vp]
    L.as_hip_graph_capture_begin.argtypes = [vp]
    L.as_hip_graph_capture_end.argtypes = [vp, C.POINTER(vp)]
    L.as_hip_graph_launch.argtypes = [vp, vp]
    L.as_hip_graph_destroy.argtypes = [vp]
    L.as_hip_mem_info.argtypes = [capi.u64p, capi.u64p]
    L.as_builder_clears_y.argtypes = [vp]
    L.as_builder_static_scratch_need.restype = C.c_int64
    L.as_builder_static_scratch_need.argtypes = [vp]
    L.as_hip_last_error.restype = C.c_char_p
    L.as_hip_alloc.argtypes = [C.POINTER(vp), C.c_uint64]
    L.as_hip_free.argtypes = [vp]
    L.as_hip_h2d.argtypes = [vp, vp, C.c_uint64]
    L.as_hip_d2h.argtypes = [vp, vp, C.c_uint64]
    _bound = True


def device_facts(read_device=None, cu_num=0, lds_bytes=0, reset=False):
    """What the format builders assume about the GPU, as a dict (cu_num, lds_bytes, xcd_num, l2_bytes_per_xcd,
    from_device).  read_device = a GPU number: ask that GPU first; cu_num / lds_bytes != 0: set them first;
    reset: back to the MI355X values first."""
    L = capi.lib()
    if reset and L.as_device_facts_reset() != 0:
        raise capi.AlphaSparseError(L.as_last_error().decode())
    L.as_device_facts.argtypes = [capi.u64p, capi.u64p, capi.u64p, capi.u64p, capi.intp]
    L.as_device_facts_set.argtypes = [C.c_uint64, C.c_uint64]
    L.as_device_facts_read.argtypes = [C.c_int]
    if read_device is not None and L.as_device_facts_read(int(read_device)) != 0:
        raise capi.AlphaSparseError(L.as_last_error().decode())
    if (cu_num or lds_bytes) and L.as_device_facts_set(int(cu_num), int(lds_bytes)) != 0:
        raise capi.AlphaSparseError(L.as_last_error().decode())
    v = [C.c_uint64(0) for _ in range(4)]
    f = C.c_int(0)
    if L.as_device_facts(*[C.byref(a) for a in v], C.byref(f)) != 0:
        raise capi.AlphaSparseError(L.as_last_error().decode())
    return {"cu_num": v[0].value, "lds_bytes": v[1].value, "xcd_num": v[2].value, "l2_bytes_per_xcd": v[3].value,
            "from_device": bool(f.value)}


class DeviceArray:
    """A caller-owned device buffer (as_hip_alloc) holding a numpy array's bytes: what a user of the C-ABI passes to
    the *_device entry points."""

    def __init__(self, host):
        self._L = capi.lib()
        _bind(self._L)
        host = np.ascontiguousarray(host)
        self.dtype, self.shape, self.nbytes = host.dtype, host.shape, host.nbytes
        self.ptr = C.c_void_p()
        if self._L.as_hip_alloc(C.byref(self.ptr), max(1, self.nbytes)) != 0:
            raise capi.AlphaSparseError(self._L.as_hip_last_error().decode())
        self.set(host)

    def set(self, host):
        host = np.ascontiguousarray(host, dtype=self.dtype)
        assert host.nbytes == self.nbytes
        if self._L.as_hip_h2d(self.ptr, host.ctypes.data_as(C.c_void_p), self.nbytes) != 0:
            raise capi.AlphaSparseError(self._L.as_hip_last_error().decode())

    def get(self):
        out = np.empty(self.shape, self.dtype)
        if self._L.as_hip_d2h(out.ctypes.data_as(C.c_void_p), self.ptr, self.nbytes) != 0:
            raise capi.AlphaSparseError(self._L.as_hip_last_error().decode())
        return out

    def free(self):
        if self.ptr:
            self._L.as_hip_free(self.ptr)
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    """A HIP stream of the caller (default priority), with the capture and replay calls of the thin HIP layer."""

    def __init__(self):
        self._L = capi.lib()
        _bind(self._L)
        self.ptr = C.c_void_p()
        self._hip(self._L.as_hip_stream_create(C.byref(self.ptr)))

    def _hip(self, status):
        if status != 0:
            raise capi.AlphaSparseError(self._L.as_hip_last_error().decode())

    def sync(self):
        self._hip(self._L.as_hip_stream_sync(self.ptr))

    def capture_begin(self):
        self._hip(self._L.as_hip_graph_capture_begin(self.ptr))

    def capture_end(self):
        g = C.c_void_p()
        self._hip(self._L.as_hip_graph_capture_end(self.ptr, C.byref(g)))
        return g

    def graph_launch(self, graph_exec):
        self._hip(self._L.as_hip_graph_launch(graph_exec, self.ptr))

    def graph_destroy(self, graph_exec):
        self._hip(self._L.as_hip_graph_destroy(graph_exec))

    def destroy(self):
        if self.ptr:
            self._L.as_hip_stream_destroy(self.ptr)
            self.ptr = C.c_void_p()


def device_memory_free_bytes():
    L = capi.lib()
    _bind(L)
    f, t = C.c_uint64(0), C.c_uint64(0)
    if L.as_hip_mem_info(C.byref(f), C.byref(t)) != 0:
        raise capi.AlphaSparseError(L.as_hip_last_error().decode())
    return f.value


def kernel_cache_stats():
    """(code objects kept by module source in this process, compilations answered from them)."""
    L = capi.lib()
    L.as_kernel_cache_stats.argtypes = [C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
    e, h = C.c_uint64(0), C.c_uint64(0)
    if L.as_kernel_cache_stats(C.byref(e), C.byref(h)) != 0:
        raise capi.AlphaSparseError(L.as_last_error().decode())
    return e.value, h.value


def device_count():
    L = capi.lib()
    _bind(L)
    return int(L.as_hip_device_count())


def template_is_supported(matrix, sub, template_type):
    L = capi.lib()
    _bind(L)
    return bool(capi.check(L.as_template_is_supported(matrix._h, sub, template_type)))


class Builder:
    """code_builder_t: one kernel template per compressed sub-matrix; compiles, uploads, runs, times."""

    def __init__(self, matrix):
        self._L = capi.lib()
        _bind(self._L)
        self.matrix = matrix  # keep the matrix alive: templates are initialised from it
        self._h = self._L.as_builder_create(matrix._h)
        if not self._h:
            raise capi.AlphaSparseError(self._L.as_last_error().decode())
        info = matrix.info()
        self.rows, self.cols, self.nnz = matrix.y_rows(), info["cols"], info["origin_nnz"]

    def _chk(self, s):
        if s is None or (isinstance(s, int) and s < 0):
            raise capi.AlphaSparseError(self._L.as_last_error().decode())
        return s

    def set_template(self, sub, template_type, compress=True):
        self._chk(self._L.as_builder_set_template(self._h, sub, template_type))
        if compress:
            self._chk(self._L.as_builder_compress(self._h, sub))
        return self

    def set_launch(self, sub, tblock_num=0, thread_num_in_block=0, thread_num_of_row_reduce=0, vec_width=0):
        self._chk(self._L.as_builder_set_launch(self._h, sub, tblock_num, thread_num_in_block,
                                                thread_num_of_row_reduce, vec_width))
        return self

    def set_relative_columns(self, sub):
        """Columns as 16-bit differences to the reading unit's number (ELL template, banded unsorted matrices);
        True when applied (upload again), False when the template or the matrix does not allow it."""
        return bool(self._chk(self._L.as_builder_set_relative_columns(self._h, sub)))

    def set_diagonal_columns(self, sub):
        """Stencils: every element in the slot of its diagonal, columns computed by the kernel, no column array;
        True when applied (upload again), False when the template or the matrix does not allow it."""
        return bool(self._chk(self._L.as_builder_set_diagonal_columns(self._h, sub)))

    def set_column_runs(self, sub):
        """Tile template in its column-run form (first columns of up to four runs of consecutive columns per lane of
        eight elements + a byte of run starts); True when applied (upload again), False when the template is another
        one or the element stream would not get shorter."""
        return bool(self._chk(self._L.as_builder_set_column_runs(self._h, sub)))

    def set_row_ownership(self, sub):
        """Tile template under row ownership (every row group belongs to one workgroup, rows stored to y without
        atomics); True when applied (upload again), False when the template is another one or the form does not
        fit the sub-matrix."""
        return bool(self._chk(self._L.as_builder_set_row_ownership(self._h, sub)))

    def set_row_blocks(self, sub, rows_per_block):
        """Tile template under row ownership: blocks of 2-4 consecutive rows that hold the same columns stored as
        one piece; True when applied (upload again), False when the rows do not come in such blocks."""
        return bool(self._chk(self._L.as_builder_set_row_blocks(self._h, sub, rows_per_block)))

    def get_launch(self, sub):
        out = (C.c_long * 4)()
        self._chk(self._L.as_builder_get_launch(self._h, sub, out))
        return dict(tblock_num=out[0], thread_num_in_block=out[1], thread_num_of_row_reduce=out[2], vec_width=out[3])

    def describe(self, sub):
        s = self._L.as_template_describe(self._h, sub)
        if s is None:
            raise capi.AlphaSparseError(self._L.as_last_error().decode())
        d = {"arrays": {}}
        for line in s.decode().splitlines():
            k, v = line.split("=", 1)
            if k.startswith("array:"):
                dt, n, comp = v.split(",")
                d["arrays"][k[6:]] = (dt, int(n), comp)
            else:
                d[k] = v if k == "template" else int(v)
        return d

    def get_array(self, sub, name):
        if name == "val_arr":
            n = self._chk(self._L.as_template_get_f64(self._h, sub, None, 0))
            out = np.zeros(n, np.float64)
            self._L.as_template_get_f64(self._h, sub, out.ctypes.data_as(capi.f64p), n)
            return out
        dt, ct = C.c_int(0), C.c_int(0)
        n = self._L.as_template_get_u64(self._h, sub, name.encode(), None, 0, C.byref(dt), C.byref(ct))
        if n == -1:
            return None
        self._chk(n)
        out = np.zeros(n, np.uint64)
        self._L.as_template_get_u64(self._h, sub, name.encode(), out.ctypes.data_as(capi.u64p), n, C.byref(dt), C.byref(ct))
        return out, capi.DTYPE_NAMES[dt.value]

    COMPRESS_TYPES = ["NONE_COMPRESS", "LINEAR_COMPRESS", "CONSTANT_COMPRESS", "BRANCH_COMPRESS",
                      "CYCLE_LINEAR_COMPRESS", "CYCLE_INCREASE_COMPRESS"]

    def template_dump(self, sub):
        """Same shape as the upstream harness' template_dump:
        {"scalars": {...}, "arrays": {name: (values, dtype name, compress type ordinal)}, "val_arr": f64}."""
        d = self.describe(sub)
        out = {"scalars": {k: v for k, v in d.items() if k not in ("arrays", "template")}, "arrays": {}}
        for name, (dt, n, comp) in d["arrays"].items():
            if name == "val_arr":
                continue
            vals, dtn = self.get_array(sub, name)
            out["arrays"][name] = (vals, dtn, self.COMPRESS_TYPES.index(comp))
        out["val_arr"] = self.get_array(sub, "val_arr")
        return out

    def kernel_source(self):
        s = self._L.as_builder_kernel_source(self._h)
        if s is None:
            raise capi.AlphaSparseError(self._L.as_last_error().decode())
        return s.decode()

    def compile(self):
        self._chk(self._L.as_builder_compile(self._h))
        return self

    def upload(self, device=0):
        self._chk(self._L.as_builder_upload(self._h, device))
        return self

    def spmv(self, x):
        """y = A x through the generated kernels (x, y host arrays in the matrix value type)."""
        x = np.ascontiguousarray(x)
        if len(x) != self.cols:
            raise ValueError("x has %d entries, matrix has %d columns" % (len(x), self.cols))
        y = np.zeros(self.rows, dtype=x.dtype)
        self._chk(self._L.as_builder_spmv(self._h, x.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.c_void_p)))
        return y

    def spmv_device_async(self, x_dev, y_dev, stream=None, no_alloc=False):
        """Enqueue y = A x on the caller's stream (a Stream, or None for the builder's own stream) and return:
        as_builder_spmv_device_async / as_builder_spmv_device_no_alloc_async on DeviceArray buffers."""
        call = self._L.as_builder_spmv_device_no_alloc_async if no_alloc else self._L.as_builder_spmv_device_async
        s = stream.ptr if stream is not None else self._L.as_builder_stream(self._h)
        self._chk(call(self._h, x_dev.ptr, y_dev.ptr, s))

    def sync(self):
        """Wait for the builder's own stream."""
        if self._L.as_hip_stream_sync(self._L.as_builder_stream(self._h)) != 0:
            raise capi.AlphaSparseError(self._L.as_hip_last_error().decode())

    def spmv_device(self, x, y_before=None, no_alloc=False):
        """y = A x on device buffers of the caller (as_builder_spmv_device, or as_builder_spmv_device_no_alloc): y
        holds `y_before` (a scalar or an array; default NaN) when the call starts, so a row that no kernel writes,
        or a sum added to what was there, shows."""
        L = self._L
        x = np.ascontiguousarray(x)
        if len(x) != self.cols:
            raise ValueError("x has %d entries, matrix has %d columns" % (len(x), self.cols))
        y = np.full(self.rows, np.nan if y_before is None else y_before, dtype=x.dtype)
        dx, dy = C.c_void_p(), C.c_void_p()
        if L.as_hip_alloc(C.byref(dx), x.nbytes) != 0 or L.as_hip_alloc(C.byref(dy), y.nbytes) != 0:
            raise capi.AlphaSparseError(L.as_hip_last_error().decode())
        try:
            if L.as_hip_h2d(dx, x.ctypes.data_as(C.c_void_p), x.nbytes) != 0 or L.as_hip_h2d(dy, y.ctypes.data_as(C.c_void_p), y.nbytes) != 0:
                raise capi.AlphaSparseError(L.as_hip_last_error().decode())
            call = L.as_builder_spmv_device_no_alloc if no_alloc else L.as_builder_spmv_device
            self._chk(call(self._h, dx, dy))
            if L.as_hip_d2h(y.ctypes.data_as(C.c_void_p), dy, y.nbytes) != 0:
                raise capi.AlphaSparseError(L.as_hip_last_error().decode())
        finally:
            L.as_hip_free(dx)
            L.as_hip_free(dy)
        return y

    def clears_y(self):
        """True when an SpMV of the current templates starts with a clear of y."""
        return bool(self._chk(self._L.as_builder_clears_y(self._h)))

    def static_scratch_need(self):
        """Bytes of the library's static scratch array the kernels would use in spmv_device(no_alloc=True)."""
        return int(self._chk(self._L.as_builder_static_scratch_need(self._h)))

    def set_x(self, x):
        x = np.ascontiguousarray(x)
        self._chk(self._L.as_builder_set_x(self._h, x.ctypes.data_as(C.c_void_p)))

    def time_sub_matrix(self, sub, reps):
        """-> (ms for all reps, format bytes, rows of the strip, accumulates y atomically) for one sub-matrix."""
        ms, fb, rows, atom = C.c_float(0), C.c_uint64(0), C.c_uint64(0), C.c_int(0)
        self._chk(self._L.as_builder_time_sub_matrix(self._h, sub, reps, C.byref(ms), C.byref(fb), C.byref(rows), C.byref(atom)))
        return ms.value, int(fb.value), int(rows.value), bool(atom.value)

    def time_sub_matrix_pass(self, sub, which, reps):
        """ms for `reps` launches of one kernel of a two-kernel template (1 = first, 2 = finish), alone."""
        ms = C.c_float(0)
        self._chk(self._L.as_builder_time_sub_matrix_pass(self._h, sub, which, reps, C.byref(ms)))
        return ms.value

    def set_serial_launch(self, serial=True):
        self._chk(self._L.as_builder_set_serial_launch(self._h, int(bool(serial))))
        return self

    def set_fuse_launches(self, on=True):
        """With a carried finish and equal workgroup sizes: the first kernels of the tile strip and of the product-bin
        strip behind it as one launch (default on)."""
        self._chk(self._L.as_builder_set_fuse_launches(self._h, int(bool(on))))
        return self

    def launch_is_fused(self, sub):
        """True when the strip behind `sub` runs the trips of its first kernel (a whole SpMV launches nothing for `sub`)."""
        return bool(self._chk(self._L.as_builder_launch_is_fused(self._h, sub)))

    def set_finish_carry(self, on=True):
        """With serial launch: let the first kernel of a product-bin strip do the work of the finish kernel of the
        tile strip in front of it (default on)."""
        self._chk(self._L.as_builder_set_finish_carry(self._h, int(bool(on))))
        return self

    def finish_carrier(self, sub):
        """The sub-matrix whose first kernel carries the finish of `sub`, or -1."""
        out = C.c_int64(-1)
        self._chk(self._L.as_builder_finish_carrier(self._h, sub, C.byref(out)))
        return out.value

    def time(self, reps, sync_each_launch=False):
        ms, gf = C.c_float(0), C.c_float(0)
        self._chk(self._L.as_builder_time(self._h, reps, int(sync_each_launch), C.byref(ms), C.byref(gf)))
        return ms.value, gf.value

    def algorithmic_bytes(self):
        return int(self._chk(self._L.as_builder_algorithmic_bytes(self._h)))

    def scratch_bytes(self, sub=-1):
        """Bytes of the kernels' scratch arrays (products, row sums) of one sub-matrix, or of all."""
        return int(self._chk(self._L.as_builder_scratch_bytes(self._h, sub)))

    def close(self):
        if self._h:
            self._L.as_builder_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
