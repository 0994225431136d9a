"""Mirror of the reference's src/hip RAII wrappers over the C ABI:
Device, DeviceBuf, Stream, Event, Graph, Module, Function (src/hip/mod.rs:88-503)."""
import ctypes as C

import numpy as np

from ._lib import check, init, lib


def device_count():
    n = C.c_int(0)
    check(lib.rein_device_count(C.byref(n)))
    return n.value


def set_device(dev=0):
    check(lib.rein_set_device(dev))


def device_name(dev=0):
    buf = C.create_string_buffer(256)
    check(lib.rein_device_name(dev, buf, 256))
    return buf.value.decode()


def mem_info():
    f, t = C.c_size_t(0), C.c_size_t(0)
    check(lib.rein_mem_info(C.byref(f), C.byref(t)))
    return f.value, t.value


def synchronize():
    check(lib.rein_device_synchronize())


class DeviceBuf:
    """Owns one hipMalloc; freed on drop (src/hip/mod.rs:170-186, 322-330)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p(0)
        check(lib.rein_malloc(C.byref(p), max(self.nbytes, 1)))
        self.ptr = p.value

    @classmethod
    def from_host(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.copy_from_host(arr)
        return buf

    def copy_from_host(self, arr, offset=0):
        arr = np.ascontiguousarray(arr)
        assert offset + arr.nbytes <= self.nbytes, "copy_from_host: length mismatch"
        if arr.nbytes:
            check(lib.rein_memcpy_h2d(self.ptr + offset, arr.ctypes.data_as(C.c_void_p), arr.nbytes))

    def to_host(self, dtype, count=None, offset=0):
        dtype = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset) // dtype.itemsize
        out = np.empty(count, dtype)
        assert offset + out.nbytes <= self.nbytes, "to_host: length mismatch"
        if out.nbytes:
            check(lib.rein_memcpy_d2h(out.ctypes.data_as(C.c_void_p), self.ptr + offset, out.nbytes))
        return out

    def free(self):
        if getattr(self, "ptr", None):
            lib.rein_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        p = C.c_void_p(0)
        check(lib.rein_stream_create(C.byref(p)))
        self.raw = p.value

    def synchronize(self):
        check(lib.rein_stream_synchronize(self.raw))

    def begin_capture(self):
        check(lib.rein_stream_begin_capture(self.raw))

    def end_capture(self):
        g = C.c_void_p(0)
        check(lib.rein_stream_end_capture(self.raw, C.byref(g)))
        return Graph(g.value)

    def __del__(self):
        try:
            if self.raw:
                lib.rein_stream_destroy(self.raw)
        except Exception:
            pass


class Event:
    def __init__(self):
        p = C.c_void_p(0)
        check(lib.rein_event_create(C.byref(p)))
        self.raw = p.value

    def record(self, stream=None):
        check(lib.rein_event_record(self.raw, stream.raw if stream else None))

    def synchronize(self):
        check(lib.rein_event_synchronize(self.raw))

    def elapsed_ms(self, later):
        ms = C.c_float(0)
        check(lib.rein_event_elapsed_ms(C.byref(ms), self.raw, later.raw))
        return ms.value

    def __del__(self):
        try:
            if self.raw:
                lib.rein_event_destroy(self.raw)
        except Exception:
            pass


class Graph:
    def __init__(self, raw):
        self.raw = raw

    def instantiate(self):
        ge = C.c_void_p(0)
        check(lib.rein_graph_instantiate(C.byref(ge), self.raw))
        return GraphExec(ge.value)

    def __del__(self):
        try:
            if self.raw:
                lib.rein_graph_destroy(self.raw)
        except Exception:
            pass


class GraphExec:
    def __init__(self, raw):
        self.raw = raw

    def launch(self, stream=None):
        check(lib.rein_graph_launch(self.raw, stream.raw if stream else None))

    def __del__(self):
        try:
            if self.raw:
                lib.rein_graph_exec_destroy(self.raw)
        except Exception:
            pass


class Function:
    """Borrowed kernel handle; launch(grid, block, shared, stream, args) with
    args a list of ctypes values, passed as kernelParams (src/hip/mod.rs:478-502)."""

    def __init__(self, raw, module):
        self.raw, self._module = raw, module

    def launch(self, grid, block, shared_mem, stream, args):
        holders = list(args)
        arr = (C.c_void_p * len(holders))(*[C.cast(C.pointer(a), C.c_void_p) for a in holders])
        check(lib.rein_launch_kernel(self.raw, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                     shared_mem, stream.raw if stream else None, arr))


class Module:
    """A loaded .hsaco; kernels are found by symbol name (src/hip/mod.rs:437-458)."""

    def __init__(self, raw, owned):
        self.raw, self._owned = raw, owned

    @classmethod
    def load(cls, path):
        m = C.c_void_p(0)
        check(lib.rein_module_load(C.byref(m), str(path).encode()))
        return cls(m.value, True)

    @classmethod
    def builtin(cls):
        """The code object librein loaded at init (all reference-named kernels)."""
        init()
        m = C.c_void_p(0)
        check(lib.rein_builtin_module(C.byref(m)))
        return cls(m.value, False)

    def function(self, name):
        f = C.c_void_p(0)
        check(lib.rein_module_get_function(C.byref(f), self.raw, name.encode()))
        return Function(f.value, self)

    def __del__(self):
        try:
            if self._owned and self.raw:
                lib.rein_module_unload(self.raw)
        except Exception:
            pass
