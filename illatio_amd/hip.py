"""The device, from Python: the host-side counterpart of the reference's src/cuda.lisp.

src/cuda.lisp binds libcuda through SBCL's alien interface and offers OPEN-CUDA,
CUDA-ALLOC / -FREE / -ZERO, CUDA-UPLOAD(-VECTOR), CUDA-DOWNLOAD, CUDA-FLOATS, CUDA-SYNC,
LAUNCH and the stream / event / pinned-memory calls.  This module offers the same set, with
the same argument meaning and the same error behaviour (every non-zero status raises),
over libillatio_hip.so's C ABI (include/illatio_hip.h).  There is no fallback: without the
built library, importing the kernels fails.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("ILLATIO_HIP_LIB") or os.path.join(_HERE, "libillatio_hip.so")

NOT_READY = 600


class HipError(RuntimeError):
    """A non-zero status from the library (cuda.lisp:41-49 signals a Lisp ERROR)."""

    def __init__(self, what, code, text):
        super().__init__(f"HIP: {what}: {text} ({code})")
        self.code = code


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_int), ("total_memory", C.c_uint64),
                ("max_shared", C.c_int), ("numa_node", C.c_int), ("compute_units", C.c_int), ("wave_size", C.c_int)]


_lib = None


def lib():
    """The loaded library; raises if it has not been built (no CPU stand-in exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `make -C illatio_amd/csrc` "
                              "(or __graft_entry__.build()); there is no CPU fallback")
        _lib = C.CDLL(LIB_PATH)
        _lib.ilt_error_string.restype = C.c_char_p
        _lib.ilt_error_string.argtypes = [C.c_int]
    return _lib


def check(code, what):
    if code != 0:
        raise HipError(what, code, lib().ilt_error_string(code).decode())
    return code


def call(name, *args):
    """Call the library's NAME; raise unless it returns 0."""
    return check(getattr(lib(), name)(*args), name)


class Device:
    """CUDEV (cuda.lisp:61-70): index, name, arch, stream, total-memory, max-shared, numa-node."""

    def __init__(self, index, info, stream):
        self.index = index
        self.name = info.name.decode()
        self.arch = info.arch
        self.total_memory = info.total_memory
        self.max_shared = info.max_shared
        self.numa_node = info.numa_node
        self.compute_units = info.compute_units
        self.wave_size = info.wave_size
        self.stream = stream


_devices = {}


def hip_device_count():
    call("ilt_init")
    n = C.c_int(0)
    call("ilt_device_count", C.byref(n))
    return n.value


def open_hip(index=0):
    """Device INDEX, opened once (OPEN-CUDA, cuda.lisp:94-98)."""
    if index not in _devices:
        call("ilt_init")
        info = DeviceInfo()
        call("ilt_device_get_info", C.c_int(index), C.byref(info))
        call("ilt_set_device", C.c_int(index))
        s = C.c_uint64(0)
        call("ilt_stream_create", C.byref(s), C.c_uint(0))
        _devices[index] = Device(index, info, s.value)
    return _devices[index]


def hip_current(dev):
    call("ilt_set_device", C.c_int(dev.index))


class DBuf:
    """DBUF (cuda.lisp:234): a device address, its size, its device."""
    __slots__ = ("ptr", "bytes", "dev")

    def __init__(self, ptr, nbytes, dev):
        self.ptr, self.bytes, self.dev = ptr, nbytes, dev

    def at(self, offset):
        """(dbuf . offset), as LAUNCH takes it."""
        return (self, offset)


def hip_alloc(dev, nbytes, zero=True):
    hip_current(dev)
    p = C.c_uint64(0)
    call("ilt_malloc", C.byref(p), C.c_uint64(max(int(nbytes), 256)))
    b = DBuf(p.value, int(nbytes), dev)
    if zero:
        hip_zero(b)
    return b


def hip_free(b):
    if b is not None and b.ptr and not isinstance(b, _Slice):
        call("ilt_free", C.c_uint64(b.ptr))
        b.ptr = 0


class _Slice(DBuf):
    """A DBuf carved out of a Workspace: freed with it, not by hip_free."""
    __slots__ = ()


class Workspace:
    """One device allocation handed out in 256-byte-aligned pieces, for a sequence of launches
    that must not allocate or free between them (the reference's hosts keep such buffers in
    their state structs, e.g. DKSTATE, cuda-ds4f.lisp:395-428).  alloc has hip_alloc's
    signature; reset() starts over; pieces are not zeroed."""

    def __init__(self, dev, nbytes):
        self.dev, self.buf, self.used = dev, hip_alloc(dev, nbytes, zero=False), 0

    def alloc(self, dev, nbytes, zero=False):
        n = (max(int(nbytes), 256) + 255) // 256 * 256
        if self.used + n > self.buf.bytes:
            raise MemoryError(f"workspace of {self.buf.bytes} bytes is full")
        b = _Slice(self.buf.ptr + self.used, int(nbytes), dev)
        self.used += n
        return hip_zero(b) if zero else b

    def reset(self):
        self.used = 0

    def free(self):
        hip_free(self.buf)


def hip_zero(b):
    call("ilt_memset_async", C.c_uint64(b.ptr), C.c_int(0), C.c_uint64(b.bytes), C.c_uint64(b.dev.stream))
    return b


def hip_mem_info(dev):
    hip_current(dev)
    f, t = C.c_uint64(0), C.c_uint64(0)
    call("ilt_mem_info", C.byref(f), C.byref(t))
    return f.value, t.value


def hip_sync(dev):
    call("ilt_stream_sync", C.c_uint64(dev.stream))


def hip_upload_vector(b, v, offset=0):
    """The array V's bytes into B at OFFSET; returns when the copy has been made."""
    v = np.ascontiguousarray(v)
    if offset + v.nbytes > b.bytes:
        raise ValueError("upload past the end of the buffer")
    call("ilt_memcpy_htod_async", C.c_uint64(b.ptr + offset), v.ctypes.data_as(C.c_void_p), C.c_uint64(v.nbytes),
         C.c_uint64(b.dev.stream))
    hip_sync(b.dev)
    return b


def hip_upload_new(dev, v):
    v = np.ascontiguousarray(v)
    return hip_upload_vector(hip_alloc(dev, v.nbytes, zero=False), v)


def hip_download(b, dtype, count, offset=0):
    """COUNT elements of DTYPE from B at byte OFFSET, after the work queued before it."""
    out = np.empty(count, dtype=dtype)
    if offset + out.nbytes > b.bytes:
        raise ValueError("download past the end of the buffer")
    call("ilt_memcpy_dtoh_async", out.ctypes.data_as(C.c_void_p), C.c_uint64(b.ptr + offset), C.c_uint64(out.nbytes),
         C.c_uint64(b.dev.stream))
    hip_sync(b.dev)
    return out


def hip_floats(b, n, start=0):
    return hip_download(b, np.float32, n, 4 * start)


def hip_host_alloc(dev, nbytes, mapped=True):
    """NBYTES of pinned host memory (CUDA-HOST-ALLOC, cuda.lisp:359-366); MAPPED: kernels on DEV may read it at the
    same address (an expert's matrices read through from host memory).  Returns the address."""
    hip_current(dev)
    p = C.c_uint64(0)
    call("ilt_host_alloc", C.byref(p), C.c_uint64(nbytes), C.c_uint(1 | (2 if mapped else 0)))
    return p.value


def hip_host_free(addr):
    call("ilt_host_free", C.c_uint64(addr))


def hip_event_create(dev, timing=False):
    hip_current(dev)
    e = C.c_uint64(0)
    call("ilt_event_create", C.byref(e), C.c_uint(0 if timing else 2))
    return e.value


def hip_event_destroy(event):
    call("ilt_event_destroy", C.c_uint64(event))


def hip_event_record(event, stream):
    call("ilt_event_record", C.c_uint64(event), C.c_uint64(stream))


def hip_event_done_p(event):
    r = lib().ilt_event_query(C.c_uint64(event))
    if r == 0:
        return True
    if r == NOT_READY:
        return False
    check(r, "ilt_event_query")


def hip_event_elapsed_ms(start, stop):
    ms = C.c_float(0)
    call("ilt_event_elapsed_ms", C.c_uint64(start), C.c_uint64(stop), C.byref(ms))
    return ms.value


def hip_stream_create(dev):
    hip_current(dev)
    s = C.c_uint64(0)
    call("ilt_stream_create", C.byref(s), C.c_uint(1))
    return s.value


def hip_stream_destroy(stream):
    call("ilt_stream_destroy", C.c_uint64(stream))


def hip_stream_wait(stream, event):
    call("ilt_stream_wait_event", C.c_uint64(stream), C.c_uint64(event))


def hip_stream_sync(stream):
    call("ilt_stream_sync", C.c_uint64(stream))


class beside:
    """with beside(dev): what is queued inside goes to DEV's second stream, which first waits for everything DEV's
    stream holds so far; rejoin(dev) then makes DEV's stream wait for it.  For launches that do not depend on each
    other and do not fill the GPU one by one (a prompt chunk's V product beside its Q and K product).  Both streams
    at the default priority."""

    def __init__(self, dev):
        self.dev = dev

    def __enter__(self):
        dev = self.dev
        if getattr(dev, "second", None) is None:
            dev.second = hip_stream_create(dev)
            dev.forked, dev.joined = hip_event_create(dev), hip_event_create(dev)
        hip_event_record(dev.forked, dev.stream)
        hip_stream_wait(dev.second, dev.forked)
        self.main, dev.stream = dev.stream, dev.second
        return self

    def __exit__(self, *exc):
        dev = self.dev
        dev.stream = self.main
        hip_event_record(dev.joined, dev.second)
        return False


def rejoin(dev):
    hip_stream_wait(dev.stream, dev.joined)


class I64:
    """(:i64 n): a long long argument for LAUNCH."""

    def __init__(self, n):
        self.n = int(n)


def launch(dev, kernel, grid, block, args, shared=0):
    """Queue KERNEL on DEV's stream (LAUNCH, cuda.lisp:323-352).  ARGS in the kernel's order:
    DBufs or (DBuf, byte-offset) for pointers, None for a null pointer, ints for ints, floats
    for floats, I64(n) for a long long -- each written into an 8-byte slot, as the reference
    writes them."""
    n = len(args)
    slots = (C.c_uint64 * max(n, 1))()
    base = C.addressof(slots)
    ptrs = (C.c_void_p * max(n, 1))()
    for i, a in enumerate(args):
        if a is None:
            slots[i] = 0
        elif isinstance(a, DBuf):
            slots[i] = a.ptr
        elif isinstance(a, tuple) and isinstance(a[0], DBuf):
            slots[i] = a[0].ptr + int(a[1])
        elif isinstance(a, I64):
            slots[i] = a.n & 0xFFFFFFFFFFFFFFFF
        elif isinstance(a, (bool, int, np.integer)):
            slots[i] = int(a) & 0xFFFFFFFF
        elif isinstance(a, (float, np.floating)):
            slots[i] = int(np.float32(a).view(np.uint32))
        else:
            raise TypeError(f"launch {kernel}: argument {i} is a {type(a).__name__}")
        ptrs[i] = base + 8 * i

    def dim(x, k):
        xs = list(x) if isinstance(x, (list, tuple)) else [x]
        return int(xs[k]) if k < len(xs) else 1

    check(lib().ilt_launch(kernel.encode(), dim(grid, 0), dim(grid, 1), dim(grid, 2), dim(block, 0), dim(block, 1),
                           dim(block, 2), C.c_uint(shared), C.c_uint64(dev.stream), ptrs), f"launch {kernel}")
