"""Device memory and the execution stream.

Two providers, chosen once per process (``dpnp_amd._lib.MEMORY``):

* ``native`` (the default): the library's own pool and stream (``dpx_mem_alloc`` /
  ``dpx_mem_free`` / ``dpx_stream_create``).
* ``torch`` (DPNP_AMD_MEMORY=torch): PyTorch as plumbing.  Its caching allocator hands out
  device memory (a uint8 CUDA tensor per allocation) and its current stream is the hipStream_t
  every kernel of the library is enqueued on, so this library's work interleaves correctly
  with torch work of the same process.

Both allocators are stream-ordered: a temporary released right after a launch is not
reused before that launch has run.
"""
import ctypes

import numpy as np

from .. import _lib


def _torch():
    if _lib.torch is None:
        raise RuntimeError("this process runs dpnp_amd on its own allocator: PyTorch is not loaded")
    return _lib.torch


_NATIVE = _lib.MEMORY == "native"
_native_stream = None


def _native_stream_ptr():
    """The library stream of this process (created at first use)."""
    global _native_stream
    if _native_stream is None:
        s = ctypes.c_void_p()
        _lib.check(_lib.lib.dpx_stream_create(ctypes.byref(s)))
        _native_stream = s.value or 0
    return _native_stream


class NativeBuffer:
    """A block of dpx_mem_alloc; returned to the pool, in stream order, when the last reference goes.

    Quacks like the uint8 tensor of the torch provider where this package uses one:
    ``data_ptr()`` and ``numel()``.
    """

    __slots__ = ("_base", "_ptr", "_nbytes", "__weakref__")

    def __init__(self, nbytes, skew=0):
        p = ctypes.c_void_p()
        _lib.check(_lib.lib.dpx_mem_alloc(ctypes.byref(p), nbytes + skew, _native_stream_ptr()))
        self._base = p.value
        self._ptr = p.value + skew
        self._nbytes = nbytes

    def data_ptr(self):
        return self._ptr

    def numel(self):
        return self._nbytes

    def __del__(self):
        base, self._base = getattr(self, "_base", None), None
        if base:
            try:
                _lib.lib.dpx_mem_free(base, _native_stream)
            except Exception:  # interpreter shutdown: the process ends, the driver reclaims the memory
                pass


class ExecutionPlacementError(Exception):
    """Raised when arrays of one call live on different devices."""


class Device:
    """Stand-in for dpctl.SyclDevice: the one GPU this process uses."""

    has_aspect_fp16 = True
    has_aspect_fp64 = True
    has_aspect_gpu = True

    def __init__(self, index=0):
        self.index = index

    @property
    def name(self):
        if not gpu_available():
            return "AMD GPU (not present)"
        buf = ctypes.create_string_buffer(256)
        _lib.check(_lib.lib.dpx_device_name(self.index, buf, len(buf)))
        return buf.value.decode()

    def __eq__(self, other):
        return isinstance(other, Device) and other.index == self.index

    def __hash__(self):
        return hash(("dpnp_amd.Device", self.index))

    def __repr__(self):
        return f"<Device hip:{self.index}>"


class Queue:
    """Stand-in for dpctl.SyclQueue: an in-order HIP stream on one device.

    With the torch provider the queue denotes the stream that is current in PyTorch at
    call time; with the native provider it is the library's one stream.
    """

    def __init__(self, device=None):
        self.sycl_device = device if isinstance(device, Device) else Device(0)

    @property
    def stream_ptr(self):
        return current_stream_ptr(self.sycl_device.index)

    def wait(self):
        _lib.check(_lib.lib.dpx_stream_synchronize(self.stream_ptr))

    def __eq__(self, other):
        return isinstance(other, Queue) and other.sycl_device == self.sycl_device

    def __hash__(self):
        return hash(("dpnp_amd.Queue", self.sycl_device.index))

    def __repr__(self):
        return f"<Queue on {self.sycl_device!r}>"


_raw_stream = None


def current_stream_ptr(device_index=0):
    """hipStream_t (as an integer) the library's kernels are enqueued on."""
    global _raw_stream
    if _raw_stream is None:
        if _NATIVE:
            _raw_stream = lambda i: _native_stream_ptr()  # noqa: E731
        else:
            t = _torch()
            fast = getattr(t._C, "_cuda_getCurrentRawStream", None)
            _raw_stream = fast if fast is not None else (lambda i: t.cuda.current_stream(i).cuda_stream)
    return _raw_stream(device_index)


_DEFAULT_QUEUE = Queue()


def default_queue():
    return _DEFAULT_QUEUE


def get_execution_queue(queues):
    """The common queue of `queues`, or None when they differ (compute follows data)."""
    qs = [q for q in queues if q is not None]
    if not qs:
        return None
    first = qs[0]
    return first if all(q == first for q in qs[1:]) else None


class Event:
    """Completion handle returned by the kernel entry points (in place of sycl::event)."""

    def __init__(self, queue=None):
        self._queue = queue or _DEFAULT_QUEUE

    def wait(self):
        self._queue.wait()


_gpu_count = None


def gpu_available():
    global _gpu_count
    if _gpu_count is None:
        if _NATIVE:
            n = ctypes.c_int(0)
            _lib.check(_lib.lib.dpx_device_count(ctypes.byref(n)))
            _gpu_count = n.value
        else:
            _gpu_count = 1 if _torch().cuda.is_available() else 0
    return _gpu_count > 0


_alloc_state = {}


_STAGGER_MIN = 4 << 20


def alloc(nbytes):
    """A device allocation of at least `nbytes` bytes (a uint8 CUDA tensor or a NativeBuffer)."""
    st = _alloc_state
    if not st:
        if not gpu_available():
            raise RuntimeError("dpnp_amd needs an AMD GPU: no HIP device is visible to this process")
        if not _NATIVE:
            t = _torch()
            st["empty"], st["u8"], st["dev"] = t.empty, t.uint8, t.device("cuda", t.cuda.current_device())
        st["ready"] = True
    if _NATIVE:
        nbytes = int(nbytes)
        if nbytes < _STAGGER_MIN:
            return NativeBuffer(nbytes)
        k = st["k"] = (st.get("k", 0) + 1) & 15
        return NativeBuffer(nbytes, (k * 12288) & 0xFFFF)  # staggered like the torch blocks below
    if nbytes < _STAGGER_MIN:
        return st["empty"](nbytes if nbytes > 0 else 1, dtype=st["u8"], device=st["dev"])
    # Large arrays start at staggered offsets (multiples of 12 KiB modulo 64 KiB) inside their
    # allocations.  The allocator aligns every large block to 2 MiB, so the operands of one
    # kernel would otherwise walk the memory channels in lockstep: fp32 add over 2^28 elements
    # runs at 6.67 TB/s with equal alignments and 6.79-6.82 TB/s with 4-12 KiB between them.
    k = st["k"] = (st.get("k", 0) + 1) & 15
    skew = (k * 12288) & 0xFFFF
    return st["empty"](nbytes + 65536, dtype=st["u8"], device=st["dev"])[skew:skew + nbytes]


def to_device_bytes(host_bytes_array):
    """Copy a contiguous NumPy uint8 array to a new device allocation."""
    if not gpu_available():
        raise RuntimeError("dpnp_amd needs an AMD GPU: no HIP device is visible to this process")
    n = int(host_bytes_array.size)
    buf = alloc(n)
    if n:
        _lib.check(_lib.lib.dpx_copy_from_host(buf.data_ptr(), host_bytes_array.ctypes.data, n,
                                               current_stream_ptr()))
    return buf


def to_host_bytes(buf, byte_offset, nbytes):
    """Copy `nbytes` bytes starting at `byte_offset` of allocation `buf` to a NumPy uint8 array."""
    out = np.empty(nbytes, dtype=np.uint8)
    if nbytes:
        _lib.check(_lib.lib.dpx_copy_to_host(out.ctypes.data, buf.data_ptr() + byte_offset, nbytes,
                                             current_stream_ptr()))
    return out
