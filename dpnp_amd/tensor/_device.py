"""Device memory and the execution stream.

PyTorch is used as plumbing only: its caching allocator hands out device memory
(a uint8 CUDA tensor per allocation) and its current stream is the hipStream_t
every kernel of the library is enqueued on.  The allocator is stream-ordered, so
a temporary released right after a launch is not reused before that launch ran.
"""
import numpy as np


def _torch():
    import torch

    return torch


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
        t = _torch()
        return t.cuda.get_device_name(self.index) if t.cuda.is_available() else "AMD GPU (not present)"

    def __eq__(self, other):
        return isinstance(other, Device) and other.index == self.index

    def __hash__(self):
        return hash(("dpnp_amd.Device", self.index))

    def __repr__(self):
        return f"<Device hip:{self.index}>"


class Queue:
    """Stand-in for dpctl.SyclQueue: an in-order HIP stream on one device.

    The queue always denotes the stream that is current in PyTorch at call
    time, so work submitted by this library interleaves correctly with torch
    work of the same process.
    """

    def __init__(self, device=None):
        self.sycl_device = device if isinstance(device, Device) else Device(0)

    @property
    def stream_ptr(self):
        return current_stream_ptr(self.sycl_device.index)

    def wait(self):
        _torch().cuda.current_stream(self.sycl_device.index).synchronize()

    def __eq__(self, other):
        return isinstance(other, Queue) and other.sycl_device == self.sycl_device

    def __hash__(self):
        return hash(("dpnp_amd.Queue", self.sycl_device.index))

    def __repr__(self):
        return f"<Queue on {self.sycl_device!r}>"


_raw_stream = None


def current_stream_ptr(device_index=0):
    """hipStream_t (as an integer) of torch's current stream on the device."""
    global _raw_stream
    if _raw_stream is None:
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


def gpu_available():
    t = _torch()
    return t.cuda.is_available()


_alloc_state = {}


_STAGGER_MIN = 4 << 20


def alloc(nbytes):
    """A device allocation of at least `nbytes` bytes (a uint8 CUDA tensor)."""
    st = _alloc_state
    if not st:
        t = _torch()
        if not t.cuda.is_available():
            raise RuntimeError("dpnp_amd needs an AMD GPU: no HIP device is visible to this process")
        st["empty"], st["u8"], st["dev"] = t.empty, t.uint8, t.device("cuda", t.cuda.current_device())
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
    t = _torch()
    if not t.cuda.is_available():
        raise RuntimeError("dpnp_amd needs an AMD GPU: no HIP device is visible to this process")
    n = int(host_bytes_array.size)
    buf = alloc(n)
    if n:
        from .. import _lib

        _lib.check(_lib.lib.dpx_copy_from_host(buf.data_ptr(), host_bytes_array.ctypes.data, n,
                                               current_stream_ptr()))
    return buf


def to_host_bytes(buf, byte_offset, nbytes):
    """Copy `nbytes` bytes starting at `byte_offset` of allocation `buf` to a NumPy uint8 array."""
    out = np.empty(nbytes, dtype=np.uint8)
    if nbytes:
        from .. import _lib

        _lib.check(_lib.lib.dpx_copy_to_host(out.ctypes.data, buf.data_ptr() + byte_offset, nbytes,
                                             current_stream_ptr()))
    return out
