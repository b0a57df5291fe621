"""ctypes binding of include/iomx.h, plus small helpers to hold tiled tensors
in device memory.  Everything here calls the HIP library; nothing computes on
the host."""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libiomx.so")
PROBE_LIB_PATH = os.path.join(HERE, "lib", "libiomx_probe.so")

# numeric values of iom::DataType (include/iom/tensor.hpp:10-33)
(DT_BOOL, DT_I2, DT_U2, DT_I4, DT_U4, DT_I8, DT_U8, DT_I16, DT_U16, DT_I32, DT_U32, DT_I64,
 DT_U64, DT_F4_E2M1, DT_F6_E2M3, DT_F6_E3M2, DT_F8_E4M3FN, DT_F8_E5M2, DT_F8_E8M0, DT_F16,
 DT_BF16, DT_F32, DT_F64) = range(23)
LEAF_BITS = (8, 2, 2, 4, 4, 8, 8, 16, 16, 32, 32, 64, 64, 4, 6, 6, 8, 8, 8, 16, 16, 32, 64)
OP_ADD, OP_MUL, OP_SUB, OP_DIV = 0, 1, 2, 3
# status codes of include/iomx.h (positive values are HIP error codes)
OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_OVERFLOW, ERR_EXHAUSTED = 0, -1, -2, -3, -4
TILE = 16


def carrier(dtype: int):
    """Unsigned numpy type that holds one raw element of the leaf."""
    bits = LEAF_BITS[dtype]
    return np.uint8 if bits <= 8 else {16: np.uint16, 32: np.uint32, 64: np.uint64}[bits]


NP_OF = {d: carrier(d) for d in range(23)}


def pack_bits(values: np.ndarray, bits: int) -> np.ndarray:
    """One element per item -> the packed host format: element i in bits
    [i*bits, (i+1)*bits) of a little-endian stream (src/cpu/transfer_helpers.hpp:14-40)."""
    values = np.ascontiguousarray(values).reshape(-1)
    if bits % 8 == 0:
        return values.view(np.uint8)
    planes = np.unpackbits(values.astype(np.uint8)[:, None], axis=1, bitorder="little")[:, :bits]
    return np.packbits(planes.reshape(-1), bitorder="little")


def unpack_bits(stream: np.ndarray, bits: int, count: int) -> np.ndarray:
    if bits % 8 == 0:
        return stream[:count * bits // 8].view(NP_OF[{8: 5, 16: 7, 32: 9, 64: 11}[bits]]).copy()
    flat = np.unpackbits(np.ascontiguousarray(stream, dtype=np.uint8), bitorder="little")
    full = np.zeros((count, 8), np.uint8)
    full[:, :bits] = flat[:count * bits].reshape(count, bits)
    return np.packbits(full, axis=1, bitorder="little").reshape(-1)

# every symbol include/iomx.h declares
SYMBOLS = [
    "iomx_error_string", "iomx_device_count", "iomx_set_device", "iomx_get_device",
    "iomx_get_device_props", "iomx_device_synchronize", "iomx_malloc", "iomx_free",
    "iomx_host_alloc", "iomx_host_free", "iomx_pointer_device", "iomx_fill_async",
    "iomx_memcpy_h2d", "iomx_memcpy_d2h", "iomx_memcpy_h2d_async", "iomx_memcpy_d2h_async",
    "iomx_memcpy_d2d_async", "iomx_stream_create", "iomx_stream_destroy",
    "iomx_stream_synchronize", "iomx_event_create", "iomx_event_destroy", "iomx_event_record",
    "iomx_event_synchronize", "iomx_event_query", "iomx_event_elapsed_ms", "iomx_host_device_address", "iomx_stream_write_word",
    "iomx_stream_begin_capture", "iomx_stream_end_capture", "iomx_graph_launch", "iomx_graph_destroy",
    "iomx_launch_linear", "iomx_sdpa_workspace", "iomx_launch_sdpa", "iomx_launch_sdpa_static",
    "iomx_launch_cache_append", "iomx_launch_embedding", "iomx_launch_rope",
    "iomx_launch_binary", "iomx_launch_rmsnorm", "iomx_launch_silu", "iomx_launch_silu_mul", "iomx_launch_add_rmsnorm",
    "iomx_launch_copy", "iomx_launch_scatter", "iomx_launch_gather", "iomx_launch_softmax",
    "iomx_last_launch",
]

# every symbol include/iomx_probe.h declares (libiomx_probe.so: measurement and self-tests,
# loaded by the benchmark and the tests only)
PROBE_SYMBOLS = ["iomx_probe_stream", "iomx_selftest_bf16_convert", "iomx_selftest_f16_binary"]


class View(C.Structure):
    _fields_ = [
        ("base", C.c_void_p), ("rank", C.c_uint32), ("dims", C.c_uint64 * 8),
        ("plane_offset", C.c_uint64), ("plane_strides", C.c_uint64 * 6),
    ]


class StageLayout(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "plane_offset", "plane_stride", "head_stride", "row_stride", "column_stride",
        "rows", "columns")]


class SoftmaxDesc(C.Structure):
    _fields_ = [
        ("planes", C.c_uint64), ("heads", C.c_uint64), ("rows", C.c_uint64),
        ("a", C.c_uint64), ("L", C.c_uint64), ("scale", C.c_float),
        ("scores", C.c_void_p), ("p_bf16", C.c_void_p),
        ("scores_layout", StageLayout), ("probability_layout", StageLayout),
    ]


class DeviceProps(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("compute_units", C.c_int), ("wavefront_size", C.c_int),
                ("lds_bytes_per_cu", C.c_int), ("global_bytes", C.c_uint64)]


class LaunchInfo(C.Structure):
    _fields_ = [("kernel", C.c_char * 48), ("grid", C.c_uint32), ("block", C.c_uint32),
                ("work_items", C.c_uint64)]


class IomxError(RuntimeError):
    def __init__(self, status: int, what: str):
        super().__init__(f"{what}: status {status}: {lib().iomx_error_string(status).decode()}")
        self.status = status


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    """The HIP library.  Raises when it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m iom_amd.build` "
                "(__graft_entry__.build()); iom_amd has no CPU fallback")
        l = C.CDLL(LIB_PATH)
        VP, P = C.POINTER(View), C.c_void_p
        l.iomx_error_string.restype = C.c_char_p
        l.iomx_error_string.argtypes = [C.c_int]
        l.iomx_device_count.argtypes = [C.POINTER(C.c_int)]
        l.iomx_set_device.argtypes = [C.c_int]
        l.iomx_get_device.argtypes = [C.POINTER(C.c_int)]
        l.iomx_get_device_props.argtypes = [C.c_int, C.POINTER(DeviceProps)]
        l.iomx_malloc.argtypes = [C.POINTER(P), C.c_size_t]
        l.iomx_free.argtypes = [P]
        l.iomx_host_alloc.argtypes = [C.POINTER(P), C.c_size_t]
        l.iomx_host_free.argtypes = [P]
        l.iomx_pointer_device.argtypes = [P, C.POINTER(C.c_int)]
        l.iomx_fill_async.argtypes = [P, C.c_uint8, C.c_size_t, P]
        for name in ("iomx_memcpy_h2d", "iomx_memcpy_d2h"):
            getattr(l, name).argtypes = [P, P, C.c_size_t]
        for name in ("iomx_memcpy_h2d_async", "iomx_memcpy_d2h_async", "iomx_memcpy_d2d_async"):
            getattr(l, name).argtypes = [P, P, C.c_size_t, P]
        l.iomx_stream_create.argtypes = [C.POINTER(P)]
        l.iomx_stream_destroy.argtypes = [P]
        l.iomx_stream_synchronize.argtypes = [P]
        l.iomx_event_create.argtypes = [C.POINTER(P), C.c_int]
        l.iomx_event_destroy.argtypes = [P]
        l.iomx_event_record.argtypes = [P, P]
        l.iomx_event_synchronize.argtypes = [P]
        l.iomx_event_query.argtypes = [P, C.POINTER(C.c_int)]
        l.iomx_host_device_address.argtypes = [P, C.POINTER(P)]
        l.iomx_stream_write_word.argtypes = [P, P, C.c_uint32]
        l.iomx_event_elapsed_ms.argtypes = [P, P, C.POINTER(C.c_float)]
        l.iomx_launch_binary.argtypes = [C.c_int, C.c_int, VP, VP, VP, P]
        l.iomx_launch_rmsnorm.argtypes = [C.c_int, VP, VP, VP, C.c_float, P]
        l.iomx_stream_begin_capture.argtypes = [P]
        l.iomx_stream_end_capture.argtypes = [P, C.POINTER(C.c_void_p)]
        l.iomx_graph_launch.argtypes = [P, P]
        l.iomx_graph_destroy.argtypes = [P]
        l.iomx_launch_silu.argtypes = [C.c_int, VP, VP, P]
        l.iomx_launch_silu_mul.argtypes = [C.c_int, VP, VP, VP, P]
        l.iomx_launch_add_rmsnorm.argtypes = [C.c_int, VP, VP, VP, VP, VP, C.c_float, P]
        l.iomx_launch_copy.argtypes = [C.c_int, VP, VP, P]
        l.iomx_launch_cache_append.argtypes = [C.c_int, VP, VP, C.c_uint64, P]
        l.iomx_launch_linear.argtypes = [C.c_int, VP, VP, VP, C.c_uint64, C.c_uint64, C.c_int, C.c_uint64,
                                         C.c_uint64, C.c_int, P]
        l.iomx_sdpa_workspace.argtypes = [C.c_int, VP, VP, VP, VP, C.c_uint64, C.c_uint64,
                                          C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        l.iomx_launch_sdpa.argtypes = [C.c_int, VP, VP, VP, VP, C.c_uint64, C.c_uint64, C.c_void_p,
                                       C.c_uint64, C.c_int, C.c_void_p]
        l.iomx_launch_sdpa_static.argtypes = [C.c_int, VP, VP, VP, VP, C.c_uint64, C.c_uint64,
                                              C.c_int, C.c_void_p]
        l.iomx_launch_embedding.argtypes = [C.c_int, C.c_int, VP, VP, VP, P, P]
        l.iomx_launch_rope.argtypes = [C.c_int, VP, VP, C.c_uint64, C.c_double, P]
        l.iomx_launch_scatter.argtypes = [C.c_int, VP, P, P]
        l.iomx_launch_gather.argtypes = [C.c_int, VP, P, P]
        l.iomx_launch_softmax.argtypes = [C.POINTER(SoftmaxDesc), P]
        l.iomx_last_launch.argtypes = [C.POINTER(LaunchInfo)]
        _lib = l
    return _lib


def check(status: int, what: str = "iomx") -> None:
    if status != 0:
        raise IomxError(status, what)


def device_count() -> int:
    n = C.c_int(0)
    status = lib().iomx_device_count(C.byref(n))
    return n.value if status == 0 else 0


def device_props(ordinal: int = 0) -> DeviceProps:
    p = DeviceProps()
    check(lib().iomx_get_device_props(ordinal, C.byref(p)), "get_device_props")
    return p


def synchronize() -> None:
    check(lib().iomx_device_synchronize(), "device_synchronize")


def last_launch() -> LaunchInfo:
    info = LaunchInfo()
    check(lib().iomx_last_launch(C.byref(info)))
    return info


class Stream:
    def __init__(self):
        self.h = C.c_void_p()
        check(lib().iomx_stream_create(C.byref(self.h)), "stream_create")

    def synchronize(self):
        check(lib().iomx_stream_synchronize(self.h), "stream_synchronize")

    def close(self):
        if self.h:
            lib().iomx_stream_destroy(self.h)
            self.h = C.c_void_p()

    def begin_capture(self):
        check(lib().iomx_stream_begin_capture(self.h), "begin_capture")

    def end_capture(self) -> "Graph":
        g = C.c_void_p()
        check(lib().iomx_stream_end_capture(self.h, C.byref(g)), "end_capture")
        return Graph(g)


class Graph:
    """A recorded sequence of launches, replayed with one submission."""

    def __init__(self, handle):
        self.h = handle

    def launch(self, stream: "Stream"):
        check(lib().iomx_graph_launch(self.h, stream.h), "graph_launch")

    def close(self):
        if self.h:
            lib().iomx_graph_destroy(self.h)
            self.h = C.c_void_p()


class Event:
    def __init__(self, timing: bool = True):
        self.h = C.c_void_p()
        check(lib().iomx_event_create(C.byref(self.h), int(timing)), "event_create")

    def record(self, stream: Optional[Stream] = None):
        check(lib().iomx_event_record(self.h, stream.h if stream else None), "event_record")

    def synchronize(self):
        check(lib().iomx_event_synchronize(self.h), "event_synchronize")

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        check(lib().iomx_event_elapsed_ms(self.h, stop.h, C.byref(ms)), "event_elapsed")
        return ms.value

    def close(self):
        if self.h:
            lib().iomx_event_destroy(self.h)
            self.h = C.c_void_p()


_STAGE_BYTES = 32 << 20
_stage = None


def _staging():
    """(address, numpy window) of one page-locked host buffer, allocated on first use and kept
    for the life of the process.  Every transfer of this module goes host array -> this buffer
    (a numpy copy) -> device by an asynchronous copy that is waited for, and back the same way:
    the runtime then always moves page-locked memory by DMA and never has to choose, per call
    and per size, between pinning the caller's pages, its own staging copies and direct host
    access to device memory."""
    global _stage
    if _stage is None:
        p = C.c_void_p()
        check(lib().iomx_host_alloc(C.byref(p), _STAGE_BYTES), "host_alloc")
        _stage = (p.value, np.ctypeslib.as_array((C.c_uint8 * _STAGE_BYTES).from_address(p.value)))
    return _stage


class Buffer:
    """One device allocation."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = C.c_void_p()
        check(lib().iomx_malloc(C.byref(self.ptr), max(self.nbytes, 16)), "malloc")

    def upload(self, arr: np.ndarray, offset: int = 0):
        """Host array -> device, through the page-locked staging buffer (see _staging)."""
        arr = np.ascontiguousarray(arr)
        if not self.ptr or offset < 0 or offset + arr.nbytes > self.nbytes:
            raise ValueError(f"upload of {arr.nbytes} bytes at {offset} into a buffer of {self.nbytes}")
        src = arr.reshape(-1).view(np.uint8)
        address, window = _staging()
        for at in range(0, src.size, _STAGE_BYTES):
            m = min(_STAGE_BYTES, src.size - at)
            window[:m] = src[at:at + m]
            check(lib().iomx_memcpy_h2d_async(self.ptr.value + offset + at, address, m, None), "h2d")
            check(lib().iomx_stream_synchronize(None), "h2d sync")

    def download(self, dtype, count: Optional[int] = None, offset: int = 0) -> np.ndarray:
        itemsize = np.dtype(dtype).itemsize
        if count is None:
            count = (self.nbytes - offset) // itemsize
        if not self.ptr or offset < 0 or count < 0 or offset + count * itemsize > self.nbytes:
            raise ValueError(f"download of {count} x {itemsize} bytes at {offset} from a buffer of {self.nbytes}")
        out = np.empty(count, dtype=dtype)
        dst = out.view(np.uint8)
        address, window = _staging()
        for at in range(0, dst.size, _STAGE_BYTES):
            m = min(_STAGE_BYTES, dst.size - at)
            check(lib().iomx_memcpy_d2h_async(address, self.ptr.value + offset + at, m, None), "d2h")
            check(lib().iomx_stream_synchronize(None), "d2h sync")
            dst[at:at + m] = window[:m]
        return out

    def fill(self, byte: int, stream: Optional[Stream] = None):
        check(lib().iomx_fill_async(self.ptr, byte, self.nbytes, stream.h if stream else None), "fill")

    def free(self):
        if self.ptr:
            lib().iomx_free(self.ptr)
            self.ptr = C.c_void_p()


def padded(n: int) -> int:
    return (n + TILE - 1) // TILE * TILE


def leaf_bytes(dtype: int) -> int:
    assert LEAF_BITS[dtype] % 8 == 0
    return LEAF_BITS[dtype] // 8


class DeviceTensor:
    """Owner storage in the standard tiled layout, in device memory, with the
    leading-axis view transforms of iom::TensorView (src/tensor_view.cpp:99-256)."""

    def __init__(self, dtype: int, dims: Sequence[int], fill: Optional[int] = 0):
        self.dtype = dtype
        self.dims = tuple(int(d) for d in dims)
        lead = self.dims[:-2]
        self.planes = int(np.prod(lead, dtype=np.int64)) if lead else 1
        self.plane_elems = padded(self.dims[-2]) * padded(self.dims[-1])
        self.bits = LEAF_BITS[dtype]
        self.nbytes = self.planes * self.plane_elems * self.bits // 8
        self.buf = Buffer(self.nbytes)
        if fill is not None:
            self.buf.fill(fill)

    def view(self) -> "DeviceView":
        lead = self.dims[:-2]
        strides, s = [], 1
        for d in reversed(lead):
            strides.append(s)
            s *= d
        return DeviceView(self, self.dims, 0, tuple(reversed(strides)))

    def raw(self) -> np.ndarray:
        """The owner storage: one item per slot for byte-sized leaves, bytes otherwise."""
        synchronize()
        return self.buf.download(NP_OF[self.dtype] if self.bits % 8 == 0 else np.uint8)

    def upload_raw(self, storage: np.ndarray):
        assert storage.nbytes == self.nbytes
        self.buf.upload(storage)

    def free(self):
        self.buf.free()


class DeviceView:
    def __init__(self, owner: DeviceTensor, dims, plane_offset, plane_strides):
        self.owner = owner
        self.dims = tuple(int(d) for d in dims)
        self.plane_offset = int(plane_offset)
        self.plane_strides = tuple(int(s) for s in plane_strides)

    @property
    def dtype(self):
        return self.owner.dtype

    def slice(self, dim, first, count, step=1):
        lead = list(self.dims[:-2])
        assert dim < len(lead) and count > 0 and step > 0 and first + (count - 1) * step < lead[dim]
        strides = list(self.plane_strides)
        off = self.plane_offset + first * strides[dim]
        lead[dim] = count
        strides[dim] *= step
        return DeviceView(self.owner, tuple(lead) + self.dims[-2:], off, strides)

    def select(self, dim, index):
        lead = list(self.dims[:-2])
        assert dim < len(lead) and index < lead[dim]
        strides = list(self.plane_strides)
        off = self.plane_offset + index * strides[dim]
        del lead[dim]
        del strides[dim]
        return DeviceView(self.owner, tuple(lead) + self.dims[-2:], off, strides)

    def permute(self, order):
        lead = self.dims[:-2]
        assert sorted(order) == list(range(len(lead)))
        return DeviceView(self.owner, tuple(lead[i] for i in order) + self.dims[-2:],
                          self.plane_offset, [self.plane_strides[i] for i in order])

    def reshape_leading(self, new_lead):
        lead = self.dims[:-2]
        assert int(np.prod(new_lead, dtype=np.int64)) == int(np.prod(lead, dtype=np.int64))
        expected = 1
        for d, s in zip(reversed(lead), reversed(self.plane_strides)):
            if d > 1:
                assert s == expected
                expected *= d
        strides, s = [], 1
        for d in reversed(new_lead):
            strides.append(s)
            s *= d
        return DeviceView(self.owner, tuple(new_lead) + self.dims[-2:], self.plane_offset,
                          tuple(reversed(strides)))

    def cview(self) -> View:
        v = View()
        v.base = self.owner.buf.ptr.value
        v.rank = len(self.dims)
        for i, d in enumerate(self.dims):
            v.dims[i] = d
        v.plane_offset = self.plane_offset
        for i, s in enumerate(self.plane_strides):
            v.plane_strides[i] = s
        return v

    @property
    def logical_count(self) -> int:
        return int(np.prod(self.dims, dtype=np.int64))

    def from_host(self, arr: np.ndarray, stream: Optional[Stream] = None):
        """copy_from_host: one raw element per item -> packed logical stream -> staging
        (a whole number of 32-bit words, as the reference's workspace is) -> scatter."""
        arr = np.ascontiguousarray(arr, dtype=NP_OF[self.dtype]).reshape(-1)
        assert arr.size == self.logical_count
        stream_bytes = pack_bits(arr, LEAF_BITS[self.dtype])
        staging = Buffer((stream_bytes.size + 3) // 4 * 4)
        try:
            staging.upload(stream_bytes)
            cv = self.cview()
            check(lib().iomx_launch_scatter(self.dtype, C.byref(cv), staging.ptr,
                                            stream.h if stream else None), "scatter")
            (stream.synchronize() if stream else synchronize())
        finally:
            staging.free()

    def to_host(self, stream: Optional[Stream] = None) -> np.ndarray:
        return unpack_bits(self.to_host_stream(stream), LEAF_BITS[self.dtype],
                           self.logical_count).reshape(self.dims)

    def to_host_stream(self, stream: Optional[Stream] = None) -> np.ndarray:
        """The packed logical bytes exactly as the gather kernel wrote them."""
        nbytes = (self.logical_count * LEAF_BITS[self.dtype] + 7) // 8
        staging = Buffer((nbytes + 3) // 4 * 4)
        try:
            staging.fill(0xEE)
            synchronize()
            cv = self.cview()
            check(lib().iomx_launch_gather(self.dtype, C.byref(cv), staging.ptr,
                                           stream.h if stream else None), "gather")
            (stream.synchronize() if stream else synchronize())
            return staging.download(np.uint8)[:nbytes]
        finally:
            staging.free()


def _h(stream):
    return stream.h if stream else None


def binary(op: int, lhs: DeviceView, rhs: DeviceView, out: DeviceView, stream=None) -> int:
    a, b, o = lhs.cview(), rhs.cview(), out.cview()
    return lib().iomx_launch_binary(op, out.dtype, C.byref(a), C.byref(b), C.byref(o), _h(stream))


def rmsnorm(x: DeviceView, scale: DeviceView, out: DeviceView, eps: float, stream=None) -> int:
    a, b, o = x.cview(), scale.cview(), out.cview()
    return lib().iomx_launch_rmsnorm(out.dtype, C.byref(a), C.byref(b), C.byref(o), eps, _h(stream))


def add_rmsnorm(x: DeviceView, y: DeviceView, total: DeviceView, scale: DeviceView, out: DeviceView,
                eps: float, stream=None) -> int:
    """total = x + y, out = rmsnorm(total, scale): the private fusion of ADD and RMSNorm."""
    a, b, t, w, o = x.cview(), y.cview(), total.cview(), scale.cview(), out.cview()
    return lib().iomx_launch_add_rmsnorm(out.dtype, C.byref(a), C.byref(b), C.byref(t), C.byref(w), C.byref(o),
                                         eps, _h(stream))


def silu(x: DeviceView, y: DeviceView, stream=None) -> int:
    a, o = x.cview(), y.cview()
    return lib().iomx_launch_silu(y.dtype, C.byref(a), C.byref(o), _h(stream))


def silu_mul(gate: DeviceView, up: DeviceView, y: DeviceView, stream=None) -> int:
    a, b, o = gate.cview(), up.cview(), y.cview()
    return lib().iomx_launch_silu_mul(y.dtype, C.byref(a), C.byref(b), C.byref(o), _h(stream))


def copy(src: DeviceView, dst: DeviceView, stream=None) -> int:
    a, o = src.cview(), dst.cview()
    return lib().iomx_launch_copy(dst.dtype, C.byref(a), C.byref(o), _h(stream))


def linear(x: DeviceView, w: DeviceView, out: DeviceView, s: int, R: int, head_planar: bool, H: int, D: int,
           path: int = 0, stream: Optional[Stream] = None) -> int:
    a, b, o = x.cview(), w.cview(), out.cview()
    return lib().iomx_launch_linear(out.dtype, C.byref(a), C.byref(b), C.byref(o), s, R, int(head_planar),
                                    H, D, path, _h(stream))


def sdpa_workspace(q: DeviceView, k: DeviceView, v: DeviceView, out: DeviceView, a: int, L: int):
    """(status, bytes, alignment) of the caller workspace sdpa needs for these operands."""
    cq, ck, cv, co = q.cview(), k.cview(), v.cview(), out.cview()
    nbytes, align = C.c_uint64(0), C.c_uint64(0)
    rc = lib().iomx_sdpa_workspace(out.dtype, C.byref(cq), C.byref(ck), C.byref(cv), C.byref(co), a, L,
                                   C.byref(nbytes), C.byref(align))
    return rc, nbytes.value, align.value


def sdpa(q: DeviceView, k: DeviceView, v: DeviceView, out: DeviceView, a: int, L: int,
         workspace: Optional["Buffer"] = None, path: int = 0, stream: Optional[Stream] = None) -> int:
    cq, ck, cv, co = q.cview(), k.cview(), v.cview(), out.cview()
    return lib().iomx_launch_sdpa(out.dtype, C.byref(cq), C.byref(ck), C.byref(cv), C.byref(co), a, L,
                                  workspace.ptr if workspace is not None else None,
                                  workspace.nbytes if workspace is not None else 0, path, _h(stream))


PROBE_READ, PROBE_WRITE, PROBE_COPY, PROBE_ADD, PROBE_HELD_COPY = range(5)
PROBE_KERNEL = ("probe_read", "probe_write", "probe_copy", "probe_add", "probe_held_copy")

_probe_lib: Optional[C.CDLL] = None


def probe_lib() -> C.CDLL:
    """The measurement and self-test library (include/iomx_probe.h).  Raises when not built."""
    global _probe_lib
    if _probe_lib is None:
        lib()   # the backend library first: both must see one HIP runtime state
        if not os.path.exists(PROBE_LIB_PATH):
            raise ImportError(f"{PROBE_LIB_PATH} is missing: build it with `python -m iom_amd.build`")
        l = C.CDLL(PROBE_LIB_PATH)
        P = C.c_void_p
        l.iomx_selftest_bf16_convert.argtypes = [C.POINTER(C.c_uint64), P]
        l.iomx_selftest_f16_binary.argtypes = [C.POINTER(C.c_uint64), P]
        l.iomx_probe_stream.argtypes = [C.c_int, P, P, P, C.c_uint64, P]
        _probe_lib = l
    return _probe_lib


def probe_stream(mode: int, a: Optional["Buffer"], b: Optional["Buffer"], out: "Buffer", nbytes: int,
                 stream: Optional[Stream] = None) -> int:
    """One launch of a bare bandwidth probe over `nbytes` bytes per operand."""
    return probe_lib().iomx_probe_stream(mode, a.ptr if a is not None else None,
                                         b.ptr if b is not None else None, out.ptr, nbytes, _h(stream))


SDPA_STATIC_BYTES = 16 << 20


def sdpa_static(q: DeviceView, k: DeviceView, v: DeviceView, out: DeviceView, a: int, L: int,
                path: int = 0, stream: Optional[Stream] = None) -> int:
    """sdpa() with the workspace in the library's fixed per-GPU array: no allocation."""
    cq, ck, cv, co = q.cview(), k.cview(), v.cview(), out.cview()
    return lib().iomx_launch_sdpa_static(out.dtype, C.byref(cq), C.byref(ck), C.byref(cv),
                                         C.byref(co), a, L, path, _h(stream))


def cache_append(src: DeviceView, dst: DeviceView, a: int, stream: Optional[Stream] = None) -> int:
    s_, d = src.cview(), dst.cview()
    return lib().iomx_launch_cache_append(dst.dtype, C.byref(s_), C.byref(d), C.c_uint64(a), _h(stream))


def embedding(table: DeviceView, indices: DeviceView, out: DeviceView, status: "Buffer",
              stream: Optional[Stream] = None) -> int:
    """`status` is a device buffer of at least 4 bytes; read word 0 after completion."""
    t, i_, o = table.cview(), indices.cview(), out.cview()
    return lib().iomx_launch_embedding(out.dtype, indices.dtype, C.byref(t), C.byref(i_), C.byref(o),
                                       status.ptr, _h(stream))


def rope(x: DeviceView, out: DeviceView, a: int, theta: float, stream: Optional[Stream] = None) -> int:
    s_, o = x.cview(), out.cview()
    return lib().iomx_launch_rope(out.dtype, C.byref(s_), C.byref(o), C.c_uint64(a), C.c_double(theta),
                                  _h(stream))


def dense_layout(heads: int, rows: int, cols: int) -> StageLayout:
    l = StageLayout()
    l.plane_offset, l.plane_stride, l.head_stride = 0, heads * rows * cols, rows * cols
    l.row_stride, l.column_stride, l.rows, l.columns = cols, 1, rows, cols
    return l


def softmax_desc(scores_ptr: int, p_ptr: int, planes: int, heads: int, prows: int, pcols: int,
                 a: int, L: int, scale: float = 1.0, rows: Optional[int] = None) -> SoftmaxDesc:
    d = SoftmaxDesc()
    d.planes, d.heads, d.rows = planes, heads, prows if rows is None else rows
    d.a, d.L, d.scale = a, L, scale
    d.scores, d.p_bf16 = scores_ptr, p_ptr
    d.scores_layout = dense_layout(heads, prows, pcols)
    d.probability_layout = dense_layout(heads, prows, pcols)
    return d


def softmax(desc: SoftmaxDesc, stream=None) -> int:
    return lib().iomx_launch_softmax(C.byref(desc), _h(stream))
