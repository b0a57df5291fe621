"""ctypes bindings for the test-only checkers.

TEST INFRASTRUCTURE: only tests, the smoke check and the benchmark's
CPU-baseline leg may import this module.  Two libraries are wrapped:

* ``libiom_oracle.so`` – this repository's C restatement of the reference CPU
  backend (``iom_oracle.h``).
* ``_ref/libiom_ref.so`` – the reference's own CPU backend compiled from its
  sources (``make ref``), driven through the ``iomc_*`` handle API of
  ``iomc_shim.cpp``.  Present only where it has been built.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# numeric values of iom::DataType (include/iom/tensor.hpp:10-33)
(DT_BOOL, DT_I2, DT_U2, DT_I4, DT_U4, DT_I8, DT_U8, DT_I16, DT_U16, DT_I32, DT_U32, DT_I64,
 DT_U64, DT_F4_E2M1, DT_F6_E2M3, DT_F6_E3M2, DT_F8_E4M3FN, DT_F8_E5M2, DT_F8_E8M0, DT_F16,
 DT_BF16, DT_F32, DT_F64) = range(23)
ALL_LEAVES = tuple(range(23))
LEAF_NAME = ("BOOL I2 U2 I4 U4 I8 U8 I16 U16 I32 U32 I64 U64 F4_E2M1 F6_E2M3 F6_E3M2 "
             "F8_E4M3FN F8_E5M2 F8_E8M0 F16 BF16 F32 F64").split()
LEAF_BITS = (8, 2, 2, 4, 4, 8, 8, 16, 16, 32, 32, 64, 64, 4, 6, 6, 8, 8, 8, 16, 16, 32, 64)
INTEGER_LEAVES = tuple(range(DT_I2, DT_U64 + 1))
FLOAT_LEAVES = (DT_F4_E2M1, DT_F6_E2M3, DT_F6_E3M2, DT_F8_E4M3FN, DT_F8_E5M2, DT_F16, DT_BF16,
                DT_F32, DT_F64)
NUMERIC_LEAVES = INTEGER_LEAVES + FLOAT_LEAVES     # BOOL and F8_E8M0 carry no arithmetic
OP_ADD, OP_MUL, OP_SUB, OP_DIV = 0, 1, 2, 3
TILE = 16


def carrier(dtype: int):
    """Unsigned numpy type holding one raw element (all arithmetic is on bit patterns)."""
    bits = LEAF_BITS[dtype]
    return np.uint8 if bits <= 8 else {16: np.uint16, 32: np.uint32, 64: np.uint64}[bits]


NP_OF = {d: carrier(d) for d in ALL_LEAVES}


def leaf_bytes(dtype: int) -> int:
    assert LEAF_BITS[dtype] % 8 == 0
    return LEAF_BITS[dtype] // 8


def pack_bits(values: np.ndarray, bits: int) -> np.ndarray:
    """Elements -> the packed little-endian bit stream of the host format
    (element i in bits [i*bits, (i+1)*bits), least significant bit first)."""
    values = np.ascontiguousarray(values).reshape(-1)
    if bits % 8 == 0:
        return values.view(np.uint8).copy()
    planes = np.unpackbits(values.astype(np.uint8)[:, None], axis=1, bitorder="little")[:, :bits]
    return np.packbits(planes.reshape(-1), bitorder="little")


def unpack_bits(stream: np.ndarray, bits: int, count: int) -> np.ndarray:
    if bits % 8 == 0:
        return stream.view({8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[bits])[:count].copy()
    flat = np.unpackbits(np.ascontiguousarray(stream, dtype=np.uint8), bitorder="little")
    flat = flat[:count * bits].reshape(count, bits)
    full = np.zeros((count, 8), np.uint8)
    full[:, :bits] = flat
    return np.packbits(full, axis=1, bitorder="little").reshape(-1)


def packed_nbytes(count: int, bits: int) -> int:
    return (count * bits + 7) // 8


class View(C.Structure):
    _fields_ = [
        ("base", C.c_void_p),
        ("rank", C.c_uint32),
        ("dims", C.c_uint64 * 8),
        ("plane_offset", C.c_uint64),
        ("plane_strides", C.c_uint64 * 6),
    ]


class StageLayout(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "plane_offset", "plane_stride", "head_stride", "row_stride",
        "column_stride", "rows", "columns")]


class SoftmaxDesc(C.Structure):
    _fields_ = [
        ("planes", C.c_uint64), ("heads", C.c_uint64), ("rows", C.c_uint64),
        ("a", C.c_uint64), ("L", C.c_uint64), ("scale", C.c_float),
        ("scores", C.c_void_p), ("p_bf16", C.c_void_p),
        ("scores_layout", StageLayout), ("probability_layout", StageLayout),
    ]


def _load(path: str) -> C.CDLL:
    if not os.path.exists(path):
        raise FileNotFoundError(
            f"{path} is not built; run `make -C {HERE}` (or __graft_entry__.build())")
    return C.CDLL(path)


_lib: Optional[C.CDLL] = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        l = _load(os.path.join(HERE, "libiom_oracle.so"))
        VP = C.POINTER(View)
        l.iomo_plane_slot.restype = C.c_uint64
        l.iomo_plane_slot.argtypes = [C.c_uint64] * 5
        l.iomo_plane_elems.restype = C.c_uint64
        l.iomo_plane_elems.argtypes = [C.c_uint64] * 2
        l.iomo_scalar_binary.restype = C.c_uint64
        l.iomo_scalar_binary.argtypes = [C.c_int, C.c_int, C.c_uint64, C.c_uint64]
        l.iomo_scalar_binary_ieee.restype = C.c_uint64
        l.iomo_scalar_binary_ieee.argtypes = [C.c_int, C.c_int, C.c_uint64, C.c_uint64]
        l.iomo_scalar_silu.restype = C.c_uint64
        l.iomo_scalar_silu.argtypes = [C.c_int, C.c_uint64]
        l.iomo_encode_bf16.restype = C.c_uint16
        l.iomo_encode_bf16.argtypes = [C.c_float]
        l.iomo_binary.argtypes = [C.c_int, C.c_int, VP, VP, VP, C.c_int]
        l.iomo_rmsnorm.argtypes = [C.c_int, VP, VP, VP, C.c_float]
        l.iomo_silu.argtypes = [C.c_int, VP, VP]
        l.iomo_copy.argtypes = [C.c_int, VP, VP]
        l.iomo_scatter.argtypes = [C.c_int, VP, C.c_void_p]
        l.iomo_gather.argtypes = [C.c_int, VP, C.c_void_p]
        l.iomo_softmax.argtypes = [C.POINTER(SoftmaxDesc)]
        l.iomo_cache_append.argtypes = [C.c_int, VP, VP, C.c_uint64]
        l.iomo_embedding.argtypes = [C.c_int, C.c_int, VP, VP, VP]
        l.iomo_rope.argtypes = [C.c_int, VP, VP, C.c_uint64, C.c_double]
        l.iomo_linear.argtypes = [C.c_int, VP, VP, VP, C.c_uint64, C.c_uint64, C.c_int, C.c_uint64, C.c_uint64]
        l.iomo_sdpa.argtypes = [C.c_int, VP, VP, VP, VP, C.c_uint64, C.c_uint64]
        _lib = l
    return _lib


# --------------------------------------------------------------------------
# Host-side tensors in tiled storage (numpy), with leading-axis views.
# --------------------------------------------------------------------------

def padded(n: int) -> int:
    return (n + TILE - 1) // TILE * TILE


def plane_elems(rows: int, cols: int) -> int:
    return padded(rows) * padded(cols)


class HostTensor:
    """Owner storage in the standard 16x16 tiled layout, held in numpy.

    Mirrors ``iom::Tensor`` + ``iom::TensorView`` (include/iom/tensor.hpp:262-411)
    as far as the checkers need: a full view plus slice/select/permute/
    reshape_leading returning new views over the same storage.
    """

    def __init__(self, dtype: int, dims: Sequence[int], fill: Optional[int] = None):
        self.dtype = dtype
        self.dims = tuple(int(d) for d in dims)
        assert 2 <= len(self.dims) <= 8 and all(d > 0 for d in self.dims)
        planes = int(np.prod(self.dims[:-2], dtype=np.int64)) if len(self.dims) > 2 else 1
        self.planes = planes
        n = planes * plane_elems(self.dims[-2], self.dims[-1])
        self.bits = LEAF_BITS[dtype]
        # byte-sized leaves: one array item per slot; narrower ones: the packed bytes
        if self.bits % 8 == 0:
            self.storage = np.zeros(n, dtype=NP_OF[dtype])
        else:
            self.storage = np.zeros(n * self.bits // 8, dtype=np.uint8)
        if fill is not None:
            self.storage.view(np.uint8)[:] = fill

    def view(self) -> "HostView":
        lead = self.dims[:-2]
        strides = []
        s = 1
        for d in reversed(lead):
            strides.append(s)
            s *= d
        return HostView(self, self.dims, 0, tuple(reversed(strides)))


class HostView:
    def __init__(self, owner: HostTensor, dims, plane_offset: int, plane_strides):
        self.owner = owner
        self.dims = tuple(int(d) for d in dims)
        self.plane_offset = int(plane_offset)
        self.plane_strides = tuple(int(s) for s in plane_strides)

    @property
    def dtype(self) -> int:
        return self.owner.dtype

    # src/tensor_view.cpp:99-256
    def slice(self, dim, first, count, step=1):
        lead = list(self.dims[:-2])
        assert dim < len(lead) and count > 0 and step > 0
        assert first + (count - 1) * step < lead[dim]
        strides = list(self.plane_strides)
        off = self.plane_offset + first * strides[dim]
        lead[dim] = count
        strides[dim] *= step
        return HostView(self.owner, tuple(lead) + self.dims[-2:], off, strides)

    def select(self, dim, index):
        lead = list(self.dims[:-2])
        assert dim < len(lead) and index < lead[dim]
        strides = list(self.plane_strides)
        off = self.plane_offset + index * strides[dim]
        del lead[dim]
        del strides[dim]
        return HostView(self.owner, tuple(lead) + self.dims[-2:], off, strides)

    def permute(self, order):
        lead = self.dims[:-2]
        assert sorted(order) == list(range(len(lead)))
        return HostView(self.owner, tuple(lead[i] for i in order) + self.dims[-2:],
                        self.plane_offset, [self.plane_strides[i] for i in order])

    def reshape_leading(self, new_lead):
        lead = self.dims[:-2]
        assert int(np.prod(new_lead, dtype=np.int64)) == int(np.prod(lead, dtype=np.int64))
        expected = 1
        for d, s in zip(reversed(lead), reversed(self.plane_strides)):
            if d > 1:
                assert s == expected, "reshape requires a contiguous view"
                expected *= d
        strides = []
        s = 1
        for d in reversed(new_lead):
            strides.append(s)
            s *= d
        return HostView(self.owner, tuple(new_lead) + self.dims[-2:], self.plane_offset,
                        tuple(reversed(strides)))

    def cview(self, base: Optional[int] = None) -> View:
        v = View()
        v.base = self.owner.storage.ctypes.data if base is None else base
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

    def from_logical(self, arr: np.ndarray) -> None:
        """region_from_host: one raw element per array item, in the view's logical shape."""
        arr = np.ascontiguousarray(arr, dtype=NP_OF[self.dtype]).reshape(-1)
        assert arr.size == self.logical_count
        stream = pack_bits(arr, LEAF_BITS[self.dtype])
        cv = self.cview()
        rc = lib().iomo_scatter(self.dtype, C.byref(cv), stream.ctypes.data)
        assert rc == 0, rc

    def to_logical(self) -> np.ndarray:
        bits = LEAF_BITS[self.dtype]
        stream = np.full(packed_nbytes(self.logical_count, bits), 0xEE, dtype=np.uint8)
        cv = self.cview()
        rc = lib().iomo_gather(self.dtype, C.byref(cv), stream.ctypes.data)
        assert rc == 0, rc
        return unpack_bits(stream, bits, self.logical_count).reshape(self.dims)

    def slots(self) -> np.ndarray:
        """Every slot of the owner storage as one raw element per item."""
        o = self.owner
        if o.bits % 8 == 0:
            return o.storage.copy()
        return unpack_bits(o.storage, o.bits, o.storage.size * 8 // o.bits)


def tile_plane(logical: np.ndarray, fill=0) -> np.ndarray:
    """Closed-form numpy tiling of [..., R, C] -> flat tiled storage (independent of
    the C scatter): pad to 16, split into tiles, order plane/tile-row/tile-col/r/c."""
    *lead, R, Cc = logical.shape
    PR, PC = padded(R), padded(Cc)
    buf = np.full(tuple(lead) + (PR, PC), fill, dtype=logical.dtype)
    buf[..., :R, :Cc] = logical
    nlead = len(lead)
    buf = buf.reshape(tuple(lead) + (PR // TILE, TILE, PC // TILE, TILE))
    axes = tuple(range(nlead)) + (nlead, nlead + 2, nlead + 1, nlead + 3)
    return np.ascontiguousarray(buf.transpose(axes)).reshape(-1)


def untile_plane(flat: np.ndarray, dims) -> np.ndarray:
    *lead, R, Cc = dims
    PR, PC = padded(R), padded(Cc)
    nlead = len(lead)
    buf = flat.reshape(tuple(lead) + (PR // TILE, PC // TILE, TILE, TILE))
    axes = tuple(range(nlead)) + (nlead, nlead + 2, nlead + 1, nlead + 3)
    buf = buf.transpose(axes).reshape(tuple(lead) + (PR, PC))
    return np.ascontiguousarray(buf[..., :R, :Cc])


# -- op wrappers -------------------------------------------------------------

def binary(op: int, lhs: HostView, rhs: HostView, out: HostView, ieee: bool = False) -> int:
    a, b, o = lhs.cview(), rhs.cview(), out.cview()
    return lib().iomo_binary(op, out.dtype, C.byref(a), C.byref(b), C.byref(o), int(ieee))


def rmsnorm(x: HostView, scale: HostView, out: HostView, eps: float) -> int:
    a, b, o = x.cview(), scale.cview(), out.cview()
    return lib().iomo_rmsnorm(out.dtype, C.byref(a), C.byref(b), C.byref(o), eps)


def silu(x: HostView, y: HostView) -> int:
    a, o = x.cview(), y.cview()
    return lib().iomo_silu(y.dtype, C.byref(a), C.byref(o))


def copy(src: HostView, dst: HostView) -> int:
    a, o = src.cview(), dst.cview()
    return lib().iomo_copy(dst.dtype, C.byref(a), C.byref(o))


def cache_append(src: HostView, dst: HostView, a: int) -> int:
    s, d = src.cview(), dst.cview()
    return lib().iomo_cache_append(dst.dtype, C.byref(s), C.byref(d), a)


def embedding(table: HostView, indices: HostView, out: HostView) -> int:
    t, i, o = table.cview(), indices.cview(), out.cview()
    return lib().iomo_embedding(out.dtype, indices.dtype, C.byref(t), C.byref(i), C.byref(o))


def rope(x: HostView, out: HostView, a: int, theta: float) -> int:
    s, o = x.cview(), out.cview()
    return lib().iomo_rope(out.dtype, C.byref(s), C.byref(o), a, theta)


def linear(x: HostView, w: HostView, out: HostView, s: int, R: int, head_planar: bool, H: int, D: int) -> int:
    a, b, o = x.cview(), w.cview(), out.cview()
    return lib().iomo_linear(out.dtype, C.byref(a), C.byref(b), C.byref(o), s, R, int(head_planar), H, D)


def sdpa(q: HostView, k: HostView, v: HostView, out: HostView, a: int, L: int) -> int:
    cq, ck, cv, co = q.cview(), k.cview(), v.cview(), out.cview()
    return lib().iomo_sdpa(out.dtype, C.byref(cq), C.byref(ck), C.byref(cv), C.byref(co), a, L)


def dense_layout(heads: int, rows: int, cols: int) -> StageLayout:
    l = StageLayout()
    l.plane_offset = 0
    l.plane_stride = heads * rows * cols
    l.head_stride = rows * cols
    l.row_stride = cols
    l.column_stride = 1
    l.rows = rows
    l.columns = cols
    return l


def softmax(scores: np.ndarray, a: int, L: int, scale: float = 1.0,
            rows: Optional[int] = None) -> np.ndarray:
    """scores: float32 [planes, heads, phys_rows, phys_cols] -> uint16 same shape."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    planes, heads, prow, pcol = scores.shape
    out = np.full(scores.shape, 0xAAAA, dtype=np.uint16)
    d = SoftmaxDesc()
    d.planes, d.heads, d.rows = planes, heads, prow if rows is None else rows
    d.a, d.L, d.scale = a, L, scale
    d.scores, d.p_bf16 = scores.ctypes.data, out.ctypes.data
    d.scores_layout = dense_layout(heads, prow, pcol)
    d.probability_layout = dense_layout(heads, prow, pcol)
    rc = lib().iomo_softmax(C.byref(d))
    assert rc == 0, rc
    return out


# -- bf16 helpers (numpy, independent of the C code) --------------------------

def f32_to_bf16_rne(x: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    r = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = 0x7FC0
    return r


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# --------------------------------------------------------------------------
# The compiled reference CPU backend (optional).
# --------------------------------------------------------------------------

REF_PATH = os.path.join(HERE, "_ref", "libiom_ref.so")


def ref_available() -> bool:
    return os.path.exists(REF_PATH)


def bind_iomc(l: C.CDLL) -> C.CDLL:
    """Declare the iomc_* handle API (iomc_shim.cpp) on a loaded library."""
    P = C.c_void_p
    U64P = C.POINTER(C.c_uint64)
    l.iomc_last_error.restype = C.c_char_p
    l.iomc_cpu_device_create.restype = P
    l.iomc_cpu_device_create.argtypes = [C.c_size_t]
    if hasattr(l, "iomc_mi355x_device_create"):
        l.iomc_mi355x_device_create.restype = P
        l.iomc_mi355x_device_create.argtypes = [C.c_uint32, C.c_size_t, C.c_size_t]
    l.iomc_device_destroy.argtypes = [P]
    l.iomc_device_backend_kind.argtypes = [P]
    l.iomc_device_supported_types.restype = C.c_uint32
    l.iomc_device_supported_types.argtypes = [P, C.POINTER(C.c_int), C.c_uint32]
    l.iomc_tensor_create.restype = P
    l.iomc_tensor_create.argtypes = [P, C.c_int, C.c_uint32, U64P]
    l.iomc_tensor_destroy.argtypes = [P]
    l.iomc_tensor_view.restype = P
    l.iomc_tensor_view.argtypes = [P]
    l.iomc_view_destroy.argtypes = [P]
    l.iomc_view_slice.restype = P
    l.iomc_view_slice.argtypes = [P, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t]
    l.iomc_view_select.restype = P
    l.iomc_view_select.argtypes = [P, C.c_size_t, C.c_size_t]
    l.iomc_view_permute.restype = P
    l.iomc_view_permute.argtypes = [P, U64P, C.c_size_t]
    l.iomc_view_reshape_leading.restype = P
    l.iomc_view_reshape_leading.argtypes = [P, U64P, C.c_size_t]
    l.iomc_view_rank.restype = C.c_uint32
    l.iomc_view_rank.argtypes = [P]
    l.iomc_view_describe.argtypes = [P, U64P, U64P, U64P]
    l.iomc_view_logical_nbytes.restype = C.c_uint64
    l.iomc_view_logical_nbytes.argtypes = [P]
    l.iomc_view_tiled_nbytes.restype = C.c_uint64
    l.iomc_view_tiled_nbytes.argtypes = [P]
    l.iomc_view_native_handle.restype = P
    l.iomc_view_native_handle.argtypes = [P]
    l.iomc_view_from_host.argtypes = [P, P, P, C.c_size_t]
    l.iomc_view_to_host.argtypes = [P, P, P, C.c_size_t]
    l.iomc_queue_create.restype = P
    l.iomc_queue_create.argtypes = [P]
    l.iomc_queue_destroy.argtypes = [P]
    l.iomc_binary.restype = C.c_int64
    l.iomc_binary.argtypes = [P, C.c_int, P, P, P]
    l.iomc_copy.restype = C.c_int64
    l.iomc_copy.argtypes = [P, P, P]
    l.iomc_rmsnorm.restype = C.c_int64
    l.iomc_rmsnorm.argtypes = [P, P, P, P, C.c_float]
    l.iomc_silu.restype = C.c_int64
    l.iomc_silu.argtypes = [P, P, P]
    if hasattr(l, "iomc_sdpa_case_count"):
        U16P, U8P = C.POINTER(C.c_uint16), C.POINTER(C.c_uint8)
        l.iomc_sdpa_case_info.argtypes = [C.c_int, U64P, C.c_char_p, C.c_size_t]
        l.iomc_sdpa_case_data.argtypes = [C.c_int, U16P, U16P, U16P]
        l.iomc_sdpa_case_expected.restype = C.c_int64
        l.iomc_sdpa_case_expected.argtypes = [C.c_int, U16P, U8P, C.c_size_t]
        l.iomc_sdpa_matches.argtypes = [C.c_uint16, C.c_uint16, C.c_uint8]
    l.iomc_sdpa.restype = C.c_int64
    l.iomc_sdpa.argtypes = [P, P, P, P, P, P, C.c_size_t, C.c_size_t]
    l.iomc_wait.argtypes = [P, C.c_int64]
    l.iomc_linear.restype = C.c_int64
    l.iomc_linear.argtypes = [P, P, P, P, C.c_size_t, C.c_size_t, C.c_int, C.c_size_t, C.c_size_t]
    l.iomc_cache_append.restype = C.c_int64
    l.iomc_cache_append.argtypes = [P, P, P, C.c_size_t]
    l.iomc_rope.restype = C.c_int64
    l.iomc_rope.argtypes = [P, P, P, C.c_size_t, C.c_double]
    l.iomc_embedding.restype = C.c_int64
    l.iomc_embedding.argtypes = [P, P, P, P, P, C.POINTER(C.c_int)]
    l.iomc_workspace_create.restype = P
    l.iomc_workspace_create.argtypes = [P, C.c_size_t]
    l.iomc_workspace_destroy.argtypes = [P]
    l.iomc_sdpa_workspace_bytes.restype = C.c_int64
    l.iomc_sdpa_workspace_bytes.argtypes = [P, P, P, P, P, C.c_size_t, C.c_size_t]
    l.iomc_sdpa_submit.restype = C.c_int64
    l.iomc_sdpa_submit.argtypes = [P, P, P, P, P, C.c_size_t, C.c_size_t, P]
    l.iomc_embedding_submit.restype = C.c_int64
    l.iomc_embedding_submit.argtypes = [P, P, P, P, P]
    l.iomc_embedding_workspace_bytes.restype = C.c_int64
    l.iomc_embedding_workspace_bytes.argtypes = [P, P, P, P]
    if hasattr(l, "iomc_inject_fault"):
        l.iomc_inject_fault.argtypes = [C.c_int]
        l.iomc_inject_fault.restype = None
        l.iomc_test_counter.restype = C.c_uint64
        l.iomc_test_counter.argtypes = [C.c_int]
        l.iomc_queue_snapshot.argtypes = [P, U64P]
        l.iomc_retained_leases.restype = C.c_int64
        l.iomc_retained_leases.argtypes = [P]
        l.iomc_reclaim_leases.argtypes = [P]
        l.iomc_reclaim_leases.restype = None
    return l


# numeric values of iom::rocm_detail::SubmissionFault (iom_amd/host/mi355x_testing.hpp)
(FAULT_NONE, FAULT_EVENT_CREATE, FAULT_QUEUE_EVENT_CREATE, FAULT_QUEUE_STREAM_CREATE,
 FAULT_KERNEL_LAUNCH, FAULT_EMBEDDING_STATUS_COPY, FAULT_EVENT_RECORD, FAULT_STREAM_SYNCHRONIZE,
 FAULT_SILU_LAUNCH, FAULT_SDPA_LAUNCH, FAULT_EVENT_RECORD_UNPROVED) = range(11)
(COUNT_EVENT_CREATE, COUNT_EVENT_DESTROY, COUNT_STREAM_CREATE, COUNT_STREAM_DESTROY,
 COUNT_DEVICE_ALLOC, COUNT_DEVICE_FREE, COUNT_LINEAR_NATIVE, COUNT_LINEAR_SCALAR, COUNT_SILU) = range(9)


class IomTensor:
    """One owner created through an iomc device, with view transforms."""

    def __init__(self, backend: "IomBackend", dtype: int, dims: Sequence[int]):
        self.b = backend
        self.dtype = dtype
        self.dims = tuple(int(d) for d in dims)
        arr = (C.c_uint64 * len(self.dims))(*self.dims)
        self.handle = backend.l.iomc_tensor_create(backend.dev, dtype, len(self.dims), arr)
        if not self.handle:
            raise RuntimeError(backend.error())
        self.full = IomView(self, backend.l.iomc_tensor_view(self.handle))

    def view(self) -> "IomView":
        return self.full

    def close(self):
        if self.handle:
            self.b.l.iomc_tensor_destroy(self.handle)
            self.handle = None


class IomView:
    def __init__(self, owner: IomTensor, handle):
        if not handle:
            raise RuntimeError(owner.b.error())
        self.owner = owner
        self.h = handle

    @property
    def l(self):
        return self.owner.b.l

    def slice(self, dim, first, count, step=1):
        return IomView(self.owner, self.l.iomc_view_slice(self.h, dim, first, count, step))

    def select(self, dim, index):
        return IomView(self.owner, self.l.iomc_view_select(self.h, dim, index))

    def permute(self, order):
        arr = (C.c_uint64 * len(order))(*order)
        return IomView(self.owner, self.l.iomc_view_permute(self.h, arr, len(order)))

    def reshape_leading(self, lead):
        arr = (C.c_uint64 * len(lead))(*lead)
        return IomView(self.owner, self.l.iomc_view_reshape_leading(self.h, arr, len(lead)))

    def describe(self):
        rank = self.l.iomc_view_rank(self.h)
        dims = (C.c_uint64 * 8)()
        strides = (C.c_uint64 * 6)()
        off = C.c_uint64()
        self.l.iomc_view_describe(self.h, dims, C.byref(off), strides)
        return tuple(dims[:rank]), off.value, tuple(strides[:rank - 2])

    def from_host(self, arr: np.ndarray):
        """One raw element per array item; packed to the host bit stream here."""
        arr = np.ascontiguousarray(arr, dtype=NP_OF[self.owner.dtype])
        stream = pack_bits(arr, LEAF_BITS[self.owner.dtype])
        rc = self.l.iomc_view_from_host(self.owner.b.dev, self.h, stream.ctypes.data, stream.nbytes)
        if rc != 0:
            raise RuntimeError(self.owner.b.error())

    def to_host_stream(self) -> np.ndarray:
        """The packed host bytes exactly as the backend wrote them."""
        dims, _, _ = self.describe()
        bits = LEAF_BITS[self.owner.dtype]
        stream = np.full(packed_nbytes(int(np.prod(dims, dtype=np.int64)), bits), 0xEE, np.uint8)
        rc = self.l.iomc_view_to_host(self.owner.b.dev, self.h, stream.ctypes.data, stream.nbytes)
        if rc != 0:
            raise RuntimeError(self.owner.b.error())
        return stream

    def to_host(self) -> np.ndarray:
        dims, _, _ = self.describe()
        count = int(np.prod(dims, dtype=np.int64))
        return unpack_bits(self.to_host_stream(), LEAF_BITS[self.owner.dtype], count).reshape(dims)

    def raw_storage(self) -> np.ndarray:
        """Copy of the owner's raw tiled bytes (host-memory backends only)."""
        n = self.l.iomc_view_tiled_nbytes(self.owner.full.h)
        p = self.l.iomc_view_native_handle(self.h)
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(n,)).copy()


class IomBackend:
    """A device + one queue behind the iomc_* handle API."""

    def __init__(self, l: C.CDLL, dev):
        if not dev:
            raise RuntimeError(l.iomc_last_error().decode())
        self.l = l
        self.dev = dev
        self.queue = l.iomc_queue_create(dev)
        if not self.queue:
            raise RuntimeError(self.error())

    def error(self) -> str:
        return self.l.iomc_last_error().decode()

    def tensor(self, dtype, dims) -> IomTensor:
        return IomTensor(self, dtype, dims)

    def supported_types(self):
        codes = (C.c_int * 64)()
        n = self.l.iomc_device_supported_types(self.dev, codes, 64)
        return list(codes[:n])

    def second_queue(self) -> "IomBackend":
        """Another queue of the same device (shares the device handle; close() it first)."""
        other = object.__new__(IomBackend)
        other.l, other.dev = self.l, self.dev
        other.queue = self.l.iomc_queue_create(self.dev)
        if not other.queue:
            raise RuntimeError(self.error())
        other.borrowed = True
        return other

    def wait(self, token: int) -> int:
        return self.l.iomc_wait(self.queue, token)

    def run(self, token: int) -> int:
        """Wait when accepted; return the oid (negative = synchronous error)."""
        if token > 0:
            rc = self.wait(token)
            if rc != 0:
                raise RuntimeError(self.error())
        return token

    def binary(self, op, lhs: IomView, rhs: IomView, out: IomView) -> int:
        return self.run(self.l.iomc_binary(self.queue, op, lhs.h, rhs.h, out.h))

    def copy(self, src: IomView, dst: IomView) -> int:
        return self.run(self.l.iomc_copy(self.queue, src.h, dst.h))

    def rmsnorm(self, x, scale, out, eps) -> int:
        return self.run(self.l.iomc_rmsnorm(self.queue, x.h, scale.h, out.h, eps))

    def silu(self, x, y) -> int:
        return self.run(self.l.iomc_silu(self.queue, x.h, y.h))

    def linear(self, x, w, out, s, R, head_planar, H, D) -> int:
        return self.run(self.l.iomc_linear(self.queue, x.h, w.h, out.h, s, R, int(head_planar), H, D))

    def cache_append(self, src, dst, a) -> int:
        return self.run(self.l.iomc_cache_append(self.queue, src.h, dst.h, a))

    def rope(self, x, out, a, theta) -> int:
        return self.run(self.l.iomc_rope(self.queue, x.h, out.h, a, theta))

    def embedding(self, table, indices, out):
        """(token or negative oid, wait status: 0 or the retained failure's class)."""
        status = C.c_int(0)
        token = self.l.iomc_embedding(self.dev, self.queue, table.h, indices.h, out.h, C.byref(status))
        return token, status.value

    def sdpa(self, q, k, v, out, a, L) -> int:
        return self.run(self.l.iomc_sdpa(self.dev, self.queue, q.h, k.h, v.h, out.h, a, L))

    # ---- submissions that do not wait (the caller waits, and owns any workspace) --------

    def submit(self, name: str, *args) -> int:
        """The oid of iomc_<name>(queue, ...) without waiting for it."""
        return getattr(self.l, "iomc_" + name)(self.queue, *[getattr(a, "h", a) for a in args])

    def workspace(self, nbytes: int):
        h = self.l.iomc_workspace_create(self.dev, nbytes)
        if not h:
            raise RuntimeError(self.error())
        return h

    def drop_workspace(self, handle):
        self.l.iomc_workspace_destroy(handle)

    def sdpa_workspace_bytes(self, q, k, v, out, a, L) -> int:
        return self.l.iomc_sdpa_workspace_bytes(self.queue, q.h, k.h, v.h, out.h, a, L)

    def sdpa_submit(self, q, k, v, out, a, L, workspace=None) -> int:
        return self.l.iomc_sdpa_submit(self.queue, q.h, k.h, v.h, out.h, a, L, workspace)

    def embedding_workspace_bytes(self, table, indices, out) -> int:
        return self.l.iomc_embedding_workspace_bytes(self.queue, table.h, indices.h, out.h)

    def embedding_submit(self, table, indices, out, workspace=None) -> int:
        return self.l.iomc_embedding_submit(self.queue, table.h, indices.h, out.h, workspace)

    # ---- the MI355X backend's test seams ------------------------------------------------

    def inject(self, fault: int):
        self.l.iomc_inject_fault(fault)

    def counter(self, which: int) -> int:
        return int(self.l.iomc_test_counter(which))

    def snapshot(self):
        """(events_total, events_in_use, operations_in_flight) of this queue."""
        out = (C.c_uint64 * 3)()
        rc = self.l.iomc_queue_snapshot(self.queue, out)
        if rc != 0:
            raise RuntimeError(self.error())
        return tuple(int(v) for v in out)

    def retained_leases(self) -> int:
        return int(self.l.iomc_retained_leases(self.dev))

    def reclaim_leases(self):
        self.l.iomc_reclaim_leases(self.dev)

    def close_queue(self):
        if self.queue:
            self.l.iomc_queue_destroy(self.queue)
            self.queue = None

    def close(self):
        if self.queue:
            self.l.iomc_queue_destroy(self.queue)
            self.queue = None
        if getattr(self, "borrowed", False):
            self.dev = None
        if self.dev:
            self.l.iomc_device_destroy(self.dev)
            self.dev = None


_ref_lib: Optional[C.CDLL] = None


def ref_backend(max_in_flight: int = 16) -> IomBackend:
    """The reference's own CPU backend (make_cpu_device)."""
    global _ref_lib
    if _ref_lib is None:
        _ref_lib = bind_iomc(_load(REF_PATH))
    return IomBackend(_ref_lib, _ref_lib.iomc_cpu_device_create(max_in_flight))


REF512_PATH = os.path.join(HERE, "_ref", "libiom_ref_avx512.so")
_ref512_lib: Optional[C.CDLL] = None


def ref512_available() -> bool:
    """The reference's opt-in AVX-512 BF16 CPU build (make ref512) and a CPU that has the ISA."""
    if not os.path.exists(REF512_PATH):
        return False
    try:
        with open("/proc/cpuinfo") as f:
            return "avx512_bf16" in f.read()
    except OSError:
        return False


def ref_backend_avx512(max_in_flight: int = 16) -> IomBackend:
    """The reference CPU backend built with AVX_512_BF16_ENABLED (a timing baseline only)."""
    global _ref512_lib
    if _ref512_lib is None:
        _ref512_lib = bind_iomc(_load(REF512_PATH))
    return IomBackend(_ref512_lib, _ref512_lib.iomc_cpu_device_create(max_in_flight))


MI355X_SHIM_PATH = os.path.join(HERE, "_ref", "libiom_mi355x_shim.so")
_mi355x_lib: Optional[C.CDLL] = None


def mi355x_available() -> bool:
    return os.path.exists(MI355X_SHIM_PATH)


def mi355x_lib() -> C.CDLL:
    """The handle API over this repository's C++ backend (iom::make_rocm_device) and,
    in the same process and over the same libiom core, the reference CPU backend."""
    global _mi355x_lib
    if _mi355x_lib is None:
        _mi355x_lib = bind_iomc(_load(MI355X_SHIM_PATH))
    return _mi355x_lib


def mi355x_backend(arena_bytes: int = 1 << 30, max_in_flight: int = 16, ordinal: int = 0) -> IomBackend:
    l = mi355x_lib()
    return IomBackend(l, l.iomc_mi355x_device_create(ordinal, arena_bytes, max_in_flight))


def cpu_backend_beside_mi355x(max_in_flight: int = 16) -> IomBackend:
    l = mi355x_lib()
    return IomBackend(l, l.iomc_cpu_device_create(max_in_flight))
