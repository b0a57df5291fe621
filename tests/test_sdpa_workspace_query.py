"""The pure workspace query of attention (iomx_sdpa_workspace = sdpa_workspace_requirements):
host arithmetic only, no GPU.  The sizes are fixed here by their closed forms: 4 bytes of flags
per (plane, KV head, pack share) rounded up to 256, plus 2 KiB per (plane, KV head, 32 tokens of
the prefix, 16 features) for the packed V fragments and the flushed K tiles; nothing for a decode
step ((Hq/Hkv) * R <= 16) or heads wider than 128 -- except a decode step of few sequences
against a long prefix, whose shares leave 32 + 4 D bytes per plane, KV head, share and tile row."""
import ctypes as C

import pytest

from iom_amd import iomx

DT_BF16 = iomx.DT_BF16


def dense_view(dims, slot=0):
    """A whole dense tensor at a made-up address (the query never touches memory)."""
    v = iomx.View()
    v.base = 0x7F0000000000 + slot * (1 << 36)
    v.rank = len(dims)
    for i, d in enumerate(dims):
        v.dims[i] = d
    v.plane_offset = 0
    stride = 1
    for i in range(len(dims) - 3, -1, -1):
        v.plane_strides[i] = stride
        stride *= dims[i]
    return v


def query(lead, Hq, Hkv, R, D, C_, a, L, dtype=DT_BF16):
    q, k = dense_view(lead + (Hq, R, D), 0), dense_view(lead + (Hkv, C_, D), 1)
    v, o = dense_view(lead + (Hkv, C_, D), 2), dense_view(lead + (R, Hq * D), 3)
    nbytes, align = C.c_uint64(123), C.c_uint64(456)
    rc = iomx.lib().iomx_sdpa_workspace(dtype, C.byref(q), C.byref(k), C.byref(v), C.byref(o), a, L,
                                        C.byref(nbytes), C.byref(align))
    return rc, nbytes.value, align.value


def tiled(planes, Hkv, L, D, splits):
    flags = (4 * planes * Hkv * splits + 255) // 256 * 256
    return flags + 2048 * planes * Hkv * ((L + 31) // 32) * ((D + 15) // 16)


@pytest.mark.parametrize("lead,Hq,Hkv,R,D,C_,a,L,want", [
    ((), 32, 4, 1, 64, 512, 511, 512, (0, 1)),                  # decode, short prefix
    ((64,), 32, 4, 1, 64, 2048, 2047, 2048, (0, 1)),            # decode, many sequences
    ((), 32, 4, 2, 64, 600, 100, 102, (0, 1)),                  # two rows x grouping 8 = one tile
    ((), 4, 4, 40, 256, 64, 0, 40, (0, 1)),                     # heads wider than 128: reference order
    ((), 32, 4, 1, 64, 4096, 4095, 4096, ((4 * 8 * 16 * (8 + 64)) * 4, 256)),       # 128 groups, 8 shares
    ((2,), 32, 8, 1, 128, 16384, 16383, 16384, ((16 * 16 * 16 * (8 + 128)) * 4, 256)),  # 512 groups, 16 shares
    ((), 32, 4, 1, 64, 2048, 2015, 2016, (0, 1)),               # 63 groups: below the threshold
])
def test_decode_and_wide_heads(lead, Hq, Hkv, R, D, C_, a, L, want):
    assert query(lead, Hq, Hkv, R, D, C_, a, L) == (0,) + want


def test_prefill_sizes_follow_the_closed_form():
    rc, nbytes, align = query((8,), 32, 4, 512, 64, 512, 0, 512)
    assert rc == 0 and align == 256
    frags = 16 * 4                                   # 32-token groups x 16-feature tiles
    splits = min((4096 + 31) // 32, (frags + 3) // 4, 64)
    assert nbytes == tiled(8, 4, 512, 64, splits)
    rc, nbytes, align = query((), 8, 2, 24, 40, 100, 3, 27)
    assert rc == 0 and align == 256
    frags = 1 * 3
    splits = min(4096 // 2, (frags + 3) // 4, 64)
    assert nbytes == tiled(1, 2, 27, 40, splits)


def test_rejections_need_no_gpu_either():
    assert query((), 32, 4, 1, 64, 512, 511, 512, dtype=iomx.DT_F32)[0] != 0      # BF16 only
    assert query((), 6, 4, 1, 64, 512, 511, 512)[0] != 0                         # Hq not a multiple of Hkv
    assert query((), 8, 2, 4, 64, 16, 0, 17)[0] != 0                             # L beyond the cache
