"""The buffer and device entry points a ggml backend's buffer vtable binds (alloc/free, memset_tensor and clear,
set_tensor, get_tensor, cpy_tensor; member order pinned by src/core/gguf_loader.cpp:332-344), called through
the C ABI the way the glue calls them."""
import ctypes

import numpy as np
import pytest

import crispasr_amd as ca

pytestmark = pytest.mark.gpu

K = ca.ggml


def _alloc(n):
    p = ctypes.c_void_p()
    assert K.lib().mi355x_buffer_alloc(n, ctypes.byref(p)) == K.OK
    return p.value


def _get(ptr, n):
    host = np.empty(n, np.uint8)
    assert K.lib().mi355x_buffer_get(host.ctypes.data, ptr, n, None) == K.OK
    return host


def test_alloc_is_256_byte_aligned_and_zero_size_is_valid():
    ptrs = [_alloc(n) for n in (0, 1, 100, 1 << 20)]
    assert all(p and p % 256 == 0 for p in ptrs)
    for p in ptrs:
        assert K.lib().mi355x_buffer_free(p) == K.OK
    assert K.lib().mi355x_buffer_free(None) == K.OK


def test_set_get_round_trip_and_device_copy():
    n = 1 << 20
    data = np.random.default_rng(3).integers(0, 256, n, dtype=np.uint8)
    a, b = _alloc(n), _alloc(n)
    assert K.lib().mi355x_buffer_set(a, data.ctypes.data, n, None) == K.OK
    assert np.array_equal(_get(a, n), data)
    # the beam snapshot copy (src/core/attention.h:260-314) is a device-to-device copy of a cache slice
    off, m = 4096 + 34, 300000
    assert K.lib().mi355x_buffer_memset(b, 0, n, None) == K.OK
    assert K.lib().mi355x_buffer_copy(b + off, a + off, m, None) == K.OK
    assert K.lib().mi355x_stream_synchronize(None) == K.OK
    want = np.zeros(n, np.uint8)
    want[off:off + m] = data[off:off + m]
    assert np.array_equal(_get(b, n), want)
    for p in (a, b):
        K.lib().mi355x_buffer_free(p)


def test_set_get_copy_on_a_pinned_host_buffer():
    # the is_host buffer type goes through the same vtable entries
    n = 100000
    data = np.random.default_rng(4).integers(0, 256, n, dtype=np.uint8)
    h = ca.HostBuffer(n)
    d = _alloc(n)
    assert K.lib().mi355x_buffer_set(h.ptr, data.ctypes.data, n, None) == K.OK
    assert np.array_equal(h.array, data)                                   # the CPU sees it in place
    assert np.array_equal(_get(h.ptr, n), data)
    assert K.lib().mi355x_buffer_copy(d, h.ptr, n, None) == K.OK           # host buffer -> HBM (a split-boundary copy)
    assert K.lib().mi355x_stream_synchronize(None) == K.OK
    assert np.array_equal(_get(d, n), data)
    assert K.lib().mi355x_buffer_memset(h.ptr + 5, 0x77, 1001, None) == K.OK
    assert K.lib().mi355x_buffer_copy(h.ptr + 50000, d, 100, None) == K.OK  # and back
    assert K.lib().mi355x_stream_synchronize(None) == K.OK
    want = data.copy()
    want[5:1006] = 0x77
    want[50000:50100] = data[:100]
    assert np.array_equal(h.array, want)
    K.lib().mi355x_buffer_free(d)


@pytest.mark.parametrize("off,size", [(0, 0), (0, 1), (3, 5), (1, 15), (15, 2), (16, 16), (7, 4096), (0, 1 << 20), (34, 999999)])
def test_memset_any_alignment_and_size(off, size):
    n = (1 << 20) + 256
    buf = _alloc(n)
    base = np.full(n, 0x5A, np.uint8)
    assert K.lib().mi355x_buffer_set(buf, base.ctypes.data, n, None) == K.OK
    print("memset", off, size, flush=True)
    assert K.lib().mi355x_buffer_memset(buf + off, 0x1C3, size, None) == K.OK      # the value's low byte counts, as in memset
    assert K.lib().mi355x_stream_synchronize(None) == K.OK
    base[off:off + size] = 0xC3
    assert np.array_equal(_get(buf, n), base)
    K.lib().mi355x_buffer_free(buf)


def test_null_arguments_are_refused():
    assert K.lib().mi355x_buffer_alloc(16, None) == K.ERR_INVALID
    assert K.lib().mi355x_buffer_memset(None, 0, 16, None) == K.ERR_INVALID
    assert K.lib().mi355x_buffer_set(None, None, 16, None) == K.ERR_INVALID
    assert K.lib().mi355x_buffer_get(None, None, 16, None) == K.ERR_INVALID
    assert K.lib().mi355x_buffer_copy(None, None, 16, None) == K.ERR_INVALID
    assert K.lib().mi355x_buffer_copy(None, None, 0, None) == K.OK


def test_device_queries():
    assert ca.ggml.device_count() >= 1
    info = ca.ggml.device_info(0)
    assert info["arch"].startswith("gfx950") and info["compute_units"] > 0 and info["wavefront_size"] == 64
    assert info["total_memory"] >= info["free_memory"] > 0
    assert K.lib().mi355x_set_device(0) == K.OK
    assert K.lib().mi355x_set_device(ca.ggml.device_count() + 7) == K.ERR_HIP
    assert b"" != K.lib().mi355x_last_error()
    assert K.lib().mi355x_set_device(0) == K.OK
    # a refused call leaves nothing behind: the next launch reports its own status
    buf = _alloc(64)
    assert K.lib().mi355x_buffer_memset(buf, 1, 64, None) == K.OK
    assert K.lib().mi355x_stream_synchronize(None) == K.OK
    K.lib().mi355x_buffer_free(buf)
