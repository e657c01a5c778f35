"""Host-only checks of the C ABI: the library loads, exports every symbol the
header declares, sizes temp storage sensibly and rejects bad arguments with
the documented status before touching the GPU.  No compute calls."""
import ctypes
import os
import re

import numpy as np
import pytest

from ilgpu_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ilgpu_hip_algorithms.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ilgpu_hip_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = capi.lib()
    names = declared_functions()
    assert len(names) >= 11
    for name in names:
        assert hasattr(L, name), name
    assert sorted(capi.EXPORTS) == names


def test_binding_constants_are_the_headers():
    # every enumerator of the header has the same value under the same name
    # (without the ILGPU_HIP_ prefix) in the ctypes binding
    header = open(HEADER).read()
    enumerators = re.findall(r"\b(ILGPU_HIP_[A-Z0-9_]+)\s*=\s*(-?\d+)", header)
    assert len(enumerators) >= 39
    for name, value in enumerators:
        short = name[len("ILGPU_HIP_"):]
        assert hasattr(capi, short), name
        assert getattr(capi, short) == int(value), name


def test_version_and_status_strings():
    assert capi.lib().ilgpu_hip_version() == 100
    for status in range(6):
        assert capi.status_string(status) != "unknown status"
    assert capi.status_string(99) == "unknown status"


def test_temp_size_queries():
    n = 1 << 20
    keys_only = capi.radix_sort_temp_bytes(n, np.uint32)
    assert keys_only >= n * 4
    with_values = capi.radix_sort_temp_bytes(n, np.uint32, 4)
    assert with_values >= n * 8  # alternate buffers for keys and values
    # 2^27 pairs of (u64, u32): the size the reference's own helper overflows
    # on (RadixSortExtensions.cs:400-402) is computed in 64 bits here.
    big = capi.radix_sort_temp_bytes(1 << 27, np.uint64, 4)
    assert big > (1 << 27) * 12
    assert capi.scan_temp_bytes(n, np.int32) < n  # a few bytes per tile
    assert capi.scan_temp_bytes(n, np.float64) < n
    assert capi.reduce_temp_bytes(n, np.float32) <= 64 * 1024
    assert capi.reduce_temp_bytes(1, np.float32) == capi.reduce_temp_bytes(n, np.float32)


def test_temp_size_query_errors():
    with pytest.raises(capi.ArgumentOutOfRangeError):
        capi.radix_sort_temp_bytes(0, np.uint32)
    with pytest.raises(capi.NotSupportedError):
        capi.radix_sort_temp_bytes(16, np.uint32, 3)
    with pytest.raises(capi.NotSupportedError):
        capi.scan_temp_bytes(16, np.int16)  # not a scan/reduce type
    with pytest.raises(capi.NotSupportedError):
        capi.scan_temp_bytes(1 << 31, np.int32)  # NotSupportedArrayView64
    out = ctypes.c_int64()
    assert capi.lib().ilgpu_hip_radix_sort_temp_bytes(
        16, 99, 0, ctypes.byref(out)) == capi.ERROR_NOT_SUPPORTED


FAKE = 0x10000  # a non-null, 16-byte aligned "device pointer" that is never dereferenced


def test_sort_argument_validation():
    L = capi.lib()
    big = 1 << 40
    # invalid (null / empty) views -> ArgumentNullException
    assert L.ilgpu_hip_radix_sort_keys(None, None, 16, 1, capi.U32, 0, FAKE, big) == capi.ERROR_NULL_VIEW
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 0, 1, capi.U32, 0, FAKE, big) == capi.ERROR_NULL_VIEW
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, 1, capi.U32, 0, None, big) == capi.ERROR_NULL_VIEW
    # temp too small -> ArgumentOutOfRangeException (TempViewManager.cs:88-89)
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, 1, capi.U32, 0, FAKE, 8) == capi.ERROR_OUT_OF_RANGE
    # temp not int-aligned -> InvalidOperationException
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, 1, capi.U32, 0, FAKE + 2, big) == capi.ERROR_UNALIGNED_TEMP
    # 64-bit lengths, unknown types/flags -> NotSupportedException
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 1 << 31, 1, capi.U32, 0, FAKE, big) == capi.ERROR_NOT_SUPPORTED
    # strides below one; a strided view with the dense temp size (too small)
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, 0, capi.U32, 0, FAKE, big) == capi.ERROR_OUT_OF_RANGE
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, -2, capi.U32, 0, FAKE, big) == capi.ERROR_OUT_OF_RANGE
    dense = capi.radix_sort_temp_bytes(16, np.uint32)
    assert capi.radix_sort_temp_bytes(16, np.uint32, 0, 3) >= dense + 16 * 4
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, 3, capi.U32, 0, FAKE, dense) == capi.ERROR_OUT_OF_RANGE
    assert L.ilgpu_hip_radix_sort_pairs(None, FAKE, 1, FAKE, 0, 16, capi.U32, 4, 0, 0, FAKE, big) == capi.ERROR_OUT_OF_RANGE
    assert (capi.radix_sort_temp_bytes(16, np.uint32, 8, 1, 5)
            >= capi.radix_sort_temp_bytes(16, np.uint32, 8) + 16 * 8)
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, 1, 42, 0, FAKE, big) == capi.ERROR_NOT_SUPPORTED
    assert L.ilgpu_hip_radix_sort_keys(None, FAKE, 16, 1, capi.U32, 8, FAKE, big) == capi.ERROR_NOT_SUPPORTED
    # pairs
    assert L.ilgpu_hip_radix_sort_pairs(None, FAKE, 1, None, 1, 16, capi.U32, 4, 0, 0, FAKE, big) == capi.ERROR_NULL_VIEW
    assert L.ilgpu_hip_radix_sort_pairs(None, FAKE, 1, FAKE, 1, 16, capi.U32, 3, 0, 0, FAKE, big) == capi.ERROR_NOT_SUPPORTED
    assert L.ilgpu_hip_radix_sort_pairs(None, FAKE, 1, FAKE, 1, 16, capi.U32, 16, 0, capi.VALUES_FROM_INDEX, FAKE, big) == capi.ERROR_NOT_SUPPORTED
    assert L.ilgpu_hip_radix_sort_pairs(None, FAKE, 1, FAKE, 1, 16, capi.U32, 1, 0, capi.VALUES_FROM_INDEX_AS_FLOAT, FAKE, big) == capi.ERROR_NOT_SUPPORTED
    assert L.ilgpu_hip_radix_sort_pairs(None, FAKE, 1, FAKE, 1, 16, capi.U32, 4, 0, 3, FAKE, big) == capi.ERROR_NOT_SUPPORTED
    assert L.ilgpu_hip_radix_sort_pairs(None, FAKE, 1, FAKE, 1, 16, capi.U32, 4, 0, 0, FAKE, 64) == capi.ERROR_OUT_OF_RANGE


def test_scan_argument_validation():
    L = capi.lib()
    big = 1 << 40
    args = dict(t=capi.I32, op=capi.OP_ADD, kind=capi.SCAN_INCLUSIVE)

    def call(inp=FAKE, n_in=16, s_in=1, out=FAKE, n_out=16, s_out=1, t=args["t"],
             op=args["op"], kind=args["kind"], temp=FAKE, tb=big):
        return L.ilgpu_hip_scan(None, inp, n_in, s_in, out, n_out, s_out, t, op,
                                kind, temp, tb)

    assert call(inp=None) == capi.ERROR_NULL_VIEW
    assert call(out=None) == capi.ERROR_NULL_VIEW
    assert call(n_in=0) == capi.ERROR_NULL_VIEW
    assert call(n_out=8) == capi.ERROR_OUT_OF_RANGE        # ScanExtensions.cs:679-680
    assert call(n_in=1 << 31, n_out=1 << 31) == capi.ERROR_NOT_SUPPORTED
    assert call(s_in=0) == capi.ERROR_OUT_OF_RANGE
    assert call(s_out=-1) == capi.ERROR_OUT_OF_RANGE
    assert call(t=capi.U8) == capi.ERROR_NOT_SUPPORTED
    assert call(op=7) == capi.ERROR_NOT_SUPPORTED
    assert call(kind=5) == capi.ERROR_NOT_SUPPORTED
    assert call(temp=None) == capi.ERROR_NULL_VIEW
    assert call(tb=4) == capi.ERROR_OUT_OF_RANGE


def test_reduce_argument_validation():
    L = capi.lib()
    big = 1 << 20

    def call(inp=FAKE, n=16, stride=1, t=capi.F32, op=capi.OP_ADD, out=FAKE,
             n_out=1, temp=FAKE, tb=big):
        return L.ilgpu_hip_reduce(None, inp, n, stride, t, op, out, n_out, temp, tb)

    assert call(inp=None) == capi.ERROR_NULL_VIEW
    assert call(n=0) == capi.ERROR_NULL_VIEW
    assert call(out=None) == capi.ERROR_NULL_VIEW
    assert call(n_out=0) == capi.ERROR_NULL_VIEW
    assert call(n=1 << 31) == capi.ERROR_NOT_SUPPORTED
    assert call(t=capi.I16) == capi.ERROR_NOT_SUPPORTED
    assert call(stride=0) == capi.ERROR_OUT_OF_RANGE
    assert call(tb=16) == capi.ERROR_OUT_OF_RANGE


def test_histogram_argument_validation():
    L = capi.lib()

    def call(inp=FAKE, n=16, stride=1, t=capi.U8, bins=FAKE, nb=256,
             bt=capi.I32, loc=capi.LOCATOR_IDENTITY, ov=FAKE):
        return L.ilgpu_hip_histogram(None, inp, n, stride, t, bins, nb, bt, loc, ov)

    assert call(inp=None) == capi.ERROR_NULL_VIEW
    assert call(n=0) == capi.ERROR_NULL_VIEW
    assert call(bins=None) == capi.ERROR_NULL_VIEW
    assert call(nb=0) == capi.ERROR_NULL_VIEW
    assert call(n=1 << 31) == capi.ERROR_NOT_SUPPORTED
    assert call(t=capi.F16) == capi.ERROR_NOT_SUPPORTED
    # bins: the six AtomicNumericTypes; Half, 8- and 16-bit bins do not exist
    assert call(bt=capi.F16) == capi.ERROR_NOT_SUPPORTED
    assert call(bt=capi.U16) == capi.ERROR_NOT_SUPPORTED
    assert call(loc=9) == capi.ERROR_NOT_SUPPORTED
    assert call(stride=0) == capi.ERROR_OUT_OF_RANGE


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", "/nonexistent/libilgpu_hip_algorithms.so")
    with pytest.raises(FileNotFoundError):
        capi.lib()


def test_transform_argument_validation():
    L = capi.lib()

    def call(src=FAKE, n=16, s_in=1, st=capi.I32, dst=FAKE, n_out=16, s_out=1, tt=capi.I64,
             op=capi.TRANSFORM_CONVERT):
        return L.ilgpu_hip_transform(None, src, n, s_in, st, dst, n_out, s_out, tt, op, 0)

    assert call(src=None) == capi.ERROR_NULL_VIEW          # TransformExtensions.cs:304-305
    assert call(dst=None) == capi.ERROR_NULL_VIEW          # :308-309
    assert call(n_out=8) == capi.ERROR_OUT_OF_RANGE        # :310-317
    assert call(s_in=0) == capi.ERROR_OUT_OF_RANGE
    assert call(s_out=-1) == capi.ERROR_OUT_OF_RANGE
    assert call(st=99) == capi.ERROR_NOT_SUPPORTED
    assert call(op=7) == capi.ERROR_NOT_SUPPORTED
    assert call(st=capi.F32, tt=capi.I32) == capi.ERROR_NOT_SUPPORTED
    assert call(st=capi.F64, tt=capi.F64, op=capi.TRANSFORM_BIT_COMPLEMENT) == capi.ERROR_NOT_SUPPORTED

    def rcall(src=FAKE, n=16, dst=FAKE, n_out=16, order=FAKE, n_order=16, st=capi.U32, tt=capi.U32):
        return L.ilgpu_hip_reorder_transform(None, src, n, st, dst, n_out, tt, order, n_order,
                                             capi.TRANSFORM_MULTIPLY, 2)

    assert rcall(src=None) == capi.ERROR_NULL_VIEW         # ReorderExtensions.cs:158-159
    assert rcall(order=None) == capi.ERROR_NULL_VIEW       # :162-163
    assert rcall(n_order=8) == capi.ERROR_OUT_OF_RANGE     # :164-165
    assert rcall(n_out=8) == capi.ERROR_OUT_OF_RANGE
    assert rcall(n=(1 << 31), n_order=(1 << 31), n_out=(1 << 31)) == capi.ERROR_NOT_SUPPORTED  # :166-170
    assert rcall(st=capi.F16, tt=capi.U8) == capi.ERROR_NOT_SUPPORTED


def test_no_sort_runs_on_a_device_that_failed_the_lds_atomic_check():
    # Every sort asks first whether the device serves the lanes of an LDS atomic
    # in lane order (the ranking of a pass rests on it) and keeps the answer per
    # device.  The test hook stands in for a device that fails: both sort entry
    # points and the query itself answer NOT_SUPPORTED before anything is
    # launched, so this needs no GPU and the pointers are never touched.
    L = capi.lib()
    n = 1000
    keys, values, temp = (ctypes.c_void_p(0x10000), ctypes.c_void_p(0x20000),
                          ctypes.c_void_p(0x40000))
    temp_bytes = capi.radix_sort_temp_bytes(n, np.uint32, 4)

    def sort_keys():
        return L.ilgpu_hip_radix_sort_keys(None, keys, n, 1, capi.U32, 0, temp, temp_bytes)

    def sort_pairs():
        return L.ilgpu_hip_radix_sort_pairs(None, keys, 1, values, 1, n, capi.U32, 4, 0,
                                            capi.VALUES_FROM_VIEW, temp, temp_bytes)

    capi.sort_set_parameter(capi.SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER, 0)
    try:
        assert L.ilgpu_hip_sort_check_device(None) == capi.ERROR_NOT_SUPPORTED
        assert sort_keys() == capi.ERROR_NOT_SUPPORTED
        assert sort_pairs() == capi.ERROR_NOT_SUPPORTED
        with pytest.raises(capi.NotSupportedError):
            capi.check(L.ilgpu_hip_sort_check_device(None))
        # argument checks still come first
        assert L.ilgpu_hip_radix_sort_keys(None, None, n, 1, capi.U32, 0, temp,
                                           temp_bytes) == capi.ERROR_NULL_VIEW
        # a device that is taken to have passed is not asked either
        capi.sort_set_parameter(capi.SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER, 1)
        assert L.ilgpu_hip_sort_check_device(None) == capi.SUCCESS
    finally:
        capi.sort_set_parameter(capi.SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER, -1)
