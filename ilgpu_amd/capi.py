"""ctypes binding of ``libilgpu_hip_algorithms.so`` (the C ABI declared in
``include/ilgpu_hip_algorithms.h``).

Device memory and streams come from torch (plumbing only): a ``DeviceArray``
is a raw byte tensor on ``cuda:0`` plus the numpy dtype of its elements, so
every ILGPU element type, including the unsigned ones torch has no arithmetic
for, can be passed by pointer.

Loading fails loudly when the shared library has not been built; there is no
fallback implementation.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ILGPU_HIP_ALGORITHMS_LIB selects another build of the same library (e.g. one
# compiled with different tuning constants); it must export the same C ABI.
LIB_PATH = os.environ.get(
    "ILGPU_HIP_ALGORITHMS_LIB",
    os.path.join(_HERE, "lib", "libilgpu_hip_algorithms.so"))

# ilgpu_hip_status
SUCCESS, ERROR_NULL_VIEW, ERROR_OUT_OF_RANGE, ERROR_NOT_SUPPORTED, \
    ERROR_UNALIGNED_TEMP, ERROR_RUNTIME, ERROR_STATIC_LIMIT = range(7)
SCAN_STATIC_MAX_BYTES = 1 << 30
# ilgpu_hip_type
I8, I16, I32, I64, U8, U16, U32, U64, F16, F32, F64 = range(11)
# ilgpu_hip_op / scan kind / flags / value source / locator
OP_ADD, OP_MAX, OP_MIN = 0, 1, 2
SCAN_INCLUSIVE, SCAN_EXCLUSIVE = 0, 1
SORT_DESCENDING, SORT_FLOAT_TOTAL_ORDER = 1, 2
VALUES_FROM_VIEW, VALUES_FROM_INDEX, VALUES_FROM_INDEX_AS_FLOAT = 0, 1, 2
LOCATOR_IDENTITY, LOCATOR_MODULO = 0, 1
(TRANSFORM_CONVERT, TRANSFORM_NEGATE, TRANSFORM_BIT_COMPLEMENT,
 TRANSFORM_MULTIPLY) = 0, 1, 2, 3

EXPORTS = [
    "ilgpu_hip_version", "ilgpu_hip_status_string",
    "ilgpu_hip_last_runtime_error", "ilgpu_hip_profile_enable",
    "ilgpu_hip_profile_query", "ilgpu_hip_radix_sort_temp_bytes",
    "ilgpu_hip_radix_sort_temp_bytes_strided",
    "ilgpu_hip_radix_sort_keys", "ilgpu_hip_radix_sort_pairs",
    "ilgpu_hip_radix_sort_passes",
    "ilgpu_hip_selftest_lds_atomic_order", "ilgpu_hip_sort_check_device",
    "ilgpu_hip_sort_set_parameter",
    "ilgpu_hip_scan_temp_bytes", "ilgpu_hip_scan", "ilgpu_hip_scan_static",
    "ilgpu_hip_reduce_temp_bytes", "ilgpu_hip_reduce", "ilgpu_hip_histogram",
    "ilgpu_hip_unique_temp_bytes", "ilgpu_hip_unique", "ilgpu_hip_initialize",
    "ilgpu_hip_sequence", "ilgpu_hip_reorder",
    "ilgpu_hip_transform", "ilgpu_hip_reorder_transform",
]

_NP_TO_TYPE = {
    np.dtype(np.int8): I8, np.dtype(np.int16): I16, np.dtype(np.int32): I32,
    np.dtype(np.int64): I64, np.dtype(np.uint8): U8, np.dtype(np.uint16): U16,
    np.dtype(np.uint32): U32, np.dtype(np.uint64): U64,
    np.dtype(np.float16): F16, np.dtype(np.float32): F32,
    np.dtype(np.float64): F64,
}


def type_code(dtype) -> int:
    return _NP_TO_TYPE[np.dtype(dtype)]


# ---- errors: one class per .NET exception kind the C# layer would throw ----
class HipAlgorithmsError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"{message} (status {status})")
        self.status = status


class ArgumentNullError(HipAlgorithmsError):
    """ArgumentNullException: a view is null or empty."""


class ArgumentOutOfRangeError(HipAlgorithmsError):
    """ArgumentOutOfRangeException: output or temp too short, bad length."""


class NotSupportedError(HipAlgorithmsError):
    """NotSupportedException: 64-bit lengths, strides, unknown type or functor."""


class InvalidOperationError(HipAlgorithmsError):
    """InvalidOperationException: unaligned temp allocation."""


class HipRuntimeError(HipAlgorithmsError):
    """A HIP runtime call failed inside the library."""


_ERRORS = {
    ERROR_NULL_VIEW: ArgumentNullError,
    ERROR_OUT_OF_RANGE: ArgumentOutOfRangeError,
    ERROR_NOT_SUPPORTED: NotSupportedError,
    ERROR_UNALIGNED_TEMP: InvalidOperationError,
    ERROR_RUNTIME: HipRuntimeError,
    ERROR_STATIC_LIMIT: NotSupportedError,
}

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """The loaded shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with "
                "`python -m ilgpu_amd.build` (there is no fallback path)")
        L = ctypes.CDLL(LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32
        p64 = ctypes.POINTER(ctypes.c_int64)
        L.ilgpu_hip_version.restype = i32
        L.ilgpu_hip_status_string.argtypes = [i32]
        L.ilgpu_hip_status_string.restype = ctypes.c_char_p
        L.ilgpu_hip_last_runtime_error.restype = i32
        L.ilgpu_hip_profile_enable.argtypes = [i32]
        L.ilgpu_hip_profile_enable.restype = i32
        L.ilgpu_hip_profile_query.argtypes = [
            ctypes.c_char_p, p64, ctypes.POINTER(ctypes.c_double)]
        L.ilgpu_hip_profile_query.restype = i32
        L.ilgpu_hip_radix_sort_temp_bytes.argtypes = [i64, i32, i32, p64]
        L.ilgpu_hip_radix_sort_temp_bytes_strided.argtypes = [
            i64, i32, i32, i64, i64, p64]
        L.ilgpu_hip_radix_sort_keys.argtypes = [vp, vp, i64, i64, i32, i32, vp, i64]
        L.ilgpu_hip_radix_sort_pairs.argtypes = [
            vp, vp, i64, vp, i64, i64, i32, i32, i32, i32, vp, i64]
        L.ilgpu_hip_radix_sort_passes.argtypes = [
            vp, vp, i64, i64, i32, i32, ctypes.POINTER(i32), ctypes.POINTER(i32)]
        L.ilgpu_hip_radix_sort_passes.restype = i32
        L.ilgpu_hip_selftest_lds_atomic_order.argtypes = [vp, i32, vp]
        L.ilgpu_hip_selftest_lds_atomic_order.restype = i32
        L.ilgpu_hip_sort_check_device.argtypes = [vp]
        L.ilgpu_hip_sort_check_device.restype = i32
        L.ilgpu_hip_sort_set_parameter.argtypes = [i32, i32]
        L.ilgpu_hip_sort_set_parameter.restype = i32
        L.ilgpu_hip_scan_temp_bytes.argtypes = [i64, i32, p64]
        L.ilgpu_hip_scan.argtypes = [vp, vp, i64, i64, vp, i64, i64, i32, i32,
                                     i32, vp, i64]
        L.ilgpu_hip_scan_static.argtypes = [vp, vp, i64, i64, vp, i64, i64, i32, i32, i32]
        L.ilgpu_hip_scan_static.restype = i32
        L.ilgpu_hip_reduce_temp_bytes.argtypes = [i64, i32, p64]
        L.ilgpu_hip_unique_temp_bytes.argtypes = [i64, i32, p64]
        L.ilgpu_hip_unique.argtypes = [vp, vp, i64, i32, vp, i64, vp, i64]
        L.ilgpu_hip_initialize.argtypes = [vp, vp, i64, i64, i32, vp]
        L.ilgpu_hip_sequence.argtypes = [vp, vp, i64, i64, i32, i64, i64]
        L.ilgpu_hip_reorder.argtypes = [vp, vp, i64, vp, i64, vp, i64, i32]
        L.ilgpu_hip_transform.argtypes = [vp, vp, i64, i64, i32, vp, i64, i64, i32, i32, i64]
        L.ilgpu_hip_reorder_transform.argtypes = [vp, vp, i64, i32, vp, i64, i32, vp, i64, i32, i64]
        L.ilgpu_hip_reduce.argtypes = [vp, vp, i64, i64, i32, i32, vp, i64, vp, i64]
        L.ilgpu_hip_histogram.argtypes = [vp, vp, i64, i64, i32, vp, i64, i32,
                                          i32, vp]
        for name in EXPORTS:
            if name.endswith(("_bytes", "_keys", "_pairs", "_scan", "_reduce",
                              "_histogram")):
                getattr(L, name).restype = i32
        _lib = L
    return _lib


def profile_enable(enabled: bool) -> None:
    """Switches per-kernel event timing on (clearing totals) or off."""
    check(lib().ilgpu_hip_profile_enable(1 if enabled else 0))


def profile_query(kernel_name: str):
    """(launches, total milliseconds) of the named kernel since enabling."""
    launches, total = ctypes.c_int64(0), ctypes.c_double(0.0)
    check(lib().ilgpu_hip_profile_query(kernel_name.encode(),
                                        ctypes.byref(launches),
                                        ctypes.byref(total)))
    return launches.value, total.value


def status_string(status: int) -> str:
    return lib().ilgpu_hip_status_string(status).decode()


def check(status: int) -> None:
    if status != SUCCESS:
        raise _ERRORS.get(status, HipAlgorithmsError)(status, status_string(status))


# ---- device memory (torch as the allocator) --------------------------------
class DeviceArray:
    """``length`` elements of ``dtype`` in device memory."""

    def __init__(self, length: int, dtype, *, _bytes=None):
        import torch
        self.dtype = np.dtype(dtype)
        self.length = int(length)
        nbytes = self.length * self.dtype.itemsize
        self.bytes = _bytes if _bytes is not None else torch.empty(
            max(nbytes, 1), dtype=torch.uint8, device="cuda:0")
        self.stride = 1  # element stride (Stride1D.General when above one)

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceArray":
        import torch
        a = np.ascontiguousarray(a)
        host = torch.from_numpy(a.view(np.uint8).reshape(-1))
        if host.numel() == 0:
            return cls(0, a.dtype)
        return cls(a.size, a.dtype, _bytes=host.to("cuda:0"))

    @classmethod
    def zeros(cls, length: int, dtype) -> "DeviceArray":
        out = cls(length, dtype)
        out.bytes.zero_()
        return out

    @property
    def ptr(self) -> int:
        return self.bytes.data_ptr() if self.length > 0 else 0

    @property
    def nbytes(self) -> int:
        return self.length * self.dtype.itemsize

    @property
    def type_code(self) -> int:
        return type_code(self.dtype)

    def numpy(self) -> np.ndarray:
        if self.length == 0:
            return np.empty(0, dtype=self.dtype)
        return self.bytes[: self.nbytes].cpu().numpy().view(self.dtype).copy()

    def clone(self) -> "DeviceArray":
        return DeviceArray(self.length, self.dtype, _bytes=self.bytes.clone())

    def strided(self, stride: int) -> "DeviceArray":
        """Every ``stride``-th element of this array as a view on the same
        memory (``AsGeneral(new Stride1D.General(stride))``): element i of the
        view is element ``i * stride`` of the array."""
        view = DeviceArray((self.length + stride - 1) // stride, self.dtype,
                           _bytes=self.bytes)
        view.stride = int(stride)
        return view

    def subview(self, offset: int, length: int) -> "DeviceArray":
        """Elements [offset, offset+length) as a view on the same memory."""
        s = self.dtype.itemsize
        return DeviceArray(length, self.dtype,
                           _bytes=self.bytes[offset * s:(offset + length) * s])


def temp_buffer(nbytes: int) -> DeviceArray:
    """An ``ArrayView<int>`` of at least ``nbytes`` bytes."""
    return DeviceArray((nbytes + 3) // 4, np.int32)


def _stream_ptr(stream) -> int:
    if stream is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    return getattr(stream, "cuda_stream", stream)


def _query(fn, *args) -> int:
    out = ctypes.c_int64(0)
    check(fn(*args, ctypes.byref(out)))
    return out.value


# ---- thin wrappers, one per entry point -------------------------------------
def radix_sort_temp_bytes(n: int, key_dtype, value_bytes: int = 0,
                          key_stride: int = 1, value_stride: int = 1) -> int:
    if key_stride != 1 or value_stride != 1:
        return _query(lib().ilgpu_hip_radix_sort_temp_bytes_strided, n,
                      type_code(key_dtype), value_bytes, key_stride,
                      value_stride)
    return _query(lib().ilgpu_hip_radix_sort_temp_bytes, n,
                  type_code(key_dtype), value_bytes)


def radix_sort_keys(keys: DeviceArray, temp: Optional[DeviceArray] = None, *,
                    descending: bool = False, float_total_order: bool = False,
                    stream=None, stride: Optional[int] = None) -> None:
    stride = keys.stride if stride is None else stride
    if temp is None:
        temp = temp_buffer(radix_sort_temp_bytes(keys.length, keys.dtype, 0,
                                                 stride))
    flags = (SORT_DESCENDING if descending else 0) | (
        SORT_FLOAT_TOTAL_ORDER if float_total_order else 0)
    check(lib().ilgpu_hip_radix_sort_keys(
        _stream_ptr(stream), keys.ptr, keys.length, stride, keys.type_code,
        flags, temp.ptr, temp.nbytes))


def radix_sort_pairs(keys: DeviceArray, values: DeviceArray,
                     temp: Optional[DeviceArray] = None, *,
                     descending: bool = False, float_total_order: bool = False,
                     values_from_index: bool = False, stream=None) -> None:
    """values_from_index: the values are generated, value[i] = (TValue)i, as the
    reference's sequencers do (integer value types: the index truncated; Half,
    float and double values: the index converted)."""
    if temp is None:
        temp = temp_buffer(radix_sort_temp_bytes(
            keys.length, keys.dtype, values.dtype.itemsize, keys.stride,
            values.stride))
    flags = (SORT_DESCENDING if descending else 0) | (
        SORT_FLOAT_TOTAL_ORDER if float_total_order else 0)
    if values.length != keys.length:
        # RadixSortExtensions.cs:1053-1054
        raise ArgumentOutOfRangeError(ERROR_OUT_OF_RANGE, "values")
    check(lib().ilgpu_hip_radix_sort_pairs(
        _stream_ptr(stream), keys.ptr, keys.stride, values.ptr, values.stride,
        keys.length,
        keys.type_code, values.dtype.itemsize, flags,
        VALUES_FROM_VIEW if not values_from_index
        else (VALUES_FROM_INDEX_AS_FLOAT if values.dtype.kind == "f" else VALUES_FROM_INDEX),
        temp.ptr, temp.nbytes))


def radix_sort_passes(temp: DeviceArray, n: int, key_dtype, value_bytes: int = 0, *,
                      stream=None):
    """(executed, skipped) 8-bit passes of the last sort that used `temp`."""
    executed, skipped = ctypes.c_int32(-1), ctypes.c_int32(-1)
    check(lib().ilgpu_hip_radix_sort_passes(
        _stream_ptr(stream), temp.ptr, temp.nbytes, n, type_code(key_dtype), value_bytes,
        ctypes.byref(executed), ctypes.byref(skipped)))
    return executed.value, skipped.value


def selftest_lds_atomic_order(rows: int = 256, *, stream=None) -> int:
    """Lanes of the LDS atomics found out of lane order (0 on gfx950)."""
    out = DeviceArray.zeros(1, np.int64)
    check(lib().ilgpu_hip_selftest_lds_atomic_order(_stream_ptr(stream), rows, out.ptr))
    return int(out.numpy()[0])


def sort_check_device(*, stream=None) -> None:
    """Asks the current device once whether its LDS serves the lanes of an atomic
    in lane order (what every sort does first); raises NotSupportedError for a
    device that does not."""
    check(lib().ilgpu_hip_sort_check_device(_stream_ptr(stream)))


SORT_PARAM_LOOKBACK_SPIN_LIMIT = 0
SORT_PARAM_LARGE_BLOCK_MIN_TILES_PER_CU = 1
SORT_PARAM_ONE_TILE_KERNEL = 2
SORT_PARAM_ASSUME_LDS_ATOMIC_ORDER = 3
SORT_PARAM_SHORT_TILE_MAX_TILES = 4


def sort_set_parameter(parameter: int, value: int) -> None:
    """Process-wide sort parameter; a negative value restores the default.
    LOOKBACK_SPIN_LIMIT: polls of an empty status word before a pass counts a
    missing tile itself (0 = at once: exercises the slow path).
    LARGE_BLOCK_MIN_TILES_PER_CU: 0 = always 1024-thread blocks, 2^31-1 = never.
    SHORT_TILE_MAX_TILES: keys of at most this many full tiles take short tiles
    (0 = never; at most the default, 512).
    ASSUME_LDS_ATOMIC_ORDER: 0 / 1 = every device counts as having failed / passed
    the check that precedes every sort; negative = ask the devices (anew)."""
    check(lib().ilgpu_hip_sort_set_parameter(parameter, value))


def set_sort_lookback_spin_limit(polls: int) -> None:
    sort_set_parameter(SORT_PARAM_LOOKBACK_SPIN_LIMIT, polls)


def scan_temp_bytes(n: int, dtype) -> int:
    return _query(lib().ilgpu_hip_scan_temp_bytes, n, type_code(dtype))


def scan(inp: DeviceArray, out: DeviceArray, temp: Optional[DeviceArray] = None,
         *, op: int = OP_ADD, kind: int = SCAN_INCLUSIVE, stream=None) -> None:
    if temp is None:
        temp = temp_buffer(scan_temp_bytes(max(inp.length, 1), inp.dtype))
    check(lib().ilgpu_hip_scan(
        _stream_ptr(stream), inp.ptr, inp.length, inp.stride, out.ptr,
        out.length, out.stride, inp.type_code, op, kind, temp.ptr, temp.nbytes))


def scan_static(inp: DeviceArray, out: DeviceArray, *, op: int = OP_ADD,
                kind: int = SCAN_INCLUSIVE, stream=None) -> None:
    """The scan on the library's static scratch: no temp, no allocation."""
    check(lib().ilgpu_hip_scan_static(
        _stream_ptr(stream), inp.ptr, inp.length, inp.stride, out.ptr,
        out.length, out.stride, inp.type_code, op, kind))


def reduce_temp_bytes(n: int, dtype) -> int:
    return _query(lib().ilgpu_hip_reduce_temp_bytes, n, type_code(dtype))


def reduce(inp: DeviceArray, out: DeviceArray,
           temp: Optional[DeviceArray] = None, *, op: int = OP_ADD,
           stream=None) -> None:
    if temp is None:
        temp = temp_buffer(reduce_temp_bytes(max(inp.length, 1), inp.dtype))
    check(lib().ilgpu_hip_reduce(
        _stream_ptr(stream), inp.ptr, inp.length, inp.stride, inp.type_code,
        op, out.ptr, out.length, temp.ptr, temp.nbytes))


def histogram(inp: DeviceArray, bins: DeviceArray,
              overflow: Optional[DeviceArray] = None, *,
              locator: int = LOCATOR_IDENTITY, stream=None) -> None:
    check(lib().ilgpu_hip_histogram(
        _stream_ptr(stream), inp.ptr, inp.length, inp.stride, inp.type_code,
        bins.ptr,
        bins.length, bins.type_code, locator,
        overflow.ptr if overflow is not None else None))


def unique_temp_bytes(n: int, dtype) -> int:
    return _query(lib().ilgpu_hip_unique_temp_bytes, n, type_code(dtype))


def unique(data: DeviceArray, new_length: DeviceArray,
           temp: Optional[DeviceArray] = None, *, stream=None) -> None:
    """Removes consecutive duplicates in place; new_length[0] (int64, on the
    device) receives the number of elements kept."""
    if temp is None:
        temp = temp_buffer(unique_temp_bytes(max(data.length, 1), data.dtype))
    check(lib().ilgpu_hip_unique(
        _stream_ptr(stream), data.ptr, data.length, data.type_code,
        new_length.ptr, new_length.length, temp.ptr, temp.nbytes))


def initialize(view: DeviceArray, value, *, stream=None) -> None:
    v = np.ascontiguousarray(np.asarray(value, dtype=view.dtype)).reshape(1)
    check(lib().ilgpu_hip_initialize(
        _stream_ptr(stream), view.ptr, view.length, view.stride,
        view.dtype.itemsize, v.ctypes.data_as(ctypes.c_void_p)))


def sequence(view: DeviceArray, *, sequence_length: Optional[int] = None,
             batch_length: int = 1, stream=None) -> None:
    """Sequence / RepeatedSequence / BatchedSequence / RepeatedBatchedSequence
    with the identity sequencer of the view's element type."""
    check(lib().ilgpu_hip_sequence(
        _stream_ptr(stream), view.ptr, view.length, view.stride, view.type_code,
        view.length if sequence_length is None else sequence_length,
        batch_length))


def reorder(source: DeviceArray, target: DeviceArray, order: DeviceArray, *,
            stream=None) -> None:
    check(lib().ilgpu_hip_reorder(
        _stream_ptr(stream), source.ptr, source.length, target.ptr,
        target.length, order.ptr, order.length, source.dtype.itemsize))


def transform(source: DeviceArray, target: DeviceArray,
              transformer: int = TRANSFORM_CONVERT, factor: int = 0, *,
              stream=None) -> None:
    """Transform: target[i] = (TTarget)op(source[i])."""
    check(lib().ilgpu_hip_transform(
        _stream_ptr(stream), source.ptr, source.length, source.stride,
        source.type_code, target.ptr, target.length, target.stride,
        target.type_code, transformer, factor))


def reorder_transform(source: DeviceArray, target: DeviceArray,
                      order: DeviceArray, transformer: int = TRANSFORM_CONVERT,
                      factor: int = 0, *, stream=None) -> None:
    """ReorderTransform: target[i] = (TTarget)op(source[order[i]])."""
    check(lib().ilgpu_hip_reorder_transform(
        _stream_ptr(stream), source.ptr, source.length, source.type_code,
        target.ptr, target.length, target.type_code, order.ptr, order.length,
        transformer, factor))
